"""How the parts of one layer are arranged.

"prenorm" (crates/bitnet-core/src/llama/model.rs:236-307):
    x += mixer(norm1(x));  x += feed_forward(norm2(x))
The residual stream x is float32 and each sum is done by the norm that follows it (see
norm.py), so a block takes the previous block's not yet added output as `pending` and
returns its own.  The model adds the last one in the final norm.

Who adds what to the stream, and in which form a part's output travels to the next norm, is
`stream.py`'s business: an arrangement calls `sublayer(part, norm, x, pending, next_norm, ...)`
once per part and hands on what comes back.

"prenorm" takes two things that a plain decoder leaves out: a layer without a feed-forward (and second norm), and a
token shift in front of the mixer (block parameter `token_shift`: {"name": tensor}): what the mixer reads is
    h_t + (h_(t-1) - h_t) * s      per channel, s the tensor [E], h_(t-1) the normalised row of the token before (zeros
                                   before a sequence's first token)
in float32; the last normalised row of a sequence is part of its state in the cache (`view.states["token_shift"]`).
It is a causal convolution of two taps (-s on the row itself, s on the one before, added to the row), and runs as one.

Interface of a block: parts() -> {name: part} for the loader (names are tensor-name
segments below the layer's prefix); mixer (for the cache request);
forward(x, pending, ctx, view) -> pending (a tensor still to be added, None, or GainedRows).
A block may offer first_norm (the norm its forward begins with) and say takes_next_norm:
forward then also takes next_norm, the first norm of whatever runs after it.
"""
from __future__ import annotations

from typing import Dict

import torch

from .base import BuildEnv, Part, TensorSpec, build_part, register_block
from ..errors import ConfigError
from .short_conv import ACT_NONE, ShortConv
from .stream import GainedRows, ScaledSum, StreamCopy, WeightedTerms, normed_for, sublayer  # noqa: F401  (normed_for: its old home)

DEFAULT_SEGMENTS = {"norm1": "input_layernorm", "mixer": "self_attn", "norm2": "post_attention_layernorm",
                    "feed_forward": "mlp"}


class _ShiftTensor(Part):
    """The layer's own tensor of a token shift, loaded under the layer's prefix."""

    def __init__(self, block: "PreNormBlock"):
        self.block = block

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        return {self.block.shift_name: TensorSpec((self.block.hidden,), role="gain", init="normal")}

    def load(self, tensors: Dict[str, torch.Tensor]) -> None:
        s = tensors[self.block.shift_name].to(torch.float32)
        self.block.shift.load(torch.stack([s, -s], dim=1))      # taps: the row before, the row itself


class PreNormBlock:
    takes_next_norm = True

    def __init__(self, layer_spec, env: BuildEnv):
        params = dict(getattr(layer_spec, "params", None) or {})
        self.env, self.hidden = env, env.hidden_size
        self.norm1 = build_part("norm", layer_spec.norm1, env)
        self.mixer = build_part("mixer", layer_spec.mixer, env)
        self.norm2 = self.feed_forward = None
        if layer_spec.feed_forward is not None:
            self.norm2 = build_part("norm", layer_spec.norm2, env)
            self.feed_forward = build_part("feed_forward", layer_spec.feed_forward, env)
        self.segments = dict(DEFAULT_SEGMENTS, **(getattr(layer_spec, "segments", None) or {}))
        shift = params.get("token_shift")
        self.shift = ShortConv(self.hidden, 2, env, residual=True, act=ACT_NONE) if shift else None
        self.shift_name = str(shift.get("name", "shift")) if shift else None
        if self.shift is not None and "out_dtype" not in self.norm1.forward.__code__.co_varnames:
            raise ConfigError("a token shift needs a norm that can leave float32 rows (rmsnorm, layernorm)")

    def _all(self):
        return [p for p in (self.norm1, self.mixer, self.norm2, self.feed_forward) if p is not None]

    @property
    def graph_safe(self) -> bool:
        return all(getattr(p, "graph_safe", False) for p in self._all())

    @property
    def plan_safe(self) -> bool:
        return all(getattr(p, "plan_safe", False) for p in self._all())

    def parts(self) -> Dict[str, object]:
        out = {self.segments["norm1"]: self.norm1, self.segments["mixer"]: self.mixer}
        if self.feed_forward is not None:
            out[self.segments["norm2"]] = self.norm2
            out[self.segments["feed_forward"]] = self.feed_forward
        if self.shift is not None:
            out[""] = _ShiftTensor(self)
        return out

    def cache_requests(self):
        many = getattr(self.mixer, "cache_requests", None)
        one = getattr(self.mixer, "cache_request", None)
        out = list(many()) if many else ([one()] if one and one() is not None else [])
        if self.shift is not None:
            out.append(self.shift.cache_request("token_shift"))
        return out

    @property
    def first_norm(self):
        return self.norm1

    def _mixer(self, x: torch.Tensor, pending, after, ctx, view):
        if self.shift is None:
            return sublayer(self.mixer, self.norm1, x, pending, after, ctx, view)
        # the normalised rows in float32, then the shift towards the row before, rounded once on the way out
        delta = None if isinstance(pending, GainedRows) else pending          # such rows mean that the stream holds the sum
        hn = self.norm1.forward(x, delta, None, out_dtype=torch.float32)
        h = self.shift.forward(hn, ctx, view.states["token_shift"], self.env.dtype)
        if getattr(self.mixer, "adds_to_stream", False):
            return self.mixer.forward(h, ctx, view, stream=x, next_norm=after)
        return self.mixer.forward(h, ctx, view)

    def forward(self, x: torch.Tensor, pending, ctx, view, next_norm=None):
        if self.feed_forward is None:
            return self._mixer(x, pending, next_norm, ctx, view)
        a = self._mixer(x, pending, self.norm2, ctx, view)
        return sublayer(self.feed_forward, self.norm2, x, a, next_norm, ctx)


class ParallelBlock:
    """"parallel": one norm that both sublayers read, and a factor m on their sum:
        h = norm1(x);  x += m * (mixer(h) + feed_forward(h))
    The feed-forward may be left out.  The sum is left to the norm that reads the stream next (`ScaledSum`), which adds
    it in its own pass over the rows; that norm must say `adds_scaled_sum` (layer norm does).
    Block parameters (`LayerSpec.params`): residual_scale (m, 1.0)."""
    takes_next_norm = True

    def __init__(self, layer_spec, env: BuildEnv):
        params = dict(getattr(layer_spec, "params", None) or {})
        self.scale = float(params.get("residual_scale", 1.0))
        self.norm1 = build_part("norm", layer_spec.norm1, env)
        self.mixer = build_part("mixer", layer_spec.mixer, env)
        self.feed_forward = None if layer_spec.feed_forward is None else build_part("feed_forward", layer_spec.feed_forward, env)
        self.segments = dict({"norm1": "norm1", "mixer": "mix", "feed_forward": "mlp"}, **(getattr(layer_spec, "segments", None) or {}))
        if not getattr(self.norm1, "adds_scaled_sum", False):
            raise ConfigError("a parallel layer needs a norm that adds a scaled sum in its own pass (layernorm)")

    def _all(self):
        return [p for p in (self.norm1, self.mixer, self.feed_forward) if p is not None]

    @property
    def graph_safe(self) -> bool:
        return all(getattr(p, "graph_safe", False) for p in self._all())

    @property
    def plan_safe(self) -> bool:
        return all(getattr(p, "plan_safe", False) for p in self._all())

    def parts(self) -> Dict[str, object]:
        out = {self.segments["norm1"]: self.norm1, self.segments["mixer"]: self.mixer}
        if self.feed_forward is not None:
            out[self.segments["feed_forward"]] = self.feed_forward
        return out

    def cache_requests(self):
        many = getattr(self.mixer, "cache_requests", None)
        one = getattr(self.mixer, "cache_request", None)
        return list(many()) if many else ([one()] if one and one() is not None else [])

    @property
    def first_norm(self):
        return self.norm1

    def forward(self, x: torch.Tensor, pending, ctx, view, next_norm=None):
        if next_norm is not None and not getattr(next_norm, "adds_scaled_sum", False):
            raise ConfigError("what follows a parallel layer must begin with a norm that adds a scaled sum (layernorm)")
        h = self.norm1.forward(x, pending, None)
        a = self.mixer.forward(h, ctx, view)
        b = self.feed_forward.forward(h, ctx) if self.feed_forward is not None else None
        return ScaledSum(a, b, self.scale)


class OutNormBlock:
    """"outnorm": the norms stand on the sublayers' outputs, and the sublayers read the stream itself:
        x += norm1(mixer(x));  x += norm2(feed_forward(x))
    The feed-forward (and norm2) may be left out.  The norms must offer `add_normed` (rmsnorm does): one kernel norms the
    sublayer's output, adds it to the float32 stream and leaves the new rows in the compute dtype, which is what the next
    sublayer, or the next such block, reads (`StreamCopy`).  A mixer that hands back `WeightedTerms` has them added up in
    the same pass."""
    takes_stream_copy = True
    takes_next_norm = True

    def __init__(self, layer_spec, env: BuildEnv):
        self.env, self.hidden = env, env.hidden_size
        self.norm1 = build_part("norm", layer_spec.norm1, env)
        self.mixer = build_part("mixer", layer_spec.mixer, env)
        self.norm2 = self.feed_forward = None
        if layer_spec.feed_forward is not None:
            self.norm2 = build_part("norm", layer_spec.norm2, env)
            self.feed_forward = build_part("feed_forward", layer_spec.feed_forward, env)
        self.segments = dict({"norm1": "norm1", "mixer": "mix", "norm2": "norm2", "feed_forward": "mlp"},
                             **(getattr(layer_spec, "segments", None) or {}))
        for norm in (self.norm1, self.norm2):
            if norm is not None and not hasattr(norm, "add_normed"):
                raise ConfigError("a layer with norms on its sublayers' outputs needs norms that can stand there (rmsnorm)")

    def _all(self):
        return [p for p in (self.norm1, self.mixer, self.norm2, self.feed_forward) if p is not None]

    @property
    def graph_safe(self) -> bool:
        return all(getattr(p, "graph_safe", False) for p in self._all())

    @property
    def plan_safe(self) -> bool:
        return all(getattr(p, "plan_safe", False) for p in self._all())

    def parts(self) -> Dict[str, object]:
        out = {self.segments["norm1"]: self.norm1, self.segments["mixer"]: self.mixer}
        if self.feed_forward is not None:
            out[self.segments["norm2"]] = self.norm2
            out[self.segments["feed_forward"]] = self.feed_forward
        return out

    def cache_requests(self):
        many = getattr(self.mixer, "cache_requests", None)
        one = getattr(self.mixer, "cache_request", None)
        return list(many()) if many else ([one()] if one and one() is not None else [])

    def _rows(self, x: torch.Tensor) -> torch.Tensor:
        return x if self.env.dtype == torch.float32 else torch.empty(x.shape, dtype=self.env.dtype, device=x.device)

    def _add(self, norm, x: torch.Tensor, y) -> torch.Tensor:
        """x += norm(y); returns the new rows in the compute dtype."""
        h = self._rows(x)
        out = None if h is x else h
        if isinstance(y, WeightedTerms):
            norm.add_normed(x, y.a, y.b, y.sa, y.sb, h_out=out)
        else:
            norm.add_normed(x, y, h_out=out)
        return h

    def forward(self, x: torch.Tensor, pending, ctx, view, next_norm=None):
        if isinstance(pending, StreamCopy):
            h = pending.h
        else:
            if pending is not None:
                raise ConfigError("a layer with norms on its sublayers' outputs follows one that leaves the stream complete")
            h = self._rows(x)
            if h is not x:
                self.env.lib.place_rows(x, h)
        if getattr(self.mixer, "weighted_terms_ok", False):
            y = self.mixer.forward(h, ctx, view, weighted_terms=True)
        else:
            y = self.mixer.forward(h, ctx, view)
        h = self._add(self.norm1, x, y)
        if self.feed_forward is not None:
            h = self._add(self.norm2, x, self.feed_forward.forward(h, ctx))
        return StreamCopy(h)


register_block("prenorm", PreNormBlock)
register_block("outnorm", OutNormBlock)
register_block("parallel", ParallelBlock)
