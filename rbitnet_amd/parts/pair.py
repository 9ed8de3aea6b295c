"""Two mixers side by side: both read the same input, each output is RMS-normed over the model width with a plain weight
of its own, and the result is the mean of the two:
    out = (a / sqrt(mean a^2 + eps) * w_left + b / sqrt(mean b^2 + eps) * w_right) / 2,   a = left(h), b = right(h)
Norms and the mean in float32, one kernel.

The two are ordinary mixers from the registry (say, windowed attention beside a recurrent one); their tensors lie under
the segments `left` and `right` below the pair's own prefix, the two norm weights beside them.  Each keeps what it needs
of the cache: the pair hands on all their requests, which therefore need different names or kinds (one "kv" request
and any number of named states can share a layer).

With `combine = "weighted"` there are no norms and no weights of the pair's own: the result is
    out = left_scale * a + right_scale * b
which the pair hands, as `WeightedTerms`, to a block that asks for them (the norm on the sublayer's output adds them up in its
own pass over the rows).

Parameters: left, right (each {"kind", "params"}), eps, names ({"left_out", "right_out"}), segments ({"left", "right"}),
combine ("norm_mean"; "weighted" with left_scale and right_scale).
"""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from ..errors import ConfigError
from .base import BuildEnv, CacheRequest, Part, TensorSpec, _REGISTRIES, register_mixer
from .stream import WeightedTerms

DEFAULT_NAMES = {"left_out": "left.out", "right_out": "right.out"}
DEFAULT_SEGMENTS = {"left": "left", "right": "right"}


def _build(spec, env: BuildEnv):
    kind, params = (spec.kind, spec.params) if hasattr(spec, "kind") else (spec["kind"], spec.get("params") or {})
    table = _REGISTRIES["mixer"]
    if kind not in table:
        raise ConfigError(f"unknown mixer kind {kind!r}; registered: {', '.join(sorted(table))}")
    return table[kind](params, env)


class MixerPair(Part):
    def __init__(self, params: Dict, env: BuildEnv):
        self.env = env
        self.combine = str(params.get("combine", "norm_mean"))
        if self.combine not in ("norm_mean", "weighted"):
            raise ConfigError(f"a pair of mixers: unknown way to combine {self.combine!r} (norm_mean, weighted)")
        self.weighted_terms_ok = self.combine == "weighted"
        self.eps = float(params.get("eps", 0.0))
        self.scales = (float(params.get("left_scale", 1.0)), float(params.get("right_scale", 1.0)))
        self.names = dict(DEFAULT_NAMES, **(params.get("names") or {}))
        self.segments = dict(DEFAULT_SEGMENTS, **(params.get("segments") or {}))
        self.left, self.right = _build(params["left"], env), _build(params["right"], env)
        self.hidden = env.hidden_size
        # what the model asks a mixer about the cache it reads from another layer: the left one's, if any
        self.cache_from = getattr(self.left, "cache_from", None)
        self.window = getattr(self.left, "window", None)
        if getattr(self.right, "cache_from", None) is not None:
            raise ConfigError("a pair of mixers: only the left one may read another layer's cache")

    @property
    def graph_safe(self) -> bool:
        return bool(getattr(self.left, "graph_safe", False) and getattr(self.right, "graph_safe", False))

    @property
    def plan_safe(self) -> bool:
        return bool(getattr(self.left, "plan_safe", False) and getattr(self.right, "plan_safe", False))

    def _sub(self):
        return ((self.segments["left"], self.left), (self.segments["right"], self.right))

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        out = {}
        for segment, part in self._sub():
            for name, ts in part.tensor_specs().items():
                out[f"{segment}.{name}"] = ts
        if self.combine == "norm_mean":
            for key in ("left_out", "right_out"):
                out[self.names[key]] = TensorSpec((self.hidden,), role="gain", init="ones_normal")
        return out

    def load(self, tensors: Dict[str, torch.Tensor]) -> None:
        for segment, part in self._sub():
            part.load({name: tensors[f"{segment}.{name}"] for name in part.tensor_specs()})
        if self.combine == "norm_mean":
            self.w_left, self.w_right = tensors[self.names["left_out"]], tensors[self.names["right_out"]]

    def cache_requests(self) -> List[CacheRequest]:
        out: List[CacheRequest] = []
        for _, part in self._sub():
            many = getattr(part, "cache_requests", None)
            one = getattr(part, "cache_request", None)
            out.extend(many() if many else ([one()] if one and one() is not None else []))
        if sum(1 for r in out if r.kind == "kv") > 1:
            raise ConfigError("a pair of mixers can keep one set of keys and values a layer")
        return out

    def cache_request(self) -> Optional[CacheRequest]:
        reqs = self.cache_requests()
        return reqs[0] if reqs else None

    def forward(self, h: torch.Tensor, ctx, view, stream: Optional[torch.Tensor] = None, next_norm=None,
                weighted_terms: bool = False):
        a = self.left.forward(h, ctx, view)
        b = self.right.forward(h, ctx, view)
        if self.combine == "weighted":
            if not weighted_terms:
                raise ConfigError("a pair of mixers combined as a weighted sum needs a block that adds up its two terms (outnorm)")
            return WeightedTerms(a, self.scales[0], b, self.scales[1])
        out = torch.empty((h.shape[0], self.hidden), dtype=torch.float32, device=h.device)
        self.env.lib.pair_norm_mean(a, self.w_left, b, self.w_right, self.eps, out)
        return out


register_mixer("pair", MixerPair)
