"""RMS norm with the residual add folded in.

Reference: s = sum(x^2) / n; y_i = x_i * w_i / sqrt(s + eps), eps inside the root, the
gain multiplies directly (crates/bitnet-core/src/llama/model.rs:93-100).  The residual
sums of model.rs:292-294 and :304-306 are done by the norm that follows them: the
stream x is float32, `delta` (the previous part's output, float32) is added in place
and the normalised rows come back in the compute dtype.

Interface of a norm: forward(x, delta=None, rows=None) -> h
  x      float32 [T, E], the residual stream; updated in place when delta is given
  delta  float32 [T, E] or None; a norm that says `adds_terms` also takes [P, T, E], P terms
         to be added up in their order
  rows   int32 [R] or None: normalise only these rows (x is then left as it is)

A norm that says `folds_into_products` (with weight, eps and size as here) lets the product
before it and the product after it do its work when a step has few tokens: the first, which
adds to the stream, also leaves bf16(x * gain) and the sums of x^2 (`GainedRows`); the second
takes these as its tokens and multiplies its result by 1 / sqrt(mean(x^2) + eps).
"""
from __future__ import annotations

from typing import Dict, Optional

import torch

from .base import BuildEnv, Part, TensorSpec, register_norm
from .stream import GainedRows, ScaledSum, StreamsUpdate  # noqa: F401  (GainedRows: its old home; importers find it here too)


class RMSNorm(Part):
    """Parameters: size, eps, and two that a plain decoder leaves out: scalar (True: the gain is ONE number for all
    coordinates, a tensor without dimensions; it is spread over the width at load time, so that every kernel and every
    folding of the norm into products serves as it is), one_plus (True: the tensor holds the gain's distance from one, the
    norm multiplies by 1 + w; the sum is done once, in float32, at load time), names ({"weight": ...}: the tensor's name
    below the part's prefix; an empty name is the prefix itself).

    `add_normed` is the norm on a sublayer's OUTPUT: x <- x + norm(sa a + sb b), for layers whose sublayers read the stream
    itself; it also leaves the new rows in the compute dtype for the next sublayer."""
    graph_safe = True
    plan_safe = True
    folds_into_products = True
    adds_terms = True

    def __init__(self, params: Dict, env: BuildEnv):
        self.size = int(params["size"])
        self.eps = float(params["eps"])
        self.scalar = bool(params.get("scalar", False))
        self.one_plus = bool(params.get("one_plus", False))
        self.names = dict({"weight": "weight"}, **(params.get("names") or {}))
        self.env = env
        self.weight: Optional[torch.Tensor] = None

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        init = "zero_normal" if self.one_plus else "ones_normal"
        return {self.names["weight"]: TensorSpec(() if self.scalar else (self.size,), role="gain", init=init)}

    def load(self, tensors: Dict[str, torch.Tensor]) -> None:
        w = tensors[self.names["weight"]]
        self.weight = w.reshape(1).expand(self.size).contiguous() if self.scalar else w
        if self.one_plus:
            self.weight = (self.weight.to(torch.float32) + 1.0).contiguous()

    def add_normed(self, x: torch.Tensor, a: torch.Tensor, b: Optional[torch.Tensor] = None, sa: float = 1.0, sb: float = 1.0,
                   h_out: Optional[torch.Tensor] = None, assign: bool = False) -> None:
        """x [T, E] float32 <- (assign ? 0 : x) + norm(sa a + sb b); h_out (compute dtype) gets the new rows."""
        self.env.lib.outnorm_residual(x, a, b, sa, sb, self.weight, self.eps, assign, h_out)

    def forward(self, x: torch.Tensor, delta: Optional[torch.Tensor] = None,
                rows: Optional[torch.Tensor] = None, out_dtype: Optional[torch.dtype] = None) -> torch.Tensor:
        n = x.shape[0] if rows is None else rows.shape[0]
        out = torch.empty((n, self.size), dtype=out_dtype or self.env.dtype, device=x.device)
        self.env.lib.add_rmsnorm(x, delta, self.weight, self.eps, rows, out)
        return out


class LayerNorm(Part):
    """(x - mean) / sqrt(variance + eps) * weight + bias, the variance being the mean of the squared deviations;
    all of it in float32.  Parameters: size, eps, bias (True), names ({"weight": ..., "bias": ...}: the tensors'
    names below the part's prefix; an empty name is the prefix itself).  The stream may come in several copies
    [S, T, E]: the norm then reads sum_s coef[s] x[s] (`coef` None: the plain sum)."""
    graph_safe = True
    plan_safe = True
    adds_scaled_sum = True        # delta may be a ScaledSum: scale * (a + b), added in the norm's own pass

    def __init__(self, params: Dict, env: BuildEnv):
        self.size = int(params["size"])
        self.eps = float(params["eps"])
        self.has_bias = bool(params.get("bias", True))
        self.names = dict({"weight": "weight", "bias": "bias"}, **(params.get("names") or {}))
        self.env = env
        self.weight: Optional[torch.Tensor] = None
        self.bias: Optional[torch.Tensor] = None

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        out = {self.names["weight"]: TensorSpec((self.size,), role="gain", init="ones_normal")}
        if self.has_bias:
            out[self.names["bias"]] = TensorSpec((self.size,), role="gain", init="normal")
        return out

    def tensor_names(self, base: str) -> Dict[str, str]:
        """full name -> the part's own name, for an owner that stores the norm under `base`."""
        return {".".join(p for p in (base, name) if p): name for name in self.tensor_specs()}

    def load(self, tensors: Dict[str, torch.Tensor]) -> None:
        self.weight = tensors[self.names["weight"]]
        self.bias = tensors[self.names["bias"]] if self.has_bias else None

    def forward(self, x: torch.Tensor, delta: Optional[torch.Tensor] = None, rows: Optional[torch.Tensor] = None,
                coef: Optional[torch.Tensor] = None, out_dtype: Optional[torch.dtype] = None) -> torch.Tensor:
        t = x.shape[-2]
        n = t if rows is None else rows.shape[0]
        out = torch.empty((n, self.size), dtype=out_dtype or self.env.dtype, device=x.device)
        if isinstance(delta, ScaledSum):                  # a plain stream [T, E] and the residual sum that is still to be done
            a, b, scale = delta.parts()
            self.env.lib.layernorm_residual(x, a, b, scale, self.weight, self.bias, self.eps, rows, out)
            return out
        update = None
        if isinstance(delta, StreamsUpdate):              # an update of the copies still to be done
            if rows is None:
                update, delta = delta.parts(), None       # in this norm's own pass over the rows
            else:
                delta.apply(x)                            # only some rows are normalised: all are updated first
                delta = None
        self.env.lib.streams_layernorm(x, coef, self.weight, self.bias, self.eps, rows, out, delta=delta, update=update)
        return out


register_norm("rmsnorm", RMSNorm)
register_norm("layernorm", LayerNorm)
