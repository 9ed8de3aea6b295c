"""A short causal convolution over time, per channel: y_t = sum_d w[:, taps - 1 - d] * x_(t - d), d = 0 .. taps - 1,
with zeros before a sequence's start.  The last column of w [channels, taps] multiplies the current token.  No bias.

What a sequence carries from step to step are its last taps - 1 inputs (float32), kept in the cache's per-slot
state: a step of any number of tokens reads them for its first rows and leaves the new ones behind.  Used in front
of a mixer (y = x + conv(x), no activation) and inside one (y = silu(conv(x))).

Not a mixer or a norm: a helper that mixers and block arrangements own.  `tensor_spec()` is the weight's,
`cache_request(name)` the state's; `forward` runs on columns of a float32 matrix, so that several projections
packed into one product are convolved where they lie.
"""
from __future__ import annotations

from typing import Optional

import torch

from ..errors import ConfigError
from .base import BuildEnv, CacheRequest, TensorSpec

ACT_NONE, ACT_SILU = 0, 1
MAX_TAPS = 17


class ShortConv:
    def __init__(self, channels: int, taps: int, env: BuildEnv, residual: bool = False, act: int = ACT_NONE):
        self.channels, self.taps, self.env = int(channels), int(taps), env
        if not 1 <= self.taps <= MAX_TAPS:
            raise ConfigError(f"short convolution: {self.taps} taps not supported (1 to {MAX_TAPS})")
        self.residual, self.act = bool(residual), int(act)
        self.weight: Optional[torch.Tensor] = None

    def tensor_spec(self) -> TensorSpec:
        return TensorSpec((self.channels, self.taps), role="gain", init="normal")

    def cache_request(self, name: str) -> Optional[CacheRequest]:
        if self.taps == 1:
            return None
        return CacheRequest("state", state_shape=(self.taps - 1, self.channels), state_init=0.0, name=name)

    def load(self, weight: torch.Tensor) -> None:
        self.weight = weight.contiguous()

    def forward(self, x: torch.Tensor, ctx, state: Optional[torch.Tensor], out_dtype: torch.dtype, col0: int = 0,
                bias: Optional[torch.Tensor] = None) -> torch.Tensor:
        """x [T, W] float32; columns col0 .. col0 + channels go through the convolution -> [T, channels]; the
        state then moves on by the step's rows.  bias (float32 [channels]): added to the inputs first; the state then holds
        the inputs with it."""
        lib = self.env.lib
        out = torch.empty((x.shape[0], self.channels), dtype=out_dtype, device=x.device)
        if bias is not None:
            lib.short_conv_bias(x, col0, self.channels, bias, self.weight, state, ctx, out, self.residual, self.act)
        else:
            lib.short_conv(x, col0, self.channels, self.weight, state, ctx, out, self.residual, self.act)
        return out
