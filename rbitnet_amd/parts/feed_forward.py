"""The SiLU-gated feed-forward.

Reference (crates/bitnet-core/src/llama/model.rs:296-306): g = silu(Wgate h) with
silu(v) = v / (1 + exp(-v)) (:116-120), u = Wup h, out = Wdown (g * u).  No biases.
Gate and up share one product; on the matrix cores the gate is applied in that
product's epilogue, on the generic path by a small kernel on its float32 result.

Parameters: intermediate_size, activation ("silu"), names.
Interface of a feed-forward: tensor_specs() / load(tensors) / forward(h [T, E], ctx) ->
float32 [T, E].  It may say `takes_gained_rows` and `adds_to_stream` of itself as a mixer
may (this one does both).
"""
from __future__ import annotations

from typing import Dict, Optional

import torch

from ..errors import ConfigError
from .base import BuildEnv, Part, TensorSpec, register_feed_forward
from .linear import can_fuse_gate, gated_linear, linear, linear_to_stream, pack_gate_up, pack_rows, xielu_linear

DEFAULT_NAMES = {"gate": "gate_proj.weight", "up": "up_proj.weight", "down": "down_proj.weight"}


class SwiGLU(Part):
    graph_safe = True
    plan_safe = True
    takes_gained_rows = True
    adds_to_stream = True

    def __init__(self, params: Dict, env: BuildEnv):
        self.env = env
        self.ff = int(params["intermediate_size"])
        if params.get("activation", "silu") != "silu":
            raise ConfigError(f"feed-forward activation {params.get('activation')!r} not supported (silu)")
        self.names = dict(DEFAULT_NAMES, **(params.get("names") or {}))
        self.hidden = env.hidden_size
        self.fused = can_fuse_gate(env.dtype, self.hidden, self.ff) and not getattr(env, "generic_only", False)
        self.w_gate_up: Optional[torch.Tensor] = None
        self.w_down: Optional[torch.Tensor] = None

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        return {self.names["gate"]: TensorSpec((self.ff, self.hidden)),
                self.names["up"]: TensorSpec((self.ff, self.hidden)),
                self.names["down"]: TensorSpec((self.hidden, self.ff))}

    def load(self, tensors: Dict[str, torch.Tensor]) -> None:
        allowed = not getattr(self.env, "generic_only", False)
        self.w_gate_up = pack_gate_up(self.env.lib, tensors[self.names["gate"]], tensors[self.names["up"]], self.fused,
                                      allowed)
        down = tensors[self.names["down"]]
        self.w_down = pack_rows(self.env.lib, [(down, 0, None, None)], down.shape[0], down.shape[1], down.dtype,
                                down.device, allowed)

    def forward(self, h, ctx=None, stream: Optional[torch.Tensor] = None, next_norm=None):
        lib = self.env.lib
        t = gated_linear(lib, h, self.w_gate_up, self.ff, self.fused)
        return linear_to_stream(lib, t, self.w_down, stream, next_norm)


class DenseAct(Part):
    """out = Wdown act(Wup h), the activation applied where the first product stores its float32 sums.
    activation "xielu": for z > 0, softplus(p) z^2 + z / 2; for z <= 0, (1/2 + softplus(q)) (exp(z) - 1 - z) + z / 2,
    (p, q) being the two numbers of the tensor `act`.  activation "gelu_tanh": z / 2 (1 + tanh(sqrt(2 / pi) (z + 0.044715 z^3))),
    no tensor.  Parameters: intermediate_size, activation, names ({"up", "down", "act"})."""
    graph_safe = True
    plan_safe = True
    adds_to_stream = True
    activation = "xielu"

    def __init__(self, params: Dict, env: BuildEnv):
        self.env = env
        self.ff = int(params["intermediate_size"])
        self.activation = str(params.get("activation", type(self).activation))
        if self.activation not in ("xielu", "gelu_tanh"):
            raise ConfigError(f"dense feed-forward: activation {self.activation!r} not supported (xielu, gelu_tanh)")
        self.names = dict({"up": "up", "down": "down", "act": "act"}, **(params.get("names") or {}))
        self.hidden = env.hidden_size

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        out = {self.names["up"]: TensorSpec((self.ff, self.hidden)), self.names["down"]: TensorSpec((self.hidden, self.ff))}
        if self.activation == "xielu":
            out[self.names["act"]] = TensorSpec((2,), role="gain", init="normal")
        return out

    def load(self, tensors: Dict[str, torch.Tensor]) -> None:
        allowed = not getattr(self.env, "generic_only", False)
        up, down = tensors[self.names["up"]], tensors[self.names["down"]]
        self.w_up = pack_rows(self.env.lib, [(up, 0, None, None)], up.shape[0], up.shape[1], up.dtype, up.device, allowed)
        self.w_down = pack_rows(self.env.lib, [(down, 0, None, None)], down.shape[0], down.shape[1], down.dtype,
                                down.device, allowed)
        if self.activation == "xielu":
            self.act = tensors[self.names["act"]]
        else:       # the kernels read a first number that is no number as "the tanh form of GELU"
            self.act = torch.tensor([float("nan"), 0.0], dtype=torch.float32, device=up.device)

    def forward(self, h, ctx=None, stream: Optional[torch.Tensor] = None, next_norm=None):
        lib = self.env.lib
        t = xielu_linear(lib, h, self.w_up, self.act, self.env.dtype)      # the activation in the product's epilogue
        return linear_to_stream(lib, t, self.w_down, stream, next_norm)


class DenseXielu(DenseAct):
    activation = "xielu"


class DenseGelu(DenseAct):
    activation = "gelu_tanh"


class ClampedGLU(Part):
    """A gated feed-forward with limits on both branches:
        g = min(Wgate h, limit),  u = clamp(Wup h, -limit, limit);  out = Wdown (g * sigmoid(alpha * g) * (u + 1))
    (the unit of the routed experts, as a dense layer).  Gate and up are one product; on the matrix cores limits and gate
    are applied in that product's epilogue (gate and up rows interleaved, as for the SiLU gate), elsewhere by a kernel on
    its float32 sums.
    Parameters: intermediate_size, limit (None or <= 0: no limits), alpha (1.702), names ({"gate", "up", "down"})."""
    graph_safe = True
    plan_safe = True

    def __init__(self, params: Dict, env: BuildEnv):
        self.env = env
        self.ff = int(params["intermediate_size"])
        self.limit = float(params.get("limit") or 0.0)
        self.alpha = float(params.get("alpha", 1.702))
        self.names = dict({"gate": "gate", "up": "up", "down": "down"}, **(params.get("names") or {}))
        self.hidden = env.hidden_size
        self.fused = self.limit > 0 and can_fuse_gate(env.dtype, self.hidden, self.ff) and not getattr(env, "generic_only", False)

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        return {self.names["gate"]: TensorSpec((self.ff, self.hidden)), self.names["up"]: TensorSpec((self.ff, self.hidden)),
                self.names["down"]: TensorSpec((self.hidden, self.ff))}

    def load(self, tensors: Dict[str, torch.Tensor]) -> None:
        allowed = not getattr(self.env, "generic_only", False)
        self.w_gate_up = pack_gate_up(self.env.lib, tensors[self.names["gate"]], tensors[self.names["up"]], self.fused, allowed)
        self.gate_numbers = torch.tensor([self.limit, self.alpha], dtype=torch.float32, device=tensors[self.names["gate"]].device)
        down = tensors[self.names["down"]]
        self.w_down = pack_rows(self.env.lib, [(down, 0, None, None)], down.shape[0], down.shape[1], down.dtype, down.device,
                                allowed)

    def forward(self, h, ctx=None, stream: Optional[torch.Tensor] = None, next_norm=None):
        lib = self.env.lib
        if self.fused:
            t = gated_linear(lib, h, self.w_gate_up, self.ff, True, gate=self.gate_numbers)
        else:
            gu = linear(lib, h, self.w_gate_up, torch.float32)
            t = torch.empty((h.shape[0], self.ff), dtype=self.env.dtype, device=gu.device)
            lib.clamped_glu(gu, t, self.limit, self.alpha)
        return linear(lib, t, self.w_down, torch.float32)


register_feed_forward("swiglu", SwiGLU)
register_feed_forward("clamped_glu", ClampedGLU)
register_feed_forward("dense_xielu", DenseXielu)
register_feed_forward("dense_gelu", DenseGelu)
register_feed_forward("dense_act", DenseAct)
