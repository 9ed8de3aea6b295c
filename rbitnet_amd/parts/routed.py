"""A feed-forward of many small experts of which every token uses a few.

    z = W_router h (float32);  s = sigmoid(z);  the `top` experts with the largest s are chosen (lowest index among equals)
    out = sum over the chosen e of expert_e(s_e * h): the score multiplies the expert's INPUT and is not renormalised
    expert(x):  g = min(Wg x, limit),  u = clamp(Wu x, -limit, limit),  Wd (g * sigmoid(alpha * g) * (u + 1))

Nothing of a step goes through the host: the router's product, one launch that chooses and sorts the (token, expert)
pairs by expert in runs padded to tiles of 16 rows, one launch pair for all experts' products (on the matrix cores in
bfloat16), and, with more than one expert a token, the sum of a token's pairs in a fixed order.  A token's result does
not depend on what else the step holds.

Experts' tensors are `e<i>.gate`, `e<i>.up` [ff, E] and `e<i>.down` [E, ff]; they are stacked at load time.
Parameters: experts, top, intermediate_size, limit, alpha (1.702), names ({"router", "expert", "gate", "up", "down"}).

A second family of routers is served by the same launches, each choice a parameter of its own:
    score        "sigmoid" (above), or "softmax": s = softmax(z) over all of the router's outputs
    correction   True: the choice goes by s + the tensor "correction" (one number per output), the weights by s alone
    identity     n: the router has n more outputs behind the experts; one that is chosen gives the token's input itself
                 (times its weight) and has no tensors
    weight_on    "input" (above), or "output": out = sum over the chosen of s_e * expert_e(h)
    limit        None: no clamps, and the plain gate: expert(x) = Wd (silu(Wg x) * (Wu x))
    shared       None, or {"intermediate_size": f}: an expert of the plain gated form (tensors "shared.gate", "shared.up",
                 "shared.down") that every token uses, added times sigmoid(w . h), w the tensor "shared.sg" [1, E]
The weights of the chosen are never renormalised.  Router logits, scores, the choice and all sums are float32.
"""
from __future__ import annotations

from typing import Dict, Optional

import torch

from ..errors import ConfigError
from .base import BuildEnv, Part, TensorSpec, register_feed_forward
from .feed_forward import SwiGLU
from .linear import linear, pack_rows

DEFAULT_NAMES = {"router": "router", "expert": "e{i}", "gate": "gate", "up": "up", "down": "down", "correction": "correction",
                 "shared": "shared", "shared_gate": "shared.sg"}
MAX_EXPERTS = 1024


class RoutedExperts(Part):
    graph_safe = True
    plan_safe = True

    def __init__(self, params: Dict, env: BuildEnv):
        self.env = env
        self.n_experts, self.top = int(params["experts"]), int(params["top"])
        self.ff = int(params["intermediate_size"])
        self.limit = None if params.get("limit") is None else float(params["limit"])
        self.alpha = float(params.get("alpha", 1.702))
        self.identity = int(params.get("identity") or 0)
        self.n_outputs = self.n_experts + self.identity
        if self.identity < 0 or not 0 < self.top <= self.n_outputs <= MAX_EXPERTS or self.n_experts <= 0:
            raise ConfigError(f"routed experts: top {self.top} of {self.n_experts} experts and {self.identity} outputs behind them "
                              f"not supported (at most {MAX_EXPERTS} outputs)")
        if self.ff <= 0 or (self.limit is not None and not self.limit > 0):
            raise ConfigError("routed experts: sizes and the limit must be positive")
        self.score = {"sigmoid": 0, "softmax": 1}.get(str(params.get("score", "sigmoid")))
        if self.score is None:
            raise ConfigError(f"routed experts: score {params.get('score')!r} not supported (sigmoid, softmax)")
        self.has_correction = bool(params.get("correction"))
        if self.has_correction and self.score != 1:
            raise ConfigError("routed experts: a correction of the choice goes with the softmax")
        self.weight_on = str(params.get("weight_on", "input"))
        if self.weight_on not in ("input", "output"):
            raise ConfigError(f"routed experts: weight_on {self.weight_on!r} not supported (input, output)")
        if self.identity and self.weight_on != "output":
            raise ConfigError("routed experts: outputs behind the experts go with weights on the experts' outputs")
        self.names = dict(DEFAULT_NAMES, **(params.get("names") or {}))
        self.hidden = env.hidden_size
        shared = params.get("shared")
        self.shared = None
        if shared is not None:
            if self.weight_on != "output":
                raise ConfigError("routed experts: a shared expert goes with weights on the experts' outputs")
            base = self.names["shared"]
            self.shared = SwiGLU({"intermediate_size": int(shared["intermediate_size"]),
                                  "names": {"gate": f"{base}.gate", "up": f"{base}.up", "down": f"{base}.down"}}, env)
        self.plain = self.score == 0 and self.weight_on == "input" and not self.identity and self.shared is None

    def _name(self, i: int, what: str) -> str:
        return f"{self.names['expert'].format(i=i)}.{self.names[what]}"

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        out = {self.names["router"]: TensorSpec((self.n_outputs, self.hidden))}
        if self.has_correction:
            out[self.names["correction"]] = TensorSpec((self.n_outputs,), role="gain", init="normal")
        if self.shared is not None:
            out.update(self.shared.tensor_specs())
            out[self.names["shared_gate"]] = TensorSpec((1, self.hidden))
        for i in range(self.n_experts):
            out[self._name(i, "gate")] = TensorSpec((self.ff, self.hidden))
            out[self._name(i, "up")] = TensorSpec((self.ff, self.hidden))
            out[self._name(i, "down")] = TensorSpec((self.hidden, self.ff))
        return out

    def load(self, tensors: Dict[str, torch.Tensor]) -> None:
        lib, allowed = self.env.lib, not getattr(self.env, "generic_only", False)
        r = tensors[self.names["router"]]
        pieces = [(r, 0, None, None)]
        if self.shared is not None:          # the shared expert's gate is one more row of the router's product
            pieces.append((tensors[self.names["shared_gate"]].reshape(1, self.hidden), r.shape[0], None, None))
            self.shared.load({name: tensors[name] for name in self.shared.tensor_specs()})
        rows = r.shape[0] + len(pieces) - 1
        self.w_router = pack_rows(lib, pieces, rows, r.shape[1], r.dtype, r.device, allowed)
        self.correction = tensors[self.names["correction"]].contiguous() if self.has_correction else None
        # all experts' matrices in one tensor each; for the matrix cores (bfloat16, sizes that are multiples of 32) every
        # expert's matrix fragment-major, so that a wave's load is 1 KB in a row
        self.frag = bool(allowed and r.dtype == torch.bfloat16 and self.hidden % 32 == 0 and self.ff % 32 == 0)

        def stack(what: str) -> torch.Tensor:
            first = tensors[self._name(0, what)]
            out = torch.empty((self.n_experts,) + tuple(first.shape), dtype=first.dtype, device=first.device)
            for i in range(self.n_experts):
                lib.place_rows(tensors[self._name(i, what)].contiguous(), out[i], frag=self.frag)
            return out

        self.w_gate, self.w_up, self.w_down = stack("gate"), stack("up"), stack("down")

    def forward(self, h: torch.Tensor, ctx=None, stream: Optional[torch.Tensor] = None, next_norm=None) -> torch.Tensor:
        lib, t, dev = self.env.lib, h.shape[0], h.device
        z = linear(lib, h, self.w_router, torch.float32)
        pairs = t * self.top
        max_rows = lib.routed_rows(t, self.top, self.n_experts)
        sel = torch.empty(pairs, dtype=torch.int32, device=dev)
        weight = torch.empty(pairs, dtype=torch.float32, device=dev)
        row_pair = torch.empty(max_rows, dtype=torch.int32, device=dev)
        tile_expert = torch.empty(2 * (max_rows // 16), dtype=torch.int32, device=dev)      # experts, then positions in their runs
        if self.plain:
            lib.route_top(z, self.n_experts, self.top, sel, weight, row_pair, tile_expert)
        else:
            lib.route_choose(z, self.n_outputs, self.n_experts, self.top, self.score, self.correction, sel, weight, row_pair,
                             tile_expert)
        y = torch.empty((max_rows, self.ff + self.hidden), dtype=h.dtype, device=dev)         # scratch: gated units, scaled inputs
        out = torch.empty((pairs, self.hidden), dtype=torch.float32, device=dev)
        lib.routed_experts(h, weight if self.weight_on == "input" else None, self.top, row_pair, tile_expert, self.w_gate,
                           self.w_up, self.w_down, y, out, self.limit or 0.0, self.alpha, w_frag=self.frag)
        if self.weight_on == "output":
            total = torch.empty((t, self.hidden), dtype=torch.float32, device=dev)
            both = None if self.shared is None else self.shared.forward(h, ctx)
            lib.experts_combine(out, sel, weight, self.top, self.n_experts, h, both, z if both is not None else None,
                                self.n_outputs, total)
            return total
        if self.top == 1:
            return out
        total = torch.empty((t, self.hidden), dtype=torch.float32, device=dev)
        lib.pairs_sum(out, self.top, total)
        return total


register_feed_forward("routed_experts", RoutedExperts)
