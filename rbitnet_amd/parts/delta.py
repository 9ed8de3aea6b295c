"""The gated delta rule with a decay per key channel: a recurrent mixer whose state is, per head, a matrix
S [key dim, value dim] in float32.

Per token, with h the mixer's input:
    q, k = Wq h, Wk h  (kv_heads x dim each);  v = Wv h  (heads x vdim);  head i reads q/k head i // (heads // kv_heads)
    each of q, k, v: short causal convolution per channel, then silu
    q, k: unit vectors per head, x / sqrt(sum x^2 + 1e-6);  q also times dim^(-1/2)
    beta = sigmoid(Wb h)                                          one per head
    g = exp(-exp(A_log[head]) * softplus(Wa2 (Wa1 h) + dt_bias))  one per head and key channel
    S <- diag(g) S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q          (the read-out sees the token's own write)
    o <- o / sqrt(mean(o^2) + eps) * norm * sigmoid(Wg2 (Wg1 h));   out = Wo o

In float32: everything from the unit vectors on (decays, beta, the recurrence, the read-out norm and its gate); the
projections and the convolution's inputs are float32 sums of products in the compute dtype.  The state and the
convolution's last taps - 1 inputs live in the cache (`view.states["delta"]`, kept column by column as
[slots, heads, vdim, dim], and `view.states["conv"]`).

Parameters: heads, kv_heads, dim, vdim, conv (taps), eps (of the read-out norm), unit_eps (1e-6), low-rank sizes come
from the tensors' declared shapes: decay_rank, gate_rank.  names: the tensors below the layer's prefix.
"""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from ..errors import ConfigError
from .base import BuildEnv, CacheRequest, Part, TensorSpec, register_mixer
from .linear import linear, pack_rows
from .short_conv import ACT_SILU, ShortConv

DEFAULT_NAMES = {"q": "q", "k": "k", "v": "v", "q_conv": "q.conv", "k_conv": "k.conv", "v_conv": "v.conv", "b": "b",
                 "a_log": "A_log", "norm": "norm", "a1": "a1", "a2": "a2", "dt_bias": "dt_bias", "g1": "g1", "g2": "g2",
                 "o": "o"}


class ChannelDelta(Part):
    graph_safe = True
    plan_safe = True

    def __init__(self, params: Dict, env: BuildEnv):
        self.env = env
        self.heads = int(params["heads"])
        self.kv_heads = int(params.get("kv_heads") or self.heads)
        self.dim, self.vdim = int(params["dim"]), int(params["vdim"])
        self.taps = int(params["conv"])
        self.eps = float(params["eps"])
        self.unit_eps = float(params.get("unit_eps", 1e-6))
        self.decay_rank, self.gate_rank = int(params["decay_rank"]), int(params["gate_rank"])
        if self.heads <= 0 or self.kv_heads <= 0 or self.heads % self.kv_heads != 0:
            raise ConfigError(f"delta rule: {self.heads} heads cannot share {self.kv_heads} q/k heads")
        if not 0 < self.dim <= 512:
            raise ConfigError(f"delta rule: key size {self.dim} not supported (1 to 512)")
        self.names = dict(DEFAULT_NAMES, **(params.get("names") or {}))
        self.hidden = env.hidden_size
        self.n_qk, self.n_v = self.kv_heads * self.dim, self.heads * self.vdim
        self.n_conv = 2 * self.n_qk + self.n_v
        self.conv = ShortConv(self.n_conv, self.taps, env, residual=False, act=ACT_SILU)
        self.cache_from = None

    # ------------------------------------------------------------------ tensors
    def tensor_specs(self) -> Dict[str, TensorSpec]:
        n, e = self.names, self.hidden
        gain = lambda *shape: TensorSpec(tuple(shape), role="gain", init="normal")
        return {
            n["q"]: TensorSpec((self.n_qk, e)), n["k"]: TensorSpec((self.n_qk, e)), n["v"]: TensorSpec((self.n_v, e)),
            n["q_conv"]: gain(self.n_qk, self.taps), n["k_conv"]: gain(self.n_qk, self.taps),
            n["v_conv"]: gain(self.n_v, self.taps),
            n["b"]: TensorSpec((self.heads, e)), n["a_log"]: gain(self.heads),
            n["norm"]: TensorSpec((self.vdim,), role="gain", init="ones_normal"),
            n["a1"]: TensorSpec((self.decay_rank, e)), n["a2"]: TensorSpec((self.heads * self.dim, self.decay_rank)),
            n["dt_bias"]: gain(self.heads * self.dim),
            n["g1"]: TensorSpec((self.gate_rank, e)), n["g2"]: TensorSpec((self.n_v, self.gate_rank)),
            n["o"]: TensorSpec((e, self.n_v)),
        }

    def load(self, tensors: Dict[str, torch.Tensor]) -> None:
        lib, allowed, n = self.env.lib, not getattr(self.env, "generic_only", False), self.names
        first = tensors[n["q"]]
        # one product for q, k, v and beta, one for the two low-rank inputs
        pieces, row = [], 0
        for key in ("q", "k", "v", "b"):
            pieces.append((tensors[n[key]], row, None, None))
            row += tensors[n[key]].shape[0]
        self.w_in = pack_rows(lib, pieces, row, self.hidden, first.dtype, first.device, allowed)
        self.b_col = self.n_conv
        low = [(tensors[n["a1"]], 0, None, None), (tensors[n["g1"]], self.decay_rank, None, None)]
        self.w_low = pack_rows(lib, low, self.decay_rank + self.gate_rank, self.hidden, first.dtype, first.device, allowed)
        # the second halves as one block-diagonal matrix: [a | gate] = [a1 h | g1 h] W^T
        r = self.decay_rank + self.gate_rank
        up = torch.zeros((self.heads * self.dim + self.n_v, r), dtype=first.dtype, device=first.device)
        up[:self.heads * self.dim, :self.decay_rank] = tensors[n["a2"]]
        up[self.heads * self.dim:, self.decay_rank:] = tensors[n["g2"]]
        self.w_up = pack_rows(lib, [(up, 0, None, None)], up.shape[0], r, first.dtype, first.device, allowed)
        self.conv.load(torch.cat([tensors[n["q_conv"]], tensors[n["k_conv"]], tensors[n["v_conv"]]]))
        self.a_log, self.dt_bias, self.norm = tensors[n["a_log"]], tensors[n["dt_bias"]], tensors[n["norm"]]
        o = tensors[n["o"]]
        self.w_o = pack_rows(lib, [(o, 0, None, None)], o.shape[0], o.shape[1], o.dtype, o.device, allowed)

    def cache_requests(self) -> List[CacheRequest]:
        out = [CacheRequest("state", state_shape=(self.heads, self.vdim, self.dim), state_init=0.0, name="delta")]
        conv = self.conv.cache_request("conv")
        return out + ([conv] if conv else [])

    def cache_request(self) -> Optional[CacheRequest]:
        return self.cache_requests()[0]

    # ------------------------------------------------------------------ forward
    def forward(self, h: torch.Tensor, ctx, view, stream: Optional[torch.Tensor] = None, next_norm=None) -> torch.Tensor:
        lib, t = self.env.lib, h.shape[0]
        proj = linear(lib, h, self.w_in, torch.float32)                       # [T, q | k | v | b]
        low = linear(lib, h, self.w_low, self.env.dtype)                      # [T, a1 h | g1 h]
        up = linear(lib, low, self.w_up, torch.float32)                       # [T, a | gate]
        qkv = self.conv.forward(proj, ctx, view.states.get("conv"), torch.float32)
        n_a = self.heads * self.dim
        beta = torch.empty((t, self.heads), dtype=torch.float32, device=h.device)
        lib.delta_prep(qkv, self.kv_heads, self.dim, up, self.dt_bias, self.a_log, self.heads, proj, self.b_col, beta,
                       self.dim ** -0.5, self.unit_eps)
        o = torch.empty((t, self.n_v), dtype=torch.float32, device=h.device)
        lib.delta_rule(qkv, self.kv_heads, self.dim, self.heads, self.vdim, up, beta, view.states["delta"], ctx, o)
        on = torch.empty((t, self.n_v), dtype=self.env.dtype, device=h.device)
        lib.gated_rmsnorm(o, self.norm, up, n_a, self.eps, self.heads, self.vdim, on)
        return linear(lib, on, self.w_o, torch.float32)


class HeadDelta(Part):
    """The gated delta rule with ONE decay per head and a full gate on the read-out:
        q, k, v as above (convolution, silu; q, k unit vectors, q times dim^(-1/2));  beta = sigmoid(Wb h)
        g = exp(-exp(A_log[head]) * softplus(Wa h + dt_bias))                    one number per head
        S <- g S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q
        o <- o / sqrt(mean(o^2) + eps) * norm * silu(Wg h);   out = Wo o
    All projections are one product; the recurrence is the same kernel with the decay read once per head.
    Parameters: heads, kv_heads, dim, vdim, conv (taps), eps, unit_eps (1e-6), names."""
    graph_safe = True
    plan_safe = True

    NAMES = {"q": "q", "k": "k", "v": "v", "q_conv": "q.conv", "k_conv": "k.conv", "v_conv": "v.conv", "b": "b", "a": "a",
             "a_log": "A_log", "dt_bias": "dt_bias", "norm": "norm", "g": "g", "o": "o"}

    def __init__(self, params: Dict, env: BuildEnv):
        self.env = env
        self.heads = int(params["heads"])
        self.kv_heads = int(params.get("kv_heads") or self.heads)
        self.dim, self.vdim = int(params["dim"]), int(params["vdim"])
        self.taps = int(params["conv"])
        self.eps = float(params["eps"])
        self.unit_eps = float(params.get("unit_eps", 1e-6))
        if self.heads <= 0 or self.kv_heads <= 0 or self.heads % self.kv_heads != 0:
            raise ConfigError(f"delta rule: {self.heads} heads cannot share {self.kv_heads} q/k heads")
        if not 0 < self.dim <= 512:
            raise ConfigError(f"delta rule: key size {self.dim} not supported (1 to 512)")
        self.names = dict(self.NAMES, **(params.get("names") or {}))
        self.hidden = env.hidden_size
        self.n_qk, self.n_v = self.kv_heads * self.dim, self.heads * self.vdim
        self.n_conv = 2 * self.n_qk + self.n_v
        self.conv = ShortConv(self.n_conv, self.taps, env, residual=False, act=ACT_SILU)
        self.cache_from = None

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        n, e = self.names, self.hidden
        gain = lambda *shape: TensorSpec(tuple(shape), role="gain", init="normal")
        return {
            n["q"]: TensorSpec((self.n_qk, e)), n["k"]: TensorSpec((self.n_qk, e)), n["v"]: TensorSpec((self.n_v, e)),
            n["q_conv"]: gain(self.n_qk, self.taps), n["k_conv"]: gain(self.n_qk, self.taps),
            n["v_conv"]: gain(self.n_v, self.taps),
            n["b"]: TensorSpec((self.heads, e)), n["a"]: TensorSpec((self.heads, e)),
            n["a_log"]: gain(self.heads), n["dt_bias"]: gain(self.heads),
            n["norm"]: TensorSpec((self.vdim,), role="gain", init="ones_normal"),
            n["g"]: TensorSpec((self.n_v, e)), n["o"]: TensorSpec((e, self.n_v)),
        }

    def load(self, tensors: Dict[str, torch.Tensor]) -> None:
        lib, allowed, n = self.env.lib, not getattr(self.env, "generic_only", False), self.names
        first = tensors[n["q"]]
        pieces, row = [], 0
        self.cols = {}
        for key in ("q", "k", "v", "b", "a", "g"):           # one product: [q | k | v | beta | decay | gate]
            self.cols[key] = row
            pieces.append((tensors[n[key]], row, None, None))
            row += tensors[n[key]].shape[0]
        self.w_in = pack_rows(lib, pieces, row, self.hidden, first.dtype, first.device, allowed)
        self.conv.load(torch.cat([tensors[n["q_conv"]], tensors[n["k_conv"]], tensors[n["v_conv"]]]))
        self.a_log, self.dt_bias, self.norm = tensors[n["a_log"]], tensors[n["dt_bias"]], tensors[n["norm"]]
        o = tensors[n["o"]]
        self.w_o = pack_rows(lib, [(o, 0, None, None)], o.shape[0], o.shape[1], o.dtype, o.device, allowed)

    def cache_requests(self) -> List[CacheRequest]:
        out = [CacheRequest("state", state_shape=(self.heads, self.vdim, self.dim), state_init=0.0, name="delta")]
        conv = self.conv.cache_request("conv")
        return out + ([conv] if conv else [])

    def cache_request(self) -> Optional[CacheRequest]:
        return self.cache_requests()[0]

    def forward(self, h: torch.Tensor, ctx, view, stream: Optional[torch.Tensor] = None, next_norm=None) -> torch.Tensor:
        lib, t, c = self.env.lib, h.shape[0], self.cols
        proj = linear(lib, h, self.w_in, torch.float32)
        qkv = self.conv.forward(proj, ctx, view.states.get("conv"), torch.float32)
        beta = torch.empty((t, self.heads), dtype=torch.float32, device=h.device)
        lib.recurrence_prep(qkv, self.kv_heads, self.dim, True, self.dim ** -0.5, self.unit_eps, proj, c["a"], self.heads, 0,
                            self.dt_bias, self.a_log, 1.0, self.heads, b_in=proj, b_col=c["b"], beta=beta)
        o = torch.empty((t, self.n_v), dtype=torch.float32, device=h.device)
        lib.linear_recurrence(qkv, self.kv_heads, self.dim, self.heads, self.vdim, proj, c["a"], True, beta,
                              view.states["delta"], ctx, o)
        on = torch.empty((t, self.n_v), dtype=self.env.dtype, device=h.device)
        lib.gated_rmsnorm_act(o, self.norm, proj, c["g"], 1, self.eps, self.heads, self.vdim, on)
        return linear(lib, on, self.w_o, torch.float32)


class DecayAttention(Part):
    """Gated linear attention: a matrix state per head that decays per key channel and is read with the query.
        q = Wq h * dim^(-1/2),  k = Wk h  (heads x dim);  v = Wv h  (heads x vdim)
        alpha = sigmoid(Wa2 (Wa1 h) + bias) ^ (1 / tau)                          heads x dim, in float32
        S <- diag(alpha) S + k v^T;  o = S^T q          (the plain rule: no correction towards the new value)
        o <- o / sqrt(mean(o^2) + eps) * norm;  out = Wo (o * silu(Wg h))
    The state lives in the cache's per-slot storage (`view.states["decay"]`, [slots, heads, vdim, dim] float32).
    Parameters: heads, dim, vdim, tau, decay_rank (the inner size of the decay's two matrices), eps, names."""
    graph_safe = True
    plan_safe = True

    NAMES = {"q": "q", "k": "k", "v": "v", "g": "g", "o": "o", "norm": "norm", "a1": "a1", "a2": "a2", "a_bias": "a2.b"}

    def __init__(self, params: Dict, env: BuildEnv):
        self.env = env
        self.heads, self.dim, self.vdim = int(params["heads"]), int(params["dim"]), int(params["vdim"])
        self.tau = float(params["tau"])
        self.decay_rank = int(params["decay_rank"])
        self.eps = float(params["eps"])
        if min(self.heads, self.dim, self.vdim, self.decay_rank) <= 0 or self.dim > 512:
            raise ConfigError("decay attention: sizes must be positive, the key size at most 512")
        if not self.tau > 0:
            raise ConfigError(f"decay attention: tau must be positive, found {self.tau}")
        self.names = dict(self.NAMES, **(params.get("names") or {}))
        self.hidden = env.hidden_size
        self.n_qk, self.n_v = self.heads * self.dim, self.heads * self.vdim
        self.cache_from = None

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        n, e = self.names, self.hidden
        return {
            n["q"]: TensorSpec((self.n_qk, e)), n["k"]: TensorSpec((self.n_qk, e)), n["v"]: TensorSpec((self.n_v, e)),
            n["g"]: TensorSpec((self.n_v, e)), n["o"]: TensorSpec((e, self.n_v)),
            n["norm"]: TensorSpec((self.vdim,), role="gain", init="ones_normal"),
            n["a1"]: TensorSpec((self.decay_rank, e)), n["a2"]: TensorSpec((self.n_qk, self.decay_rank)),
            n["a_bias"]: TensorSpec((self.n_qk,), role="gain", init="normal"),
        }

    def load(self, tensors: Dict[str, torch.Tensor]) -> None:
        lib, allowed, n = self.env.lib, not getattr(self.env, "generic_only", False), self.names
        first = tensors[n["q"]]
        pieces, row = [], 0
        self.cols = {}
        for key in ("q", "k", "v", "g"):                     # one product: [q | k | v | gate]
            self.cols[key] = row
            pieces.append((tensors[n[key]], row, None, None))
            row += tensors[n[key]].shape[0]
        self.w_in = pack_rows(lib, pieces, row, self.hidden, first.dtype, first.device, allowed)
        a1, a2 = tensors[n["a1"]], tensors[n["a2"]]
        self.w_a1 = pack_rows(lib, [(a1, 0, None, None)], a1.shape[0], a1.shape[1], a1.dtype, a1.device, allowed)
        self.w_a2 = pack_rows(lib, [(a2, 0, None, None)], a2.shape[0], a2.shape[1], a2.dtype, a2.device, allowed)
        self.a_bias, self.norm = tensors[n["a_bias"]], tensors[n["norm"]]
        o = tensors[n["o"]]
        self.w_o = pack_rows(lib, [(o, 0, None, None)], o.shape[0], o.shape[1], o.dtype, o.device, allowed)

    def cache_requests(self) -> List[CacheRequest]:
        return [CacheRequest("state", state_shape=(self.heads, self.vdim, self.dim), state_init=0.0, name="decay")]

    def cache_request(self) -> Optional[CacheRequest]:
        return self.cache_requests()[0]

    def forward(self, h: torch.Tensor, ctx, view, stream: Optional[torch.Tensor] = None, next_norm=None) -> torch.Tensor:
        lib, t, c, dt = self.env.lib, h.shape[0], self.cols, self.env.dtype
        proj = linear(lib, h, self.w_in, torch.float32)                       # [T, q | k | v | gate]
        low = linear(lib, h, self.w_a1, dt)
        z = linear(lib, low, self.w_a2, torch.float32)                        # [T, heads * dim]
        lib.recurrence_prep(proj, self.heads, self.dim, False, self.dim ** -0.5, 0.0, z, 0, self.n_qk, 1, self.a_bias, None,
                            self.tau, self.heads)
        o = torch.empty((t, self.n_v), dtype=torch.float32, device=h.device)
        lib.linear_recurrence(proj, self.heads, self.dim, self.heads, self.vdim, z, 0, False, None, view.states["decay"], ctx, o)
        on = torch.empty((t, self.n_v), dtype=dt, device=h.device)
        lib.gated_rmsnorm_act(o, self.norm, proj, c["g"], 1, self.eps, self.heads, self.vdim, on)
        return linear(lib, on, self.w_o, torch.float32)


class TimeMix(Part):
    """Time mixing with a token shift: a matrix state per head that decays per key channel, read BEFORE the token's own write,
    with a bonus for the token itself.  With h' the row of the token before (zeros before a sequence's first):
        m_s = h + (h' - h) * mu_s                                   for s in r, k, v, g, w: five inputs, one per projection
        r, k, v = Wr m_r, Wk m_k, Wv m_v  (heads x dim each);  gate = silu(Wg m_g)
        w = exp(-exp(Ww2 tanh(Ww1 m_w) + w0))                       per head and key channel, in float32
        o = (S + diag(u) k v^T)^T r;   S <- diag(w) S + k v^T       u [heads, dim]: the bonus
        o <- o / sqrt(mean(o^2) + eps) per head;  out = Wo (o * norm * gate)         norm [heads * dim]
    The state S (`view.states["time_mix"]`, [slots, heads, dim, dim] float32, kept column by column) and the last row of h
    (`view.states["time_shift"]`, float32) live in the cache's per-slot storage.  The recurrence is `rb_linear_recurrence`'s
    kernel in its read-before-write form.
    Parameters: heads, dim, decay_rank (the inner size of the decay's two matrices), eps, names."""
    graph_safe = True
    plan_safe = True

    NAMES = {"mu_r": "mu.r", "mu_k": "mu.k", "mu_v": "mu.v", "mu_g": "mu.g", "mu_w": "mu.w", "r": "r", "k": "k", "v": "v", "g": "g",
             "w1": "w1", "w2": "w2", "w0": "w0", "u": "u", "norm": "norm", "o": "o"}

    def __init__(self, params: Dict, env: BuildEnv):
        self.env = env
        self.heads, self.dim = int(params["heads"]), int(params["dim"])
        self.decay_rank = int(params["decay_rank"])
        self.eps = float(params["eps"])
        if min(self.heads, self.dim, self.decay_rank) <= 0 or self.dim > 512:
            raise ConfigError("time mixing: sizes must be positive, the head size at most 512")
        self.names = dict(self.NAMES, **(params.get("names") or {}))
        self.hidden = env.hidden_size
        self.n = self.heads * self.dim
        self.cache_from = None

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        n, e = self.names, self.hidden
        gain = lambda *shape: TensorSpec(tuple(shape), role="gain", init="normal")
        out = {n["mu_" + s]: gain(e) for s in "rkvgw"}
        out.update({n[s]: TensorSpec((self.n, e)) for s in "rkvg"})
        out.update({n["w1"]: TensorSpec((self.decay_rank, e)), n["w2"]: TensorSpec((self.n, self.decay_rank)), n["w0"]: gain(self.n),
                    n["u"]: gain(self.heads, self.dim), n["norm"]: TensorSpec((self.n,), role="gain", init="ones_normal"),
                    n["o"]: TensorSpec((e, self.n))})
        return out

    def load(self, tensors: Dict[str, torch.Tensor]) -> None:
        lib, allowed, n = self.env.lib, not getattr(self.env, "generic_only", False), self.names
        pack = lambda t: pack_rows(lib, [(t, 0, None, None)], t.shape[0], t.shape[1], t.dtype, t.device, allowed)
        self.mu = torch.stack([tensors[n["mu_" + s]] for s in "rkvgw"]).contiguous()
        self.w_in = [pack(tensors[n[s]]) for s in "rkvg"]
        self.w_1, self.w_2, self.w_o = pack(tensors[n["w1"]]), pack(tensors[n["w2"]]), pack(tensors[n["o"]])
        self.w0, self.u, self.norm = tensors[n["w0"]], tensors[n["u"]], tensors[n["norm"]]

    def cache_requests(self) -> List[CacheRequest]:
        return [CacheRequest("state", state_shape=(self.heads, self.dim, self.dim), state_init=0.0, name="time_mix"),
                CacheRequest("state", state_shape=(self.hidden,), state_init=0.0, name="time_shift")]

    def cache_request(self) -> Optional[CacheRequest]:
        return self.cache_requests()[0]

    def forward(self, h: torch.Tensor, ctx, view, stream: Optional[torch.Tensor] = None, next_norm=None) -> torch.Tensor:
        lib, t, dt = self.env.lib, h.shape[0], self.env.dtype
        mixes = torch.empty((5, t, self.hidden), dtype=dt, device=h.device)
        lib.shift_mix(h, view.states["time_shift"], self.mu, ctx, mixes)
        r, k, v, g = (linear(lib, mixes[i], self.w_in[i], torch.float32) for i in range(4))
        low = torch.empty((t, self.decay_rank), dtype=dt, device=h.device)
        lib.tanh_cast(linear(lib, mixes[4], self.w_1, torch.float32), low)
        decay = linear(lib, low, self.w_2, torch.float32)
        lib.decay_exp_exp(decay, self.w0, self.heads, self.dim)
        o = torch.empty((t, self.n), dtype=torch.float32, device=h.device)
        lib.time_mix_recurrence(r, k, v, decay, self.u, view.states["time_mix"], ctx, o, self.heads, self.dim, self.dim)
        on = torch.empty((t, self.n), dtype=dt, device=h.device)
        lib.gated_rmsnorm_heads(o, self.norm, g, 1, self.eps, self.heads, self.dim, on)
        return linear(lib, on, self.w_o, torch.float32)


register_mixer("channel_delta", ChannelDelta)
register_mixer("time_mix", TimeMix)
register_mixer("gated_delta", HeadDelta)
register_mixer("decay_attention", DecayAttention)
