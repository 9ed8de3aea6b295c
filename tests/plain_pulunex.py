"""A plain, slow implementation of the Pulunex decoder in float64 on whole sequences: the oracle of the tests.

One function per mechanism, written from the equations below; it shares no code with the package.

    embedding        x_t = E[id_t] * c + P[t]                                   (P: a learned vector per position)
    scalar_rmsnorm   x / sqrt(mean(x^2) + eps) * g                              (g one number)
    token_shift      h_t + (h_(t-1) - h_t) * s   per channel, h_(-1) = 0
    talking_attention  q = Wq h + bq, k = Wk h + bk, v = Wv h + bv; q and k heads / sqrt(mean(.^2) + eps);
                     a[g, i, j] = q_gi . k_(g/(H/G))j * scale;  b[h, i, j] = sum_g T[h, g] a[g, i, j];
                     j visible from i when j <= i and i // C == j // C (C: the chunk; None: all j <= i);
                     softmax over the visible j; heads concatenated; Wo
    dense_gelu       Wd gelu(Wu h), gelu(z) = z/2 (1 + tanh(sqrt(2/pi) (z + 0.044715 z^3)))
    softmax_experts  s = softmax(Wr h) over real and identity experts; the `top` largest of s + correction (lowest index
                     among equals); sum over the chosen of s_e * expert_e(h), expert(h) = Wd (silu(Wg h) * (Wu h)), an identity
                     expert (the last `identity` outputs of the router) giving h itself; + sigmoid(w_sg . h) * shared(h)
    layer            x += mixer(shift(norm1(x)));  x += ff(norm2(x))  (no feed-forward: the first sum only)
    head             W norm(x) * logit_scale

A layer whose mixer has `kv_from = j` has no k and v matrices and attends over the normalised keys and the values of layer j.
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional

import numpy as np
import torch

F64 = torch.float64


def embedding(table: torch.Tensor, positions: torch.Tensor, ids, scale: float, first: int = 0) -> torch.Tensor:
    ids = torch.as_tensor(list(ids), dtype=torch.long)
    where = torch.arange(first, first + len(ids))
    return table.to(F64)[ids] * scale + positions.to(F64)[where]


def scalar_rmsnorm(x: torch.Tensor, gain: torch.Tensor, eps: float) -> torch.Tensor:
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * gain.to(F64).reshape(())


def unit_rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def token_shift(h: torch.Tensor, s: torch.Tensor) -> torch.Tensor:
    before = torch.cat([torch.zeros_like(h[:1]), h[:-1]], dim=0)
    return h + (before - h) * s.to(F64)


def visible(n: int, chunk: Optional[int]) -> torch.Tensor:
    i = torch.arange(n)[:, None]
    j = torch.arange(n)[None, :]
    ok = j <= i
    if chunk is not None:
        ok = ok & (i // chunk == j // chunk)
    return ok


def attention_keys_values(h: torch.Tensor, w: Dict[str, torch.Tensor], m: Dict, eps: float):
    """normalised keys [G, T, d] and values [G, T, dv] of a layer that has projections of its own"""
    t, g, d, dv = h.shape[0], m["kv_heads"], m["dim"], m["vdim"]
    k = (h @ w["k"].to(F64).T + w["k.b"].to(F64)).view(t, g, d).transpose(0, 1)
    v = (h @ w["v"].to(F64).T + w["v.b"].to(F64)).view(t, g, dv).transpose(0, 1)
    return unit_rms(k, eps), v


def mixed_weights(h: torch.Tensor, w: Dict[str, torch.Tensor], m: Dict, eps: float, k: torch.Tensor) -> torch.Tensor:
    """the softmax weights [H, T, T] of every head: zero where a key is not seen"""
    t, hq, g, d = h.shape[0], m["heads"], m["kv_heads"], m["dim"]
    q = unit_rms((h @ w["q"].to(F64).T + w["q.b"].to(F64)).view(t, hq, d).transpose(0, 1), eps)       # [H, T, d]
    kv_of = torch.arange(hq) // (hq // g)
    a = torch.einsum("hid,hjd->hij", q, k[kv_of]) * m["scale"]
    b = torch.einsum("hg,gij->hij", w["talk"].to(F64), a)
    chunk = (m.get("mask") or {}).get("size")
    b = b.masked_fill(~visible(t, chunk)[None], -math.inf)
    return torch.softmax(b, dim=-1)


def talking_attention(h: torch.Tensor, w: Dict[str, torch.Tensor], m: Dict, eps: float, k: torch.Tensor, v: torch.Tensor):
    t, hq, g = h.shape[0], m["heads"], m["kv_heads"]
    p = mixed_weights(h, w, m, eps, k)
    kv_of = torch.arange(hq) // (hq // g)
    o = torch.einsum("hij,hje->ihe", p, v[kv_of]).reshape(t, hq * m["vdim"])
    return o @ w["o"].to(F64).T


def gelu_tanh(z: torch.Tensor) -> torch.Tensor:
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def dense_gelu(h: torch.Tensor, w: Dict[str, torch.Tensor]) -> torch.Tensor:
    return gelu_tanh(h @ w["up"].to(F64).T) @ w["down"].to(F64).T


def silu_expert(h: torch.Tensor, gate, up, down) -> torch.Tensor:
    a = h @ gate.to(F64).T
    return (a * torch.sigmoid(a) * (h @ up.to(F64).T)) @ down.to(F64).T


def choose(scores: torch.Tensor, correction: torch.Tensor, top: int) -> List[List[int]]:
    """per token, the `top` experts with the largest corrected score, lowest index among equals"""
    c = (scores + correction.to(F64)).tolist()
    return [sorted(range(len(row)), key=lambda e: (-row[e], e))[:top] for row in c]


def softmax_experts(h: torch.Tensor, w: Dict[str, torch.Tensor], mlp: Dict, router_input: Optional[torch.Tensor] = None) -> torch.Tensor:
    r = mlp["router"]
    n_real, n_id, top = r["experts"], r.get("identity", 0), r["top"]
    hr = h if router_input is None else router_input
    s = torch.softmax(hr @ w["router"].to(F64).T, dim=-1)
    out = torch.zeros_like(h)
    for t, chosen in enumerate(choose(s, w["correction"], top)):
        for e in chosen:
            if e >= n_real:
                assert e < n_real + n_id
                out[t] += s[t, e] * h[t]
            else:
                out[t] += s[t, e] * silu_expert(h[t:t + 1], w[f"e{e}.gate"], w[f"e{e}.up"], w[f"e{e}.down"])[0]
    if mlp.get("shared") is not None:
        gate = torch.sigmoid(h @ w["shared.sg"].to(F64).T)                     # [T, 1]
        out = out + gate * silu_expert(h, w["shared.gate"], w["shared.up"], w["shared.down"])
    return out


def sub(tensors: Dict[str, torch.Tensor], prefix: str) -> Dict[str, torch.Tensor]:
    return {k[len(prefix):]: v for k, v in tensors.items() if k.startswith(prefix)}


def forward(config: Dict, tensors: Dict[str, torch.Tensor], ids, streams: Optional[list] = None) -> torch.Tensor:
    """logits [T, vocab] of one whole sequence; `streams` (a list) receives the stream after every layer"""
    eps = float(config["norm"]["eps"])
    x = embedding(tensors["embed"], tensors["pos"], ids, float(config["embedding"]["scale"]))
    kept = {}
    for i, layer in enumerate(config["layers"]):
        assert layer["type"] == "attention"
        m, p = layer["mixer"], f"l{i}."
        h = token_shift(scalar_rmsnorm(x, tensors[p + "norm1"], eps), tensors[p + "shift"])
        w = sub(tensors, p + "mix.")
        if m.get("kv_from") is None:
            kept[i] = attention_keys_values(h, w, m, eps)
        k, v = kept[i if m.get("kv_from") is None else m["kv_from"]]
        x = x + talking_attention(h, w, m, eps, k, v)
        mlp = layer.get("mlp")
        if mlp is not None:
            h2 = scalar_rmsnorm(x, tensors[p + "norm2"], eps)
            w2 = sub(tensors, p + "mlp.")
            x = x + (dense_gelu(h2, w2) if mlp["kind"] == "dense" else softmax_experts(h2, w2, mlp))
        if streams is not None:
            streams.append(x.clone())
    xn = scalar_rmsnorm(x, tensors["final.norm"], eps)
    return xn @ tensors["head"].to(F64).T * float(config["logit_scale"])


class PlainPulunex:
    def __init__(self, config: Dict, tensors: Dict[str, torch.Tensor]):
        self.config, self.tensors = config, tensors

    def logits(self, ids, streams: Optional[list] = None) -> torch.Tensor:
        return forward(self.config, self.tensors, ids, streams)


# ---------------------------------------------------------------------- random models for the tests

def tensor_shapes(config: Dict) -> Dict[str, tuple]:
    e, out = config["width"], {}
    out["embed"], out["pos"] = (config["vocab"], e), (config["max_positions"], e)
    for i, layer in enumerate(config["layers"]):
        m, p = layer["mixer"], f"l{i}."
        out[p + "norm1"], out[p + "shift"] = (), (e,)
        out[p + "mix.q"], out[p + "mix.q.b"] = (m["heads"] * m["dim"], e), (m["heads"] * m["dim"],)
        if m.get("kv_from") is None:
            out[p + "mix.k"], out[p + "mix.k.b"] = (m["kv_heads"] * m["dim"], e), (m["kv_heads"] * m["dim"],)
            out[p + "mix.v"], out[p + "mix.v.b"] = (m["kv_heads"] * m["vdim"], e), (m["kv_heads"] * m["vdim"],)
        out[p + "mix.talk"] = (m["heads"], m["heads"])
        out[p + "mix.o"] = (e, m["heads"] * m["vdim"])
        mlp = layer.get("mlp")
        if mlp is None:
            continue
        out[p + "norm2"] = ()
        if mlp["kind"] == "dense":
            out[p + "mlp.up"], out[p + "mlp.down"] = (mlp["ff"], e), (e, mlp["ff"])
            continue
        r, f = mlp["router"], mlp["expert"]["ff"]
        for j in range(r["experts"]):
            out[p + f"mlp.e{j}.gate"], out[p + f"mlp.e{j}.up"], out[p + f"mlp.e{j}.down"] = (f, e), (f, e), (e, f)
        n_out = r["experts"] + r.get("identity", 0)
        out[p + "mlp.router"], out[p + "mlp.correction"] = (n_out, e), (n_out,)
        if mlp.get("shared") is not None:
            fs = mlp["shared"]["ff"]
            out[p + "mlp.shared.gate"], out[p + "mlp.shared.up"], out[p + "mlp.shared.down"] = (fs, e), (fs, e), (e, fs)
            out[p + "mlp.shared.sg"] = (1, e)
    out["final.norm"], out["head"] = (), (config["vocab"], e)
    return out


def random_tensors(config: Dict, seed: int, dtype=torch.bfloat16) -> Dict[str, torch.Tensor]:
    """weights whose sizes keep every activation of order one; values that the dtype holds exactly"""
    rng = np.random.default_rng(seed)
    out = {}
    for name, shape in tensor_shapes(config).items():
        last = name.rsplit(".", 1)[-1]
        if last in ("norm1", "norm2", "norm"):
            a = 1.0 + 0.2 * rng.standard_normal(shape)
        elif last == "shift":
            a = rng.uniform(0.0, 1.0, shape)
        elif last == "talk":
            a = np.eye(shape[0]) + rng.standard_normal(shape) / math.sqrt(shape[0]) * 0.5
        elif last == "correction":
            a = 0.1 * rng.standard_normal(shape)
        elif last == "b":
            a = 0.3 * rng.standard_normal(shape)
        elif name in ("embed", "pos"):
            a = rng.standard_normal(shape) * (0.5 if name == "pos" else 1.0)
        elif last == "router" or last == "sg":
            a = rng.standard_normal(shape) * 2.0 / math.sqrt(shape[-1])
        else:
            a = rng.standard_normal(shape) / math.sqrt(shape[-1])
        out[name] = torch.tensor(a, dtype=torch.float32).to(dtype)
    return out
