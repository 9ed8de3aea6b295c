"""A plain, slow float64 implementation of the Menerax decoder, one function per mechanism, whole sequences only
(no cache, no state, no batches): the oracle of the tests.  It shares no code with the package.

Notation: T tokens, E width; weights are [out, in] and applied as x @ W.T.  A layer is
    x <- x + out_norm_1(mixer(x));  x <- x + out_norm_2(feed_forward(x))
where both sublayers read the stream itself and the norm stands on their outputs.
"""
from __future__ import annotations

import json
import math
import os
from typing import Dict, List, Optional

import torch

F64 = torch.float64


# ---------------------------------------------------------------- small things
def unit_rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def norm_plain(x, w, eps):
    return unit_rms(x, eps) * w


def norm_around_zero(x, w, eps):
    """The model's norm: its weight is stored as the distance from one."""
    return unit_rms(x, eps) * (1.0 + w)


def silu(x):
    return x * torch.sigmoid(x)


def causal_conv(u, w):
    """u [T, C], w [C, taps]: y_t = sum_j w[:, j] u_(t - taps + 1 + j), zeros before the start."""
    t_len, c = u.shape
    taps = w.shape[1]
    padded = torch.cat([torch.zeros(taps - 1, c, dtype=u.dtype), u])
    y = torch.zeros_like(u)
    for j in range(taps):
        y = y + padded[j:j + t_len] * w[:, j]
    return y


def frequencies(dims: int, base: float, scaling: Optional[Dict] = None):
    """f_i = base^(-2i/dims), i < dims/2; with `scaling` {factor, low, high, original} the long wavelengths are
    stretched: l = 2 pi / f; l < original/high keeps f; l > original/low gets f / factor; between, a blend."""
    f = torch.tensor([base ** (-2.0 * i / dims) for i in range(dims // 2)], dtype=F64)
    if not scaling:
        return f
    factor, low, high, orig = (float(scaling[k]) for k in ("factor", "low", "high", "original"))
    out = []
    for fi in f.tolist():
        wave = 2.0 * math.pi / fi
        if wave < orig / high:
            out.append(fi)
        elif wave > orig / low:
            out.append(fi / factor)
        else:
            s = (orig / wave - low) / (high - low)
            out.append((1.0 - s) * fi / factor + s * fi)
    return torch.tensor(out, dtype=F64)


def rotate(x, f, layout: str, first_pos: int = 0):
    """x [T, H, D]: the first 2 len(f) numbers of every head are rotated by position * f; "pairs": 2i with 2i + 1,
    "halves": i with i + len(f).  The rest pass."""
    t_len = x.shape[0]
    half = f.shape[0]
    dims = 2 * half
    a = (torch.arange(t_len, dtype=F64) + first_pos)[:, None] * f[None, :]
    cos, sin = torch.cos(a)[:, None, :], torch.sin(a)[:, None, :]
    if layout == "halves":
        u, v = x[..., :half], x[..., half:dims]
        return torch.cat([u * cos - v * sin, v * cos + u * sin, x[..., dims:]], dim=-1)
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    r = torch.stack([u * cos - v * sin, v * cos + u * sin], dim=-1).reshape(*x.shape[:-1], dims)
    return torch.cat([r, x[..., dims:]], dim=-1)


def visible(t_len: int, window: Optional[int] = None, keep_first: int = 0):
    """[T, T] bool: j <= i, and with a window also (i - j < window or j < keep_first)."""
    i = torch.arange(t_len)[:, None]
    j = torch.arange(t_len)[None, :]
    seen = j <= i
    if window is not None:
        seen = seen & ((i - j < window) | (j < keep_first))
    return seen


def attention_weights(q, k, scale: float, seen, softcap: Optional[float] = None):
    """q [T, H, D], k [T, G, D] -> weights [H, T, T]."""
    h, g = q.shape[1], k.shape[1]
    kk = k.repeat_interleave(h // g, 1)
    s = torch.einsum("ihd,jhd->hij", q, kk) * scale
    if softcap is not None:
        s = softcap * torch.tanh(s / softcap)
    s = s.masked_fill(~seen, -math.inf)
    return torch.softmax(s, dim=-1)


def attend(q, k, v, scale, seen, softcap=None):
    """-> [T, H, Dv]"""
    w = attention_weights(q, k, scale, seen, softcap)
    vv = v.repeat_interleave(q.shape[1] // v.shape[1], 1)
    return torch.einsum("hij,jhd->ihd", w, vv)


# ---------------------------------------------------------------- mixers
def latent_attention(h, w: Dict[str, torch.Tensor], p: Dict, eps: float):
    """Queries and keys/values through latents; every head's key is an unrotated part made from the latent beside one
    rotated part that all heads share."""
    t_len = h.shape[0]
    heads, d, r, dv, rank = p["heads"], p["dim"], p["rot_dim"], p["vdim"], p["kv_rank"]
    f = frequencies(p["rot"]["dims"], p["rot"]["base"], p["rot"].get("scaling")) if r else torch.zeros(0, dtype=F64)
    cq = norm_plain(h @ w["dq"].T, w["dq.norm"], eps)
    q = (cq @ w["uq"].T).view(t_len, heads, d + r)
    q_plain, q_rot = q[..., :d], rotate(q[..., d:], f, "pairs")
    down = h @ w["dkv"].T
    c = norm_plain(down[:, :rank], w["dkv.norm"], eps)
    k_rot = rotate(down[:, rank:].view(t_len, 1, r), f, "pairs")
    k_plain = (c @ w["uk"].T).view(t_len, heads, d)
    v = (c @ w["uv"].T).view(t_len, heads, dv)
    qq = torch.cat([q_plain, q_rot], dim=-1)
    kk = torch.cat([k_plain, k_rot.expand(t_len, heads, r)], dim=-1)
    o = attend(qq, kk, v, p["scale"], visible(t_len))
    gate = torch.sigmoid(h @ w["g"].T)                         # [T, heads]
    o = o * gate[:, :, None]
    return o.reshape(t_len, heads * dv) @ w["o"].T


def windowed_attention(h, w: Dict[str, torch.Tensor], p: Dict, eps: float):
    """Grouped-query attention: biases, a short convolution on q, k, v, per-head norms on q and k, rotation of a part of
    the head, capped scores, a window that keeps the first tokens, a gate on every output number."""
    t_len = h.shape[0]
    heads, groups, d, dv = p["heads"], p["kv_heads"], p["dim"], p["vdim"]
    q = causal_conv(h @ w["q"].T + w["q.b"], w["q.conv"]).view(t_len, heads, d)
    k = causal_conv(h @ w["k"].T + w["k.b"], w["k.conv"]).view(t_len, groups, d)
    v = causal_conv(h @ w["v"].T + w["v.b"], w["v.conv"]).view(t_len, groups, dv)
    q, k = norm_plain(q, w["q.norm"], eps), norm_plain(k, w["k.norm"], eps)
    f = frequencies(p["rot"]["dims"], p["rot"]["base"], p["rot"].get("scaling"))
    q, k = rotate(q, f, "halves"), rotate(k, f, "halves")
    mask = p.get("mask")
    seen = visible(t_len) if mask is None else visible(t_len, mask["size"], mask.get("keep_first", 0))
    o = attend(q, k, v, p["scale"], seen, p.get("softcap")).reshape(t_len, heads * dv)
    return (o * torch.sigmoid(h @ w["g"].T)) @ w["o"].T


def time_mix(h, w: Dict[str, torch.Tensor], p: Dict, eps: float):
    """A matrix state per head that decays per key channel, read before the token's own write, with a bonus for the
    token itself."""
    t_len, e = h.shape
    heads, d = p["heads"], p["dim"]
    before = torch.cat([torch.zeros(1, e, dtype=h.dtype), h[:-1]])
    mix = {s: h + (before - h) * w[f"mu.{s}"] for s in "rkvgw"}
    r = (mix["r"] @ w["r"].T).view(t_len, heads, d)
    k = (mix["k"] @ w["k"].T).view(t_len, heads, d)
    v = (mix["v"] @ w["v"].T).view(t_len, heads, d)
    gate = silu(mix["g"] @ w["g"].T)
    decay = torch.exp(-torch.exp(torch.tanh(mix["w"] @ w["w1"].T) @ w["w2"].T + w["w0"])).view(t_len, heads, d)
    u = w["u"]                                                  # [heads, d]
    state = torch.zeros(heads, d, d, dtype=h.dtype)             # [head, key channel, value channel]
    out = torch.zeros(t_len, heads, d, dtype=h.dtype)
    for t in range(t_len):
        kv = k[t][:, :, None] * v[t][:, None, :]
        out[t] = torch.einsum("hkv,hk->hv", state + u[:, :, None] * kv, r[t])
        state = decay[t][:, :, None] * state + kv
    out = unit_rms(out, eps).reshape(t_len, heads * d) * w["norm"] * gate
    return out @ w["o"].T


def sub(w: Dict[str, torch.Tensor], prefix: str) -> Dict[str, torch.Tensor]:
    return {k[len(prefix):]: v for k, v in w.items() if k.startswith(prefix)}


def parallel_mixer(h, w: Dict[str, torch.Tensor], p: Dict, eps: float):
    left = windowed_attention(h, sub(w, "left."), p["left"], eps)
    right = time_mix(h, sub(w, "right."), p["right"], eps)
    return p["left_scale"] * left + p["right_scale"] * right


def feed_forward(h, w: Dict[str, torch.Tensor], limit: float):
    g = torch.clamp(h @ w["gate"].T, max=limit)
    u = torch.clamp(h @ w["up"].T, -limit, limit)
    return (g * torch.sigmoid(1.702 * g) * (u + 1.0)) @ w["down"].T


MIXERS = {"latent_attention": latent_attention, "parallel": parallel_mixer}


# ---------------------------------------------------------------- the model
class PlainMenerax:
    def __init__(self, config: Dict, tensors: Dict[str, torch.Tensor]):
        self.cfg = config
        self.w = {k: v.to(F64) for k, v in tensors.items()}
        self.eps = float(config["norm"]["eps"])

    @classmethod
    def from_folder(cls, folder: str) -> "PlainMenerax":
        from safetensors.torch import load_file
        with open(os.path.join(folder, "config.json")) as f:
            cfg = json.load(f)
        return cls(cfg, load_file(os.path.join(folder, "model.safetensors")))

    def owner(self, i: int) -> int:
        while self.cfg["layers"][i].get("weights_of") is not None:
            i = self.cfg["layers"][i]["weights_of"]
        return i

    def layer(self, i: int, x):
        layer = self.cfg["layers"][i]
        w = sub(self.w, f"l{self.owner(i)}.")
        y = MIXERS[layer["type"]](x, sub(w, "mix."), layer["mixer"], self.eps)
        x = x + norm_around_zero(y, w["norm1"], self.eps)
        if layer.get("mlp") is not None:
            y = feed_forward(x, sub(w, "mlp."), float(layer["mlp"]["limit"]))
            x = x + norm_around_zero(y, w["norm2"], self.eps)
        return x

    def streams(self, tokens: List[int]) -> List[torch.Tensor]:
        """The stream after the embedding and after every layer."""
        x = norm_around_zero(self.w["embed"][torch.tensor(tokens)], self.w["embed.norm"], self.eps)
        out = [x]
        for i in range(len(self.cfg["layers"])):
            x = self.layer(i, x)
            out.append(x)
        return out

    def logits(self, tokens: List[int]) -> torch.Tensor:
        x = self.streams(tokens)[-1]
        return norm_around_zero(x, self.w["final.norm"], self.eps) @ self.w["head"].T


# ---------------------------------------------------------------- random models for the tests
def tensor_shapes(cfg: Dict) -> Dict[str, tuple]:
    """Name -> shape of every tensor of a model; a parallel layer's `right` names its `decay_rank` here."""
    e, v = cfg["width"], cfg["vocab"]
    out = {"embed": (v, e), "embed.norm": (e,), "final.norm": (e,), "head": (v, e)}
    for i, layer in enumerate(cfg["layers"]):
        if layer.get("weights_of") is not None:
            continue
        p = f"l{i}."
        out[p + "norm1"] = (e,)
        m = layer["mixer"]
        if layer["type"] == "latent_attention":
            h, d, r, dv = m["heads"], m["dim"], m["rot_dim"], m["vdim"]
            out.update({p + "mix.dq": (m["q_rank"], e), p + "mix.dq.norm": (m["q_rank"],), p + "mix.uq": (h * (d + r), m["q_rank"]),
                        p + "mix.dkv": (m["kv_rank"] + r, e), p + "mix.dkv.norm": (m["kv_rank"],),
                        p + "mix.uk": (h * d, m["kv_rank"]), p + "mix.uv": (h * dv, m["kv_rank"]), p + "mix.g": (h, e),
                        p + "mix.o": (e, h * dv)})
        else:
            a, b = m["left"], m["right"]
            q, k, val = a["heads"] * a["dim"], a["kv_heads"] * a["dim"], a["kv_heads"] * a["vdim"]
            lp, rp = p + "mix.left.", p + "mix.right."
            for name, rows in (("q", q), ("k", k), ("v", val)):
                out.update({lp + name: (rows, e), lp + name + ".b": (rows,), lp + name + ".conv": (rows, a["conv"])})
            out.update({lp + "q.norm": (a["dim"],), lp + "k.norm": (a["dim"],), lp + "g": (a["heads"] * a["vdim"], e),
                        lp + "o": (e, a["heads"] * a["vdim"])})
            n = b["heads"] * b["dim"]
            out.update({rp + "mu." + s: (e,) for s in "rkvgw"})
            out.update({rp + s: (n, e) for s in "rkvg"})
            out.update({rp + "w1": (b["decay_rank"], e), rp + "w2": (n, b["decay_rank"]), rp + "w0": (n,),
                        rp + "u": (b["heads"], b["dim"]), rp + "norm": (n,), rp + "o": (e, n)})
        if layer.get("mlp") is not None:
            ff = layer["mlp"]["ff"]
            out.update({p + "norm2": (e,), p + "mlp.gate": (ff, e), p + "mlp.up": (ff, e), p + "mlp.down": (e, ff)})
    return out


def random_menerax_tensors(cfg: Dict, seed: int) -> Dict[str, torch.Tensor]:
    """Weights that bfloat16 holds exactly, so that the oracle and a model loaded from a bfloat16 file see the same numbers.
    Sizes are chosen so that every mechanism matters at tiny widths."""
    g = torch.Generator().manual_seed(seed)
    out = {}
    for name, shape in tensor_shapes(cfg).items():
        last = name.rsplit(".", 1)[-1]
        if name.endswith("norm1") or name.endswith("norm2") or name in ("embed.norm", "final.norm"):
            t = 0.2 * torch.randn(shape, generator=g)                      # stored around zero
        elif name.endswith(".norm"):
            t = 1.0 + 0.2 * torch.randn(shape, generator=g)                # plain weights
        elif last == "conv":
            t = 0.6 * torch.randn(shape, generator=g)
        elif ".mu." in name:
            t = torch.rand(shape, generator=g)
        elif last == "w0":
            t = -1.0 + 1.5 * torch.randn(shape, generator=g)               # decays from nearly 1 to nearly 0
        elif last in ("u", "b"):
            t = 0.5 * torch.randn(shape, generator=g)
        elif name == "embed":
            t = torch.randn(shape, generator=g)
        else:
            t = torch.randn(shape, generator=g) * (1.5 / math.sqrt(shape[-1]))
        out[name] = t.to(torch.bfloat16).to(F64)
    return out
