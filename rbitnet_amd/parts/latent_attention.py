"""Causal attention through a latent, with a sink in the softmax, or with a rotated key part beside the latent and a gate
per head.

Per token, with h the mixer's input (all norms RMS norms with a plain weight):
    cq = norm(Wdq h),  q = Wuq cq              (heads x dim)
    c  = norm(Wdkv h)                           (kv_rank numbers: all that is cached of a token)
    per head i:  k_j = Wuk_i c_j,  v_j = Wuv_i c_j,  score_ij = (q_i . k_j) * scale  over the tokens j <= the query's
    weights = exp(score) / (sum_j exp(score_j) + exp(sink_i)): the sink has no key and no value and is not scaled
    out = Wo [sum_j weights_j v_j]_heads
A layer with `cache_from = j` has no Wdkv: it reads the latents that layer j stored, with matrices of its own.

The products with Wuk and Wuv are moved to the query's side, so that attention runs over the cached latents
themselves, one key/value head of size kv_rank shared by all query heads:
    score = (Wuk_i^T q_i) . c_j,      sum_j w_j v_j = Wuv_i (sum_j w_j c_j)
which costs a product per head on either side of attention (`heads_linear`) and never expands the cache, whatever
the step brings on top of whatever past.  Scores, softmax and norms in float32.

With a rotated part (`rot_dim` > 0 and a `position` part whose rotation covers rot_dim numbers): a query head is
[dim unrotated, rot_dim rotated] numbers, Wdkv h has kv_rank + rot_dim rows, the last rot_dim of which (not normed, rotated
by the token's position) are one key part that all heads share, and
    score_ij = (q_i[:dim] . Wuk_i c_j + rotate(q_i[dim:]) . rotate(k_j)) * scale.
The cache then holds per token [c, rotated part] as one key/value head (padded with zeros to a size the matrix cores'
attention kernels take, where that is near), the query [Wuk_i^T q_i[:dim], rotate(q_i[dim:])] in the same layout, and the
rotated part of attention's output meets zeros of Wuv: the same kernels serve.
`sink` (True) can be switched off; `head_gate` (False): head i's output times sigmoid(Wg h)_i (tensor "g" [heads, E]).

Parameters: heads, dim, vdim, q_rank, kv_rank, scale, eps, cache_from, names, rot_dim, position, sink, head_gate.
"""
from __future__ import annotations

from typing import Dict, Optional

import torch

from ..errors import ConfigError
from .base import BuildEnv, CacheRequest, Part, TensorSpec, build_part, register_mixer
from .linear import linear, pack_rows

DEFAULT_NAMES = {"dq": "dq", "dq_norm": "dq.norm", "uq": "uq", "dkv": "dkv", "dkv_norm": "dkv.norm", "uk": "uk", "uv": "uv",
                 "sink": "sink", "o": "o", "gate": "g"}
MAX_RANK = 512             # the attention kernel's largest head size
_MATRIX_CORE_RANKS = (64, 128)     # latents of these sizes in bfloat16 go through the matrix-core attention kernels


class LatentAttention(Part):
    graph_safe = True
    plan_safe = True

    def __init__(self, params: Dict, env: BuildEnv):
        self.env = env
        self.heads, self.dim, self.vdim = int(params["heads"]), int(params["dim"]), int(params["vdim"])
        self.q_rank, self.kv_rank = int(params["q_rank"]), int(params["kv_rank"])
        self.scale = float(params["scale"])
        self.eps = float(params["eps"])
        self.cache_from = params.get("cache_from")
        self.window = None
        if self.kv_rank <= 0 or self.kv_rank > MAX_RANK:
            raise ConfigError(f"latent attention: kv_rank {self.kv_rank} not supported (at most {MAX_RANK})")
        if min(self.heads, self.dim, self.vdim, self.q_rank) <= 0:
            raise ConfigError("latent attention: sizes must be positive")
        if self.dim > 768:
            raise ConfigError(f"latent attention: head size {self.dim} not supported (at most 768)")
        self.names = dict(DEFAULT_NAMES, **(params.get("names") or {}))
        self.hidden = env.hidden_size
        self.has_sink = bool(params.get("sink", True))
        self.has_gate = bool(params.get("head_gate", False))
        self.rot = int(params.get("rot_dim") or 0)
        self.position = None
        self.rot_tables = (None, None, 0)
        if self.rot:
            self.position = build_part("position", params["position"], env)
            tables = getattr(self.position, "rotation_tables", None)
            if tables is None or int(getattr(self.position, "head_dim", 0)) != self.rot or self.rot % 2:
                raise ConfigError(f"latent attention: the position part must rotate all {self.rot} numbers of the rotated part")
            self.plan_safe = bool(getattr(self.position, "plan_safe", False))
            self.graph_safe = bool(getattr(self.position, "graph_safe", False))
            self.rot_tables = tables()
        # one key/value head per token: the latent, then the rotated part; in bfloat16 padded to a head size of the
        # matrix cores' attention kernels where one is near (zeros cost cache, not correctness)
        self.page_width = self.kv_rank + self.rot
        if self.page_width > MAX_RANK:
            raise ConfigError(f"latent attention: latent and rotated part together take {self.page_width} numbers (at most {MAX_RANK})")
        if self.rot and env.dtype == torch.bfloat16 and not getattr(env, "generic_only", False):
            for size in _MATRIX_CORE_RANKS:
                if self.page_width <= size and 4 * self.page_width >= 3 * size:
                    self.page_width = size
                    break

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        n, e = self.names, self.hidden
        gain = lambda size: TensorSpec((size,), role="gain", init="ones_normal")
        out = {n["dq"]: TensorSpec((self.q_rank, e)), n["dq_norm"]: gain(self.q_rank),
               n["uq"]: TensorSpec((self.heads * (self.dim + self.rot), self.q_rank)),
               n["uk"]: TensorSpec((self.heads * self.dim, self.kv_rank)),
               n["uv"]: TensorSpec((self.heads * self.vdim, self.kv_rank)),
               n["o"]: TensorSpec((e, self.heads * self.vdim))}
        if self.has_sink:
            out[n["sink"]] = TensorSpec((self.heads,), role="gain", init="normal")
        if self.has_gate:
            out[n["gate"]] = TensorSpec((self.heads, e))
        if self.cache_from is None:
            out[n["dkv"]] = TensorSpec((self.kv_rank + self.rot, e))
            out[n["dkv_norm"]] = gain(self.kv_rank)
        return out

    def load(self, tensors: Dict[str, torch.Tensor]) -> None:
        lib, allowed, n = self.env.lib, not getattr(self.env, "generic_only", False), self.names
        owns = self.cache_from is None
        pieces = [(tensors[n["dq"]], 0, None, None)] + ([(tensors[n["dkv"]], self.q_rank, None, None)] if owns else [])
        first = tensors[n["dq"]]
        rows = self.q_rank + ((self.kv_rank + self.rot) if owns else 0)
        self.gate_col = rows
        if self.has_gate:       # the gate's rows ride in the same product (behind the others, up to a multiple of 16 with zeros)
            g = tensors[n["gate"]]
            full = torch.zeros(((rows + self.heads + 15) // 16 * 16 - rows, self.hidden), dtype=g.dtype, device=g.device)
            full[:self.heads] = g
            pieces.append((full, rows, None, None))
            rows += full.shape[0]
        self.w_down = pack_rows(lib, pieces, rows, self.hidden, first.dtype, first.device, allowed)
        self.q_gain = tensors[n["dq_norm"]]
        self.kv_gain = tensors[n["dkv_norm"]] if owns else None
        uq, o = tensors[n["uq"]], tensors[n["o"]]
        self.w_uq = pack_rows(lib, [(uq, 0, None, None)], uq.shape[0], uq.shape[1], uq.dtype, uq.device, allowed)
        self.w_o = pack_rows(lib, [(o, 0, None, None)], o.shape[0], o.shape[1], o.dtype, o.device, allowed)
        # per head, stored [inner, outer]: Wuk_i [dim, rank] as it is (q_i -> Wuk_i^T q_i), Wuv_i transposed
        self.w_uk = tensors[n["uk"]].view(self.heads, self.dim, self.kv_rank).contiguous()
        self.w_uv = tensors[n["uv"]].view(self.heads, self.vdim, self.kv_rank).transpose(1, 2).contiguous()
        self.sink = tensors[n["sink"]] if self.has_sink else None

    def cache_request(self) -> Optional[CacheRequest]:
        if self.cache_from is not None:
            return None
        return CacheRequest("kv", heads=1, head_dim=self.page_width, window=None, values=False, name="latent")

    def forward(self, h: torch.Tensor, ctx, view, stream: Optional[torch.Tensor] = None, next_norm=None) -> torch.Tensor:
        lib, t, dt = self.env.lib, h.shape[0], self.env.dtype
        owns = self.cache_from is None
        down = linear(lib, h, self.w_down, torch.float32)                     # [T, q_rank (+ kv_rank)]
        cq = torch.empty((t, self.q_rank), dtype=dt, device=h.device)
        cos, sin, style = self.rot_tables
        r = self.page_width
        if self.rot:
            lib.latent_norm_rope_store(down, self.q_rank, self.q_gain, cq, self.kv_rank if owns else 0, self.kv_gain,
                                       view.k_pages if owns else None, self.rot, cos, sin, style, ctx, view.block_table, self.eps, dt)
        else:
            lib.latent_norm_store(down, self.q_rank, self.q_gain, cq, self.kv_rank if owns else 0, self.kv_gain,
                                  view.k_pages if owns else None, ctx, view.block_table, self.eps, dt)
        q = linear(lib, cq, self.w_uq, torch.float32)                         # [T, heads * (dim + rot)]
        ql = torch.empty((t, self.heads * r), dtype=dt, device=h.device)
        if self.rot:
            # the queries in the cache's layout: the unrotated part in the latent's space, then the rotated part, then zeros
            lib.heads_linear_part(q, self.dim + self.rot, self.w_uk, ql, r,
                                  rope=(self.dim, self.rot, cos, sin, style, self.kv_rank, ctx.tok_pos))
        else:
            lib.heads_linear(q, self.w_uk, ql)                                # the queries in the latent's space
        ol = torch.empty((t, self.heads * r), dtype=dt, device=h.device)
        q3, pages = ql.view(t, self.heads, r), view.k_pages
        fast = dt == torch.bfloat16 and r in _MATRIX_CORE_RANKS and not getattr(self.env, "generic_only", False)
        if fast and ctx.max_q_len == 1:      # more than 16 heads on the latent run as several groups of at most 16
            n_splits, workspace = ctx.decode_workspace(self.heads, r, 1)
            lib.attention_decode_bf16(q3, pages, pages, ol, ctx.tok_pos, view.block_table, self.heads, 1, r, self.scale, None,
                                      n_splits, workspace, sinks=self.sink)
        elif fast:
            lib.attention_prefill_bf16(q3, pages, pages, ol, ctx.cu_seqlens, ctx.past_len, view.block_table, ctx.n_seqs,
                                       ctx.max_q_len, self.heads, 1, r, self.scale, None, sinks=self.sink)
        else:
            lib.attention_sinks(q3, pages, pages, ol, ctx.tok_pos, ctx.tok_seq, view.block_table, self.heads, 1, r,
                                self.scale, None, self.sink)
        o = torch.empty((t, self.heads * self.vdim), dtype=dt, device=h.device)
        # the latent's part of every head's sum through the head's value matrix, the head's gate on the way out
        lib.heads_linear_part(ol, r, self.w_uv, o, self.vdim, gate=down if self.has_gate else None, gate_col=self.gate_col)
        return linear(lib, o, self.w_o, torch.float32)


register_mixer("latent_attention", LatentAttention)
