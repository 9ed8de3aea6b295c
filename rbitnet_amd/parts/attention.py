"""The attention mixer: grouped-query causal attention over the paged cache.

Reference, one token (crates/bitnet-core/src/llama/model.rs:238-294): q = Wq h, k = Wk h,
v = Wv h; rotate every q head and k head; store k (rotated) and v at the token's
position; for q head qh read kv head qh / (Hq / Hk); scores (q . k) * scale over the
keys up to the token's own position; softmax; weighted sum of v; heads concatenated;
out = Wo attn.  Here the same runs for all tokens of a step at once: keys and values
of the whole step are written to the cache first, then every token attends to the
cache up to its own position, so a step may bring any number of tokens per sequence
on top of any past.

Parameters: num_heads, num_kv_heads, head_dim, scale, window (None: all keys; n: the
last n keys including the token's own), position (a PartSpec), cache_from (None, or the
index of the layer whose cache this layer reads instead of keeping one), names (tensor
names of the matrices relative to the layer's prefix), and three that a plain decoder leaves out:
  value_dim   size of a value head where it is not head_dim;
  sink        True: a learned number per query head (tensor "sink") stands in the softmax's
              denominator as exp(sink): no key, no value, not scaled;
  head_gate   True: head h's output is multiplied by sigmoid(Wg h)_h (tensor "gate" [heads, E])
              before the output matrix.
and four more, each of which sends the layer through the kernels that take all heads of a token together:
  bias        True: q, k and v have biases (tensors named like the matrices with "_bias": names "q_bias", ...), added
              to the projections before anything else;
  qk_norm     None, or {"eps": e}: every query and key head is divided by sqrt(mean(head^2) + e) (no weight); the cache
              holds the keys as they are then;
  talk        True: the heads' scores are mixed before the softmax, score_h <- sum_g T[h, g] score_g, with T the tensor
              "talk" [heads, heads] (float32);
  chunk       None, or c: a query at position i sees the keys j <= i with i // c == j // c only, chunks being counted
              from the sequence's first position, whatever a step brings.
These go without a rotation (position "none") and without a sink.
Five more send the layer through a third way, in which q, k and v are prepared by kernels of their own in front of attention
(biases and a norm with a weight belong to it too, and a rotation is welcome):
  conv        None, or the taps of a short causal convolution over time on every channel of q, k and v (tensors "q_conv",
              "k_conv", "v_conv" [channels, taps], no bias), directly behind the projection and its bias; the last taps - 1
              projected rows of a sequence are part of its state;
  qk_norm     {"eps": e, "weight": True}: the norm of every query and key head has a weight of head_dim numbers that the heads
              share (tensors "q_norm", "k_norm"), x / sqrt(mean(x^2) + e) * w, before the rotation;
  softcap     None, or c: score <- c tanh(score / c) after the scale;
  keep_first  with a window: the first keep_first tokens of a sequence stay visible behind it (at their own positions);
  gate        "elementwise": the concatenated heads are multiplied number by number with sigmoid(Wg h) (tensor "gate"
              [heads * value_dim, E]) before the output matrix.
A position part that rotates only the first numbers of a head says so with its own head_dim
(the table's width).  Where keys and values differ in size, or only a part of a head is
rotated, queries, keys and values are laid out with one head size, the larger of the two,
the rest being zeros: the scores and the sums stay what they are and every attention kernel
made for one head size serves (keys of 64 beside values of 128 cost a third more cache
traffic than their own sizes would).

Interface of a mixer:
  tensor_specs() / load(tensors)
  cache_request() -> CacheRequest or None
  forward(h [T, E] compute dtype, ctx, view) -> float32 [T, E]
Two things a mixer may say of itself (this one does both):
  adds_to_stream: forward also takes stream=x (float32 [T, E], the residual stream) and
  next_norm (the norm that follows) and may add its result to the stream itself; it then returns
  None, or the GainedRows that its last product left for next_norm;
  takes_gained_rows: h may be such GainedRows instead of a tensor.
"""
from __future__ import annotations

from typing import Dict, Optional

import torch

from ..errors import ConfigError
from .base import BuildEnv, CacheRequest, Part, TensorSpec, build_part, register_mixer
from .linear import linear, linear_or_terms, linear_to_stream, pack_rows
from .short_conv import ACT_NONE, ShortConv

DEFAULT_NAMES = {"q": "q_proj.weight", "k": "k_proj.weight", "v": "v_proj.weight", "o": "o_proj.weight", "sink": "sink",
                 "gate": "gate", "q_bias": "q_proj.bias", "k_bias": "k_proj.bias", "v_bias": "v_proj.bias", "talk": "talk",
                 "q_conv": "q.conv", "k_conv": "k.conv", "v_conv": "v.conv", "q_norm": "q.norm", "k_norm": "k.norm"}
MIXED_MAX_HEADS, MIXED_MAX_NUMBERS = 64, 8192      # what the kernels that take all heads of a token together hold
MIXED_MATRIX_CORE_HEADS = 32                       # and the one on the matrix cores
_MATRIX_CORE_HEAD_DIMS = (64, 128)
_DECODE_GROUPS = tuple(range(1, 17))    # query heads per kv head the decode kernels take


class Attention(Part):
    graph_safe = True
    plan_safe = True
    takes_gained_rows = True
    adds_to_stream = True

    def __init__(self, params: Dict, env: BuildEnv):
        self.env = env
        self.n_heads = int(params["num_heads"])
        self.n_kv = int(params["num_kv_heads"])
        self.head_dim = int(params["head_dim"])
        if self.n_heads <= 0 or self.n_kv <= 0 or self.n_heads % self.n_kv != 0:
            raise ConfigError(f"attention: {self.n_heads} heads cannot share {self.n_kv} kv heads")
        if self.head_dim <= 0 or self.head_dim > 512:
            raise ConfigError(f"attention: head_dim {self.head_dim} not supported (at most 512)")
        self.value_dim = int(params.get("value_dim") or self.head_dim)
        if not 0 < self.value_dim <= 512:
            raise ConfigError(f"attention: value_dim {self.value_dim} not supported (1 to 512)")
        self.has_sink, self.has_gate = bool(params.get("sink")), bool(params.get("head_gate"))
        self.scale = float(params.get("scale") or self.head_dim ** -0.5)
        self.window = params.get("window")
        if self.window is not None and int(self.window) <= 0:
            raise ConfigError("attention: window must be positive")
        self.cache_from = params.get("cache_from")
        self.names = dict(DEFAULT_NAMES, **(params.get("names") or {}))
        self.position = build_part("position", params["position"], env)
        self.plan_safe = bool(getattr(self.position, "plan_safe", False))
        self.hidden = env.hidden_size
        # how many numbers of a head the position part rotates (its table's width; none: 0), and the one head size
        # that queries, keys and values are laid out with
        self.rot = int(getattr(self.position, "head_dim", 0)) if getattr(self.position, "rotation_tables", None) else 0
        if self.rot > self.head_dim:
            raise ConfigError(f"attention: {self.rot} rotated numbers in a head of {self.head_dim}")
        if self.rot % 2 != 0:
            raise ConfigError(f"attention: a rotation pairs the numbers of a head, {self.rot} of them cannot be paired")
        self.pad = max(self.head_dim, self.value_dim)
        self.same_sizes = self.value_dim == self.head_dim and self.rot in (0, self.head_dim) and self.head_dim % 2 == 0
        self.has_bias, self.has_talk = bool(params.get("bias")), bool(params.get("talk"))
        qk_norm = params.get("qk_norm")
        self.qk_eps = None if qk_norm is None else float(qk_norm["eps"])
        self.chunk = None if params.get("chunk") is None else int(params["chunk"])
        if self.chunk is not None and self.chunk <= 0:
            raise ConfigError("attention: chunk must be positive")
        # q, k and v prepared in front of attention: whenever one of these is asked for
        self.taps = None if params.get("conv") is None else int(params["conv"])
        self.qk_weight = bool(qk_norm and qk_norm.get("weight"))
        self.softcap = None if params.get("softcap") is None else float(params["softcap"])
        self.keep_first = int(params.get("keep_first") or 0)
        self.gate_kind = str(params.get("gate") or ("head" if self.has_gate else "none"))
        if self.gate_kind not in ("none", "head", "elementwise"):
            raise ConfigError(f"attention: unknown gate {self.gate_kind!r} (head, elementwise)")
        self.has_gate = self.gate_kind != "none"
        if self.softcap is not None and not self.softcap > 0:
            raise ConfigError("attention: softcap must be positive")
        if self.keep_first < 0 or (self.keep_first and self.window is None):
            raise ConfigError("attention: kept first tokens go with a window")
        self.prepared = bool(self.taps is not None or self.qk_weight or self.softcap is not None or self.keep_first
                             or self.gate_kind == "elementwise")
        if self.prepared and (self.has_talk or self.chunk is not None):
            raise ConfigError("attention: mixed heads and chunks go without a convolution, weighted norms, capped scores, "
                              "kept first tokens and an elementwise gate")
        self.conv = None
        if self.prepared and (self.taps is not None or self.has_bias):
            # a bias alone runs as a convolution of one tap (of ones): the same kernel adds it
            n_ch = self.n_heads * self.head_dim
            if self.cache_from is None:
                n_ch += self.n_kv * (self.head_dim + self.value_dim)
            self.conv = ShortConv(n_ch, self.taps or 1, env, residual=False, act=ACT_NONE)
        # all heads of a token in one workgroup: whenever one of the four is asked for
        self.mixed = (not self.prepared) and (self.has_bias or self.has_talk or self.qk_eps is not None or self.chunk is not None)
        if self.mixed:
            if self.rot or self.has_sink:
                raise ConfigError("attention: biases, unit heads, mixed heads and chunks go without a rotation and without a sink")
            if self.n_heads > MIXED_MAX_HEADS or self.n_heads * self.pad > MIXED_MAX_NUMBERS:
                raise ConfigError(f"attention: {self.n_heads} heads of {self.pad} numbers are more than the kernels that take all "
                                  f"heads of a token together hold ({MIXED_MAX_HEADS} heads, {MIXED_MAX_NUMBERS} numbers)")
        self.bias: Optional[torch.Tensor] = None
        self.talk: Optional[torch.Tensor] = None
        self.mixed_on_matrix_cores = False
        self.w_gate = None
        self.sink: Optional[torch.Tensor] = None
        self.w_qkv: Optional[torch.Tensor] = None
        self.w_q: Optional[torch.Tensor] = None
        self.w_o: Optional[torch.Tensor] = None

    # ------------------------------------------------------------------ tensors
    def tensor_specs(self) -> Dict[str, TensorSpec]:
        qd, kd = self.n_heads * self.head_dim, self.n_kv * self.head_dim
        specs = {self.names["q"]: TensorSpec((qd, self.hidden)),
                 self.names["o"]: TensorSpec((self.hidden, self.n_heads * self.value_dim))}
        if self.cache_from is None:
            specs[self.names["k"]] = TensorSpec((kd, self.hidden))
            specs[self.names["v"]] = TensorSpec((self.n_kv * self.value_dim, self.hidden))
        if self.has_bias:
            specs[self.names["q_bias"]] = TensorSpec((qd,), role="gain", init="normal")
            if self.cache_from is None:
                specs[self.names["k_bias"]] = TensorSpec((kd,), role="gain", init="normal")
                specs[self.names["v_bias"]] = TensorSpec((self.n_kv * self.value_dim,), role="gain", init="normal")
        if self.has_talk:
            specs[self.names["talk"]] = TensorSpec((self.n_heads, self.n_heads), role="gain", init="eye_normal")
        if self.has_sink:
            specs[self.names["sink"]] = TensorSpec((self.n_heads,), role="gain", init="normal")
        if self.has_gate:
            rows = self.n_heads * (self.value_dim if self.gate_kind == "elementwise" else 1)
            specs[self.names["gate"]] = TensorSpec((rows, self.hidden))
        if self.taps is not None:
            gain = lambda rows: TensorSpec((rows, self.taps), role="gain", init="normal")
            specs[self.names["q_conv"]] = gain(qd)
            if self.cache_from is None:
                specs[self.names["k_conv"]] = gain(kd)
                specs[self.names["v_conv"]] = gain(self.n_kv * self.value_dim)
        if self.qk_weight:
            specs[self.names["q_norm"]] = TensorSpec((self.head_dim,), role="gain", init="ones_normal")
            if self.cache_from is None:
                specs[self.names["k_norm"]] = TensorSpec((self.head_dim,), role="gain", init="ones_normal")
        return specs

    def load(self, tensors: Dict[str, torch.Tensor]) -> None:
        # q, k and v rows in one matrix: one product per step instead of three
        lib, allowed = self.env.lib, not getattr(self.env, "generic_only", False)
        names = ("q", "k", "v") if self.cache_from is None else ("q",)
        pieces, row = [], 0
        for n in names:
            t = tensors[self.names[n]]
            pieces.append((t, row, None, None))
            row += t.shape[0]
        first = pieces[0][0]
        self.w_qkv = pack_rows(lib, pieces, row, self.hidden, first.dtype, first.device, allowed)
        o = tensors[self.names["o"]]
        if self.value_dim < self.pad:
            # attention's output comes in heads of `pad` numbers whose last ones are zero: columns of zeros for them
            wide = torch.zeros((o.shape[0], self.n_heads, self.pad), dtype=o.dtype, device=o.device)
            wide[:, :, :self.value_dim] = o.view(o.shape[0], self.n_heads, self.value_dim)
            o = wide.view(o.shape[0], self.n_heads * self.pad)
        self.w_o = pack_rows(lib, [(o, 0, None, None)], o.shape[0], o.shape[1], o.dtype, o.device, allowed)
        if self.has_bias:
            self.bias = torch.cat([tensors[self.names[n + "_bias"]].reshape(-1) for n in names]).contiguous()
        if self.has_talk:
            self.talk = tensors[self.names["talk"]].contiguous()
        # the matrix cores' kernel: bfloat16, heads of 64 or 128 numbers, at most 32 of them; it wants a mixing matrix
        self.mixed_on_matrix_cores = bool(self.mixed and allowed and self.env.dtype == torch.bfloat16
                                          and self.pad in _MATRIX_CORE_HEAD_DIMS and self.n_heads <= MIXED_MATRIX_CORE_HEADS)
        if self.mixed_on_matrix_cores and self.talk is None:
            self.talk = torch.eye(self.n_heads, dtype=torch.float32, device=o.device)
        if self.has_sink:
            self.sink = tensors[self.names["sink"]]
        if self.gate_kind == "head":
            # rows up to a multiple of 16 (zeros), so that the product's kernels find whole tiles
            g = tensors[self.names["gate"]]
            rows = (self.n_heads + 15) // 16 * 16
            full = torch.zeros((rows, self.hidden), dtype=g.dtype, device=g.device)
            full[:self.n_heads] = g
            self.w_gate = pack_rows(lib, [(full, 0, None, None)], rows, self.hidden, g.dtype, g.device, allowed)
        elif self.gate_kind == "elementwise":
            # the gate's rows in the layout of attention's output: heads of `pad` numbers, zero rows behind a head's values
            g = tensors[self.names["gate"]]
            full = torch.zeros((self.n_heads, self.pad, self.hidden), dtype=g.dtype, device=g.device)
            full[:, :self.value_dim] = g.view(self.n_heads, self.value_dim, self.hidden)
            self.w_gate = pack_rows(lib, [(full.view(-1, self.hidden), 0, None, None)], self.n_heads * self.pad, self.hidden,
                                    g.dtype, g.device, allowed)
        if self.conv is not None:
            if self.taps is not None:
                self.conv.load(torch.cat([tensors[self.names[n + "_conv"]] for n in names]))
            else:
                self.conv.load(torch.ones((self.conv.channels, 1), dtype=torch.float32, device=o.device))
        if self.qk_weight:
            self.q_norm_w = tensors[self.names["q_norm"]]
            self.k_norm_w = tensors[self.names["k_norm"]] if self.cache_from is None else None
        elif self.prepared and self.qk_eps is not None:
            self.q_norm_w = self.k_norm_w = torch.ones(self.head_dim, dtype=torch.float32, device=o.device)

    def cache_request(self) -> Optional[CacheRequest]:
        if self.cache_from is not None:
            return None
        return CacheRequest("kv", heads=self.n_kv, head_dim=self.pad,
                            window=None if self.window is None else int(self.window), keep_first=self.keep_first)

    def cache_requests(self):
        out = [r for r in (self.cache_request(),) if r is not None]
        state = self.conv.cache_request("qkv_conv") if self.conv is not None else None
        return out + ([state] if state is not None else [])

    # ------------------------------------------------------------------ forward
    def _gate_and_project(self, attn, h, stream, next_norm):
        lib = self.env.lib
        if self.gate_kind == "head":
            logits = linear(lib, h, self.w_gate, torch.float32)
            lib.head_gate(attn, logits, 0, self.n_heads, self.pad)
        elif self.gate_kind == "elementwise":
            lib.sigmoid_gate(attn, linear(lib, h, self.w_gate, torch.float32))
        return linear_to_stream(lib, attn, self.w_o, stream, next_norm)

    def _forward_prepared(self, h, ctx, view, stream, next_norm):
        """Bias and convolution, norms with weights, rotation and the cache write by kernels of their own; attention with
        capped scores and kept first tokens; the gate."""
        lib = self.env.lib
        t, hq, hk, d = h.shape[0], self.n_heads, self.n_kv, self.pad
        owns = self.cache_from is None
        qkv = linear(lib, h, self.w_qkv, torch.float32)
        if self.conv is not None:
            qkv = self.conv.forward(qkv, ctx, view.states.get("qkv_conv"), torch.float32, bias=self.bias)
        q = torch.empty((t, hq, d), dtype=self.env.dtype, device=h.device)
        cos, sin, style = self.position.rotation_tables() if self.rot else (None, None, 1)
        if self.rot and style != 1:
            raise ConfigError("attention: a head prepared in front of attention pairs i with i + rot / 2 (style 'half')")
        k_pages, v_pages = (view.k_pages, view.v_pages) if owns else (None, None)
        if self.qk_eps is not None:
            lib.norm_rope_store(qkv, cos, sin, self.rot, self.q_norm_w, self.k_norm_w, self.qk_eps, q, k_pages, v_pages,
                                ctx.tok_pos, ctx.tok_seq, view.block_table, hq, hk, self.head_dim, self.value_dim, d)
        else:
            lib.rope_store(qkv, cos, sin, self.rot, q, k_pages, v_pages, ctx.tok_pos, ctx.tok_seq, view.block_table, hq, hk,
                           self.head_dim, self.value_dim, d)
        attn = torch.empty((t, hq * d), dtype=self.env.dtype, device=h.device)
        window = int(self.window) if self.window is not None else 0
        fast = (self.env.dtype == torch.bfloat16 and d in _MATRIX_CORE_HEAD_DIMS and not getattr(self.env, "generic_only", False))
        if fast and ctx.max_q_len == 1:
            n_splits, workspace = ctx.decode_workspace(hq, d, hk)
            lib.attention_decode_bf16(q, view.k_pages, view.v_pages, attn, ctx.tok_pos, view.block_table, hq, hk, d, self.scale,
                                      window, n_splits, workspace, sinks=self.sink, keep_first=self.keep_first,
                                      softcap=self.softcap or 0.0)
        elif fast:
            lib.attention_prefill_bf16(q, view.k_pages, view.v_pages, attn, ctx.cu_seqlens, ctx.past_len, view.block_table,
                                       ctx.n_seqs, ctx.max_q_len, hq, hk, d, self.scale, window, sinks=self.sink,
                                       keep_first=self.keep_first, softcap=self.softcap or 0.0)
        else:
            lib.attention_opts(q, view.k_pages, view.v_pages, attn, ctx.tok_pos, ctx.tok_seq, view.block_table, hq, hk, d,
                               self.scale, window, self.keep_first, self.softcap or 0.0, self.sink)
        return self._gate_and_project(attn, h, stream, next_norm)

    def _forward_mixed(self, h, ctx, view, stream, next_norm):
        """Biases, unit heads, the cache write, and attention with all heads of a token together."""
        lib = self.env.lib
        t, hq, hk, d = h.shape[0], self.n_heads, self.n_kv, self.pad
        owns = self.cache_from is None
        qkv = linear(lib, h, self.w_qkv, torch.float32)
        q = torch.empty((t, hq, d), dtype=self.env.dtype, device=h.device)
        lib.bias_norm_store(qkv, self.bias, self.qk_eps is not None, self.qk_eps or 0.0, q, view.k_pages if owns else None,
                            view.v_pages if owns else None, ctx.tok_pos, ctx.tok_seq, view.block_table, hq, hk, self.head_dim,
                            self.value_dim, d)
        attn = torch.empty((t, hq * d), dtype=self.env.dtype, device=h.device)
        window = int(self.window) if self.window is not None else 0
        if self.mixed_on_matrix_cores:
            # a step of single tokens: every sequence's pages dealt out to several workgroups; so are those of a prompt
            # whose 16-query tiles leave compute units idle (the last tiles of a prompt walk the most pages)
            if t == ctx.n_seqs:
                n_splits, ws = ctx.tile_split_workspace(hq, d)
            else:
                tiles = t // 16 + ctx.n_seqs
                n_splits = max(1, min(4, (lib.n_compute_units + tiles // 2) // tiles))
                ws = torch.empty(n_splits * t * hq * (d + 2), dtype=torch.float32, device=h.device) if n_splits > 1 else None
            lib.attention_mixed_bf16(q, view.k_pages, view.v_pages, attn, ctx, view.block_table, hq, hk, d, self.scale, self.talk,
                                     self.chunk or 0, window, n_splits, ws)
        else:
            lib.attention_mixed(q, view.k_pages, view.v_pages, attn, ctx.tok_pos, ctx.tok_seq, view.block_table, hq, hk, d,
                                self.scale, self.talk, self.chunk or 0, window)
        return self._gate_and_project(attn, h, stream, next_norm)

    def forward(self, h, ctx, view, stream: Optional[torch.Tensor] = None, next_norm=None):
        if self.prepared:
            if hasattr(h, "tensor") and not isinstance(h, torch.Tensor):
                h = h.tensor()
            return self._forward_prepared(h, ctx, view, stream, next_norm)
        if self.mixed:
            if hasattr(h, "tensor") and not isinstance(h, torch.Tensor):
                h = h.tensor()
            return self._forward_mixed(h, ctx, view, stream, next_norm)
        lib = self.env.lib
        t = h.shape[0]
        hq, hk, d = self.n_heads, self.n_kv, self.pad
        owns = self.cache_from is None
        # q, k and v of the step; as the terms of the product where the position part reads such
        if self.same_sizes and getattr(self.position, "takes_terms", False):
            qkv = linear_or_terms(lib, h, self.w_qkv)
        else:
            qkv = linear(lib, h, self.w_qkv, torch.float32)
        bt = view.block_table
        attn = torch.empty((t, hq * d), dtype=self.env.dtype, device=h.device)
        window = int(self.window) if self.window is not None else 0
        fast = (self.env.dtype == torch.bfloat16 and d in _MATRIX_CORE_HEAD_DIMS
                and not getattr(self.env, "generic_only", False))
        decode = fast and ctx.max_q_len == 1 and (hq // hk) in _DECODE_GROUPS
        tables = getattr(self.position, "rotation_tables", None)
        if decode and owns and tables is not None and self.same_sizes:
            # one kernel: rotation, cache write, attention over the pages
            cos, sin, style = tables()
            n_splits, workspace = ctx.decode_workspace(hq, d, hk)
            lib.attention_decode_fused_bf16(qkv, cos, sin, style, view.k_pages, view.v_pages, attn, ctx.tok_pos, bt,
                                            hq, hk, d, self.scale, window, n_splits, workspace, sinks=self.sink)
            return self._gate_and_project(attn, h, stream, next_norm)
        q = torch.empty((t, hq, d), dtype=self.env.dtype, device=h.device)
        if self.same_sizes:
            if owns:
                self.position.encode_and_store(qkv, q, view.k_pages, view.v_pages, ctx, bt, hq, hk, d)
            else:
                self.position.encode_and_store(qkv, q, None, None, ctx, bt, hq, 0, d)
        else:
            cos, sin, style = tables() if self.rot else (None, None, 1)
            if self.rot and style != 1:
                raise ConfigError("attention: a head rotated in part pairs i with i + rot / 2 (style 'half')")
            lib.rope_store(qkv, cos, sin, self.rot, q, view.k_pages if owns else None, view.v_pages if owns else None,
                           ctx.tok_pos, ctx.tok_seq, bt, hq, hk, self.head_dim, self.value_dim, d)
        if decode:
            n_splits, workspace = ctx.decode_workspace(hq, d, hk)
            lib.attention_decode_bf16(q, view.k_pages, view.v_pages, attn, ctx.tok_pos, bt, hq, hk, d,
                                      self.scale, window, n_splits, workspace, sinks=self.sink)
        elif fast:
            lib.attention_prefill_bf16(q, view.k_pages, view.v_pages, attn, ctx.cu_seqlens, ctx.past_len, bt,
                                       ctx.n_seqs, ctx.max_q_len, hq, hk, d, self.scale, window, sinks=self.sink)
        else:
            lib.attention_sinks(q, view.k_pages, view.v_pages, attn, ctx.tok_pos, ctx.tok_seq, bt, hq, hk, d,
                                self.scale, window, self.sink)
        return self._gate_and_project(attn, h, stream, next_norm)


register_mixer("attention", Attention)
