"""ctypes binding of librbitnet_hip.so: torch tensors in, kernels launched on torch's
current HIP stream.  There is no fallback: without a GPU and the built library every
call fails with a KernelError."""
from __future__ import annotations

import atexit
import ctypes
import os
import sys
import threading
from typing import Dict, List, Optional, Tuple

import torch

from ..errors import KernelError
from . import build as _build

_RAW_STREAM = getattr(torch._C, "_cuda_getCurrentRawStream", None)
_F32, _BF16 = 0, 1
_P = ctypes.c_void_p
_I = ctypes.c_int
_F = ctypes.c_float
_L = ctypes.c_longlong


def dtype_code(dtype: torch.dtype) -> int:
    if dtype == torch.float32:
        return _F32
    if dtype == torch.bfloat16:
        return _BF16
    raise KernelError(f"the kernels take float32 or bfloat16 storage, not {dtype}")


def _ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    if t is None:
        return None
    return t.data_ptr()


def _check(t: torch.Tensor, name: str, dtype=None, shape=None) -> None:
    if not t.is_cuda:
        raise KernelError(f"{name} must be on the GPU")
    if not t.is_contiguous():
        raise KernelError(f"{name} must be contiguous")
    if dtype is not None and t.dtype != dtype:
        raise KernelError(f"{name} must be {dtype}, found {t.dtype}")
    if shape is not None and tuple(t.shape) != tuple(shape):
        raise KernelError(f"{name} must have shape {tuple(shape)}, found {tuple(t.shape)}")


def _terms(qkv: torch.Tensor, width: int):
    """qkv [T, width], or [P, T, width]: P terms to be added up in their order.  -> (T, P, stride)"""
    if qkv.dim() == 3:
        p, n = qkv.shape[0], qkv.shape[1]
        _check(qkv, "qkv", torch.float32, (p, n, width))
        return n, p, n * width
    n = qkv.shape[0]
    _check(qkv, "qkv", torch.float32, (n, width))
    return n, 1, 0


class KernelTimes:
    """Time on the GPU per kernel wrapper, from events recorded around every call: the
    "wall time per token, then a profiler" checklist of the reference (docs/PROFILING.md:7-11)
    without leaving the process.  Switched on by RBITNET_KERNEL_TIMES=1 (the decode step is then
    launched kernel by kernel instead of replayed as a graph, so that every launch can be timed);
    the table goes to standard error when the process ends, or to whoever calls `report()`."""

    def __init__(self, by_shape: bool = False) -> None:
        """by_shape (RBITNET_KERNEL_TIMES=shapes): a row per wrapper and shapes of its first two
        tensors, so that the products of a layer can be told apart."""
        self.by_shape = by_shape
        self.events: Dict[str, List[Tuple[torch.cuda.Event, torch.cuda.Event]]] = {}

    def wrap(self, name: str, fn):
        def timed(*args, **kwargs):
            key = name
            if self.by_shape:
                shapes = [tuple(a.shape) for a in args if hasattr(a, "shape")][:2]
                key = f"{name} " + " x ".join("[" + ",".join(str(d) for d in sh) + "]" for sh in shapes)
            start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            start.record()
            try:
                return fn(*args, **kwargs)
            finally:
                end.record()
                self.events.setdefault(key, []).append((start, end))
        return timed

    def totals(self) -> Dict[str, Tuple[int, float]]:
        """name -> (calls, milliseconds); waits for the GPU."""
        torch.cuda.synchronize()
        return {name: (len(pairs), sum(a.elapsed_time(b) for a, b in pairs)) for name, pairs in self.events.items()}

    def reset(self) -> None:
        self.events.clear()

    def report(self) -> str:
        totals = self.totals()
        whole = sum(ms for _, ms in totals.values()) or 1.0
        width = max([32] + [len(name) for name in totals])
        lines = [f"{'kernel':{width}} {'calls':>8} {'total ms':>10} {'mean us':>9} {'share':>6}"]
        for name, (calls, ms) in sorted(totals.items(), key=lambda kv: -kv[1][1]):
            lines.append(f"{name:{width}} {calls:8d} {ms:10.3f} {ms * 1e3 / max(1, calls):9.1f} {ms / whole:6.1%}")
        return "\n".join(lines)


TIMED_OPS = ("short_conv_bias", "decay_exp_exp", "gated_rmsnorm_heads", "outnorm_residual", "clamped_glu", "tanh_cast", "attention_opts", "norm_rope_store", "sigmoid_gate", "shift_mix", "time_mix_recurrence", "latent_norm_rope_store", "heads_linear_part", "route_choose", "experts_combine", "embed_scaled_pos", "scale", "bias_norm_store", "attention_mixed", "attention_mixed_bf16", "recurrence_prep", "linear_recurrence", "layernorm_residual", "rope_store", "head_gate", "pair_norm_mean",
             "route_top", "routed_experts", "pairs_sum", "embed_streams", "streams_layernorm", "streams_update", "xielu", "tanh_cap", "short_conv",
             "delta_prep", "delta_rule", "gated_rmsnorm", "latent_norm_store", "heads_linear", "attention_sinks", "embed_gather", "add_rmsnorm", "rope_kv_write", "swiglu", "gemm_generic", "gemm_bf16", "gemm_bf16_terms",
             "gemm_bf16_few", "attention_generic", "attention_prefill_bf16", "attention_decode_bf16",
             "attention_decode_fused_bf16", "sample")


class Kernels:
    """The loaded library.  Methods check operand shapes on the host before a launch, so
    that a kernel never sees sizes other than the ones its grid assumes."""

    def __init__(self, path: Optional[str] = None):
        if not torch.cuda.is_available():
            raise KernelError("no GPU visible: rbitnet_amd runs on an MI355X (gfx950) only and has no CPU fallback")
        path = path or _build.ensure_built()
        try:
            self._lib = ctypes.CDLL(path)
        except OSError as e:
            raise KernelError(f"cannot load the HIP kernel library {path}: {e}") from None
        self.path = path
        L = self._lib
        L.rb_last_error.restype = ctypes.c_char_p
        sig = {
            "rb_embed_gather": [_P, _I, _P, _P, _I, _I, _P],
            "rb_add_rmsnorm": [_P, _P, _I, ctypes.c_longlong, _P, _F, _P, _I, _I, _P, _I, _P],
            "rb_rope_kv_write": [_P, _I, ctypes.c_longlong, _P, _P, _I, _P, _P, _P, _I, _P, _P, _P, _I, _I, _I, _I, _I, _P],
            "rb_swiglu": [_P, _P, _I, _I, _I, _P],
            "rb_gemm_generic": [_P, _P, _I, _P, _I, _I, _I, _I, _I, _P],
            "rb_gemm_bf16": [_P, _P, _I, _P, _I, _I, _I, _I, _I, _P, _P],
            "rb_gemm_bf16_act": [_P, _P, _I, _P, _I, _I, _P, _I, _I, _I, _P, _P],
            "rb_gemm_bf16_few": [_P, _P, _F, _P, _P, _I, _P, _I, _I, _P, _P, _P, _I, _I, _I, _P],
            "rb_gemm_bf16_few_ok": [_I, _I, _I],
            "rb_gemm_bf16_terms_count": [_I, _I, _I],
            "rb_gemm_bf16_terms": [_P, _P, _I, _P, _I, _I, _I, _P],
            "rb_attention_generic": [_P, _P, _P, _P, _I, _P, _P, _P, _I, _I, _I, _I, _I, _F, _I, _P],
            "rb_attention_prefill_bf16": [_P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _F, _I, _P],
            "rb_attention_decode_bf16": [_P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _F, _I, _I, _P, _P],
            "rb_attention_decode_fused_bf16": [_P, _I, ctypes.c_longlong, _P, _P, _I, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _F, _I, _I,
                                               _P, _P],
            "rb_attention_decode_fused_bf16_sinks": [_P, _I, ctypes.c_longlong, _P, _P, _I, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I,
                                                     _F, _I, _I, _P, _P, _P],
            "rb_sample": [_P, _I, _I, _P, _P, _P, _P, _P],
            "rb_fill_normal": [_P, _I, ctypes.c_longlong, ctypes.c_ulonglong, ctypes.c_double, ctypes.c_double, _P],
            "rb_place_rows": [_P, _I, _P, _I, _I] + [ctypes.c_longlong] * 6 + [_P],
            "rb_probe_read": [_P, ctypes.c_longlong, _I, _I, _P, _P],
            "rb_probe_mfma": [_I, _I, _P, _P],
            "rb_attention_generic_sinks": [_P, _P, _P, _P, _I, _P, _P, _P, _I, _I, _I, _I, _I, _F, _I, _P, _P],
            "rb_attention_prefill_bf16_sinks": [_P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _F, _I, _P, _P],
            "rb_attention_decode_bf16_sinks": [_P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _F, _I, _I, _P, _P, _P],
            "rb_embed_streams": [_P, _I, _P, _P, _I, _L, _I, _I, _P],
            "rb_streams_layernorm": [_P, _I, _L, _P, _P, _P, _P, _F, _P, _I, _I, _P, _I, _P],
            "rb_streams_update_layernorm": [_P, _I, _L, _P, _P, _P, _P, _P, _P, _P, _P, _F, _P, _I, _I, _P, _I, _P],
            "rb_streams_update": [_P, _I, _L, _P, _P, _P, _P, _I, _I, _P],
            "rb_xielu": [_P, _P, _P, _I, _L, _P],
            "rb_tanh_cap": [_P, _F, _L, _P],
            "rb_short_conv": [_P, _L, _P, _I, _P, _P, _P, _P, _P, _P, _L, _I, _I, _I, _I, _I, _I, _P],
            "rb_delta_prep": [_P, _L, _I, _I, _P, _L, _P, _P, _I, _P, _L, _P, _F, _F, _I, _P],
            "rb_delta_rule": [_P, _P, _L, _P, _L, _P, _L, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _P],
            "rb_gated_rmsnorm": [_P, _P, _P, _L, _F, _P, _I, _I, _I, _I, _P],
            "rb_latent_norm_store": [_P, _L, _I, _P, _P, _I, _I, _P, _P, _I, _P, _P, _P, _I, _F, _I, _P],
            "rb_heads_linear": [_P, _I, _P, _I, _P, _I, _I, _I, _I, _I, _P],
            "rb_recurrence_prep": [_P, _L, _I, _I, _I, _F, _F, _P, _L, _I, _I, _P, _P, _F, _I, _P, _L, _P, _I, _P],
            "rb_linear_recurrence": [_P, _P, _L, _P, _L, _P, _L, _I, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _P],
            "rb_gated_rmsnorm_act": [_P, _P, _P, _L, _I, _F, _P, _I, _I, _I, _I, _P],
            "rb_layernorm_residual": [_P, _P, _P, _F, _P, _P, _F, _P, _I, _I, _P, _I, _P],
            "rb_rope_store": [_P, _L, _P, _P, _I, _P, _P, _P, _I, _P, _P, _P, _I, _I, _I, _I, _I, _I, _I, _P],
            "rb_head_gate": [_P, _I, _P, _L, _I, _I, _I, _P],
            "rb_pair_norm_mean": [_P, _P, _P, _P, _F, _P, _I, _I, _P],
            "rb_route_top": [_P, _L, _I, _I, _P, _P, _P, _P, _I, _I, _P],
            "rb_routed_experts": [_P, _I, _P, _I, _P, _P, _I, _P, _P, _P, _I, _P, _P, _I, _I, _I, _F, _F, _P],
            "rb_pairs_sum": [_P, _I, _P, _I, _I, _P],
            "rb_route_choose": [_P, _L, _I, _I, _I, _I, _P, _P, _P, _P, _P, _I, _I, _P],
            "rb_experts_combine": [_P, _P, _P, _I, _I, _P, _I, _P, _P, _L, _P, _I, _I, _P],
            "rb_embed_scaled_pos": [_P, _I, _P, _F, _P, _P, _P, _I, _I, _P],
            "rb_scale": [_P, _F, _L, _P],
            "rb_bias_norm_store": [_P, _L, _P, _I, _F, _P, _P, _P, _I, _P, _P, _P, _I, _I, _I, _I, _I, _I, _I, _P],
            "rb_outnorm_residual": [_P, _P, _P, _F, _F, _P, _F, _I, _P, _I, _I, _I, _P],
            "rb_clamped_glu": [_P, _P, _I, _I, _I, _F, _F, _P],
            "rb_tanh_cast": [_P, _P, _I, _L, _P],
            "rb_attention_prefill_bf16_opts": [_P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _F, _I, _I, _F, _P, _P],
            "rb_attention_decode_bf16_opts": [_P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _F, _I, _I, _F, _I, _P, _P, _P],
            "rb_attention_generic_opts": [_P, _P, _P, _P, _I, _P, _P, _P, _I, _I, _I, _I, _I, _F, _I, _I, _F, _P, _P],
            "rb_norm_rope_store": [_P, _L, _P, _P, _I, _P, _P, _F, _P, _P, _P, _I, _P, _P, _P, _I, _I, _I, _I, _I, _I, _I, _P],
            "rb_sigmoid_gate": [_P, _I, _P, _L, _P],
            "rb_shift_mix": [_P, _I, _P, _P, _I, _P, _P, _P, _P, _I, _I, _I, _P],
            "rb_short_conv_bias": [_P, _L, _P, _P, _I, _P, _P, _P, _P, _P, _P, _L, _I, _I, _I, _I, _I, _I, _P],
            "rb_linear_recurrence_bonus": [_P, _P, _L, _P, _L, _P, _L, _I, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _P],
            "rb_gated_rmsnorm_heads": [_P, _P, _L, _P, _L, _I, _F, _P, _I, _I, _I, _I, _P],
            "rb_heads_linear_more": [_P, _I, _L, _P, _I, _P, _I, _L, _I, _I, _I, _I, _P, _L, _I, _I, _I, _P, _P, _I, _P, _P],
            "rb_heads_linear_strided": [_P, _I, _L, _P, _I, _P, _I, _L, _I, _I, _I, _I, _P],
            "rb_latent_norm_rope_store": [_P, _L, _I, _P, _P, _I, _I, _P, _P, _I, _I, _I, _P, _P, _I, _I, _P, _P, _P, _I, _F, _I, _P],
            "rb_attention_mixed": [_P, _P, _P, _P, _I, _P, _P, _P, _I, _I, _I, _I, _I, _F, _P, _I, _I, _P],
            "rb_attention_mixed_bf16": [_P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _F, _P, _I, _I, _I, _P, _P],
        }
        for name, args in sig.items():
            fn = getattr(L, name)
            fn.argtypes = args
            fn.restype = _I
        L.rb_plan_begin.argtypes, L.rb_plan_begin.restype = [], _P
        L.rb_plan_end.argtypes, L.rb_plan_end.restype = [_P], _I
        L.rb_plan_calls.argtypes, L.rb_plan_calls.restype = [_P], _I
        L.rb_plan_replay.argtypes, L.rb_plan_replay.restype = [_P, _P], _I
        L.rb_plan_free.argtypes, L.rb_plan_free.restype = [_P], None
        L.rb_gemm_workspace_floats.argtypes = [_I, _I, _I, _I]
        L.rb_gemm_workspace_floats.restype = ctypes.c_longlong
        L.rb_sample_workspace_bytes.argtypes = [_I, _I]
        L.rb_sample_workspace_bytes.restype = _I
        self.page_size = int(L.rb_page_size())
        self.times: Optional[KernelTimes] = None
        if os.environ.get("RBITNET_KERNEL_TIMES", "") in ("1", "true", "yes", "shapes"):
            self.times = KernelTimes(by_shape=os.environ["RBITNET_KERNEL_TIMES"] == "shapes")
            for name in TIMED_OPS:
                setattr(self, name, self.times.wrap(name, getattr(self, name)))
            atexit.register(lambda: print(self.times.report(), file=sys.stderr, flush=True))
        self.device_index = int(torch.cuda.current_device())
        self.n_compute_units = int(torch.cuda.get_device_properties(torch.cuda.current_device()).multi_processor_count)

    # ------------------------------------------------------------------ helpers
    def _stream(self) -> int:
        """torch's current HIP stream of this GPU, as a raw handle.  Asked for at every launch (a
        step that is being captured runs on another stream than the one before it), through torch's
        own fast path where it has one: `torch.cuda.current_stream()` builds a Python object at
        8 us a call, a third of what a launch costs on the host."""
        if _RAW_STREAM is not None:
            return _RAW_STREAM(self.device_index)
        return torch.cuda.current_stream().cuda_stream

    def _ok(self, rc: int) -> None:
        if rc != 0:
            raise KernelError(self._lib.rb_last_error().decode("utf-8", "replace"))

    # ------------------------------------------------------------------ ops
    def embed_gather(self, table: torch.Tensor, ids: torch.Tensor, out: torch.Tensor) -> None:
        n, width = out.shape
        _check(table, "table")
        _check(ids, "ids", torch.int32, (n,))
        _check(out, "out", torch.float32)
        if table.shape[1] != width:
            raise KernelError("embedding width mismatch")
        self._ok(self._lib.rb_embed_gather(_ptr(table), dtype_code(table.dtype), _ptr(ids), _ptr(out), n, width,
                                           self._stream()))

    def add_rmsnorm(self, x: torch.Tensor, delta: Optional[torch.Tensor], gain: torch.Tensor, eps: float,
                    rows: Optional[torch.Tensor], out: torch.Tensor) -> None:
        n_rows, width = out.shape
        _check(x, "x", torch.float32)
        if x.shape[1] != width:
            raise KernelError("norm width mismatch")
        n_terms, term_stride = 1, 0
        if delta is not None:
            if delta.dim() == 3:            # several terms, to be added up first
                n_terms, term_stride = delta.shape[0], x.numel()
                _check(delta, "delta", torch.float32, (n_terms,) + tuple(x.shape))
            else:
                _check(delta, "delta", torch.float32, x.shape)
        _check(gain, "gain", torch.float32, (width,))
        if rows is not None:
            _check(rows, "rows", torch.int32, (n_rows,))
        elif x.shape[0] != n_rows:
            raise KernelError("norm row count mismatch")
        _check(out, "out")
        self._ok(self._lib.rb_add_rmsnorm(_ptr(x), _ptr(delta), n_terms, term_stride, _ptr(gain), float(eps),
                                          _ptr(rows), n_rows, width, _ptr(out), dtype_code(out.dtype),
                                          self._stream()))

    def rope_kv_write(self, qkv, cos, sin, style, q_out, k_pages, v_pages, tok_pos, tok_seq, block_table,
                      n_heads, n_kv, head_dim) -> None:
        n, n_terms, term_stride = _terms(qkv, (n_heads + 2 * n_kv) * head_dim)
        _check(q_out, "q_out", None, (n, n_heads, head_dim))
        _check(tok_pos, "tok_pos", torch.int32, (n,))
        _check(tok_seq, "tok_seq", torch.int32, (n,))
        _check(block_table, "block_table", torch.int32)
        if cos is not None:
            _check(cos, "cos", torch.float32)
            _check(sin, "sin", torch.float32, cos.shape)
            if cos.shape[1] != head_dim // 2:
                raise KernelError("angle table width mismatch")
        if k_pages is not None:
            _check(k_pages, "k_pages", q_out.dtype)
            _check(v_pages, "v_pages", q_out.dtype, k_pages.shape)
            if tuple(k_pages.shape[1:]) != (n_kv, self.page_size, head_dim):
                raise KernelError(f"cache pages have shape {tuple(k_pages.shape)}, expected "
                                  f"[*, {n_kv}, {self.page_size}, {head_dim}]")
        self._ok(self._lib.rb_rope_kv_write(_ptr(qkv), n_terms, term_stride, _ptr(cos), _ptr(sin), int(style),
                                            _ptr(q_out), _ptr(k_pages), _ptr(v_pages), dtype_code(q_out.dtype),
                                            _ptr(tok_pos), _ptr(tok_seq),
                                            _ptr(block_table), block_table.shape[1], n, n_heads, n_kv, head_dim,
                                            self._stream()))

    def swiglu(self, gu: torch.Tensor, out: torch.Tensor) -> None:
        n, ff = out.shape
        _check(gu, "gu", torch.float32, (n, 2 * ff))
        _check(out, "out")
        self._ok(self._lib.rb_swiglu(_ptr(gu), _ptr(out), dtype_code(out.dtype), n, ff, self._stream()))

    def gemm_generic(self, a: torch.Tensor, w: torch.Tensor, c: torch.Tensor, w_frag: bool = False) -> None:
        """w_frag: w [N, K] (float32) is stored fragment-major (`place_rows(..., frag=True)` writes that)."""
        m, k = a.shape
        n = w.shape[0]
        _check(a, "a")
        _check(w, "w", a.dtype, (n, k))
        _check(c, "c", None, (m, n))
        self._ok(self._lib.rb_gemm_generic(_ptr(a), _ptr(w), int(bool(w_frag)), _ptr(c), dtype_code(a.dtype),
                                           dtype_code(c.dtype), m, n, k, self._stream()))

    def gemm_bf16(self, a: torch.Tensor, w: torch.Tensor, c: torch.Tensor, epilogue: int = 0,
                  w_frag: bool = False, act: Optional[torch.Tensor] = None) -> None:
        """w_frag: w [N, K] is stored fragment-major (`place_rows(..., frag=True)` writes that).
        act (epilogue 0): the two numbers of xIELU, float32 [2]; the result is xIELU(a w^T).  act (epilogue 1): the gated
        pair's limit and alpha, float32 [2]; the result is g sigmoid(alpha g) (u + 1) with g and u limited."""
        m, k = a.shape
        n = w.shape[0]
        _check(a, "a", torch.bfloat16)
        _check(w, "w", torch.bfloat16, (n, k))
        _check(c, "c", None, (m, n // 2 if epilogue == 1 else n))
        need = int(self._lib.rb_gemm_workspace_floats(m, n, k, int(epilogue)))
        workspace = torch.empty(need, dtype=torch.float32, device=a.device) if need else None
        if act is not None:
            _check(act, "act", torch.float32, (2,))
            if epilogue not in (0, 1):
                raise KernelError("gemm_bf16: an activation goes with epilogue 0, a gate's numbers with epilogue 1")
        self._ok(self._lib.rb_gemm_bf16_act(_ptr(a), _ptr(w), int(bool(w_frag)), _ptr(c), dtype_code(c.dtype), int(epilogue),
                                            _ptr(act), m, n, k, _ptr(workspace), self._stream()))

    def gemm_bf16_terms_count(self, m: int, n: int, k: int) -> int:
        return int(self._lib.rb_gemm_bf16_terms_count(int(m), int(n), int(k)))

    def gemm_bf16_terms(self, a: torch.Tensor, w: torch.Tensor, w_frag: bool = False) -> torch.Tensor:
        """a w^T as float32 terms [P, M, N] to be added up in their order: what the K slices of
        the kernel for these sizes computed (P = 1: the product itself)."""
        m, k = a.shape
        n = w.shape[0]
        _check(a, "a", torch.bfloat16)
        _check(w, "w", torch.bfloat16, (n, k))
        terms = torch.empty((int(self._lib.rb_gemm_bf16_terms_count(m, n, k)), m, n), dtype=torch.float32,
                            device=a.device)
        self._ok(self._lib.rb_gemm_bf16_terms(_ptr(a), _ptr(w), int(bool(w_frag)), _ptr(terms), m, n, k, self._stream()))
        return terms

    def gemm_bf16_few_ok(self, m: int, n: int, k: int) -> bool:
        """Whether gemm_bf16_few takes these sizes (1..16 tokens)."""
        return bool(self._lib.rb_gemm_bf16_few_ok(int(m), int(n), int(k)))

    def gemm_bf16_few(self, a: torch.Tensor, w: torch.Tensor, c: torch.Tensor, epilogue: int = 0,
                      squares: Optional[torch.Tensor] = None, eps: float = 0.0, rows: Optional[torch.Tensor] = None,
                      gain: Optional[torch.Tensor] = None, gained: Optional[torch.Tensor] = None,
                      squares_out: Optional[torch.Tensor] = None, w_frag: bool = False) -> None:
        """The product of 1..16 tokens with its neighbours folded in.
        squares [*, ceil(K / 16)]: a holds rows times a norm's gain and squares the sums of squares
        of the rows themselves; the product is scaled to that of the RMS-normalised rows (eps).
        rows: the tokens are these rows of a (and of squares).
        epilogue 2: c (float32) += product.  epilogue 3: the same, and gained [M, N] =
        bf16(c * gain), squares_out [M, ceil(N / 16)] = sums of c^2, for the norm that follows."""
        n, k = w.shape
        _check(a, "a", torch.bfloat16)
        if a.dim() != 2 or a.shape[1] != k:
            raise KernelError(f"a must have rows of {k} values, found {tuple(a.shape)}")
        m = a.shape[0] if rows is None else rows.shape[0]
        if rows is not None:
            _check(rows, "rows", torch.int32, (m,))
        if squares is not None:
            _check(squares, "squares", torch.float32, (a.shape[0], (k + 15) // 16))
        _check(w, "w", torch.bfloat16, (n, k))
        _check(c, "c", torch.float32 if epilogue >= 2 else None, (m, n // 2 if epilogue == 1 else n))
        if epilogue == 3:
            _check(gain, "gain", torch.float32, (n,))
            _check(gained, "gained", torch.bfloat16, (m, n))
            _check(squares_out, "squares_out", torch.float32, (m, (n + 15) // 16))
        self._ok(self._lib.rb_gemm_bf16_few(_ptr(a), _ptr(squares), float(eps), _ptr(rows), _ptr(w), int(bool(w_frag)),
                                            _ptr(c), dtype_code(c.dtype), int(epilogue), _ptr(gain), _ptr(gained),
                                            _ptr(squares_out), m, n, k, self._stream()))

    def attention_generic(self, q, k_pages, v_pages, out, tok_pos, tok_seq, block_table, n_heads, n_kv, head_dim,
                          scale, window) -> None:
        n = q.shape[0]
        _check(q, "q", None, (n, n_heads, head_dim))
        _check(k_pages, "k_pages", q.dtype)
        _check(v_pages, "v_pages", q.dtype, k_pages.shape)
        if tuple(k_pages.shape[1:]) != (n_kv, self.page_size, head_dim):
            raise KernelError("cache pages do not match the head counts")
        _check(out, "out", q.dtype, (n, n_heads * head_dim))
        _check(tok_pos, "tok_pos", torch.int32, (n,))
        _check(tok_seq, "tok_seq", torch.int32, (n,))
        _check(block_table, "block_table", torch.int32)
        self._ok(self._lib.rb_attention_generic(_ptr(q), _ptr(k_pages), _ptr(v_pages), _ptr(out), dtype_code(q.dtype),
                                                _ptr(tok_pos), _ptr(tok_seq), _ptr(block_table),
                                                block_table.shape[1], n, n_heads, n_kv, head_dim, float(scale),
                                                int(window or 0), self._stream()))

    def attention_prefill_bf16(self, q, k_pages, v_pages, out, cu_seqlens, past_len, block_table, n_seqs,
                               max_q_len, n_heads, n_kv, head_dim, scale, window, sinks=None, keep_first: int = 0,
                               softcap: float = 0.0) -> None:
        n = q.shape[0]
        _check(q, "q", torch.bfloat16, (n, n_heads, head_dim))
        _check(k_pages, "k_pages", torch.bfloat16)
        _check(v_pages, "v_pages", torch.bfloat16, k_pages.shape)
        if tuple(k_pages.shape[1:]) != (n_kv, self.page_size, head_dim):
            raise KernelError("cache pages do not match the head counts")
        _check(out, "out", torch.bfloat16, (n, n_heads * head_dim))
        _check(cu_seqlens, "cu_seqlens", torch.int32, (n_seqs + 1,))
        _check(past_len, "past_len", torch.int32, (n_seqs,))
        _check(block_table, "block_table", torch.int32)
        if sinks is not None:
            _check(sinks, "sinks", torch.float32, (n_heads,))
        self._ok(self._lib.rb_attention_prefill_bf16_opts(_ptr(q), _ptr(k_pages), _ptr(v_pages), _ptr(out),
                                                          _ptr(cu_seqlens), _ptr(past_len), _ptr(block_table),
                                                          block_table.shape[1], n_seqs, int(max_q_len), n_heads, n_kv,
                                                          head_dim, float(scale), int(window or 0), int(keep_first or 0),
                                                          float(softcap or 0.0), _ptr(sinks), self._stream()))

    def attention_decode_bf16(self, q, k_pages, v_pages, out, tok_pos, block_table, n_heads, n_kv, head_dim,
                              scale, window, n_splits, workspace, sinks=None, keep_first: int = 0, softcap: float = 0.0) -> None:
        n = q.shape[0]
        _check(q, "q", torch.bfloat16, (n, n_heads, head_dim))
        _check(k_pages, "k_pages", torch.bfloat16)
        _check(v_pages, "v_pages", torch.bfloat16, k_pages.shape)
        if tuple(k_pages.shape[1:]) != (n_kv, self.page_size, head_dim):
            raise KernelError("cache pages do not match the head counts")
        _check(out, "out", torch.bfloat16, (n, n_heads * head_dim))
        _check(tok_pos, "tok_pos", torch.int32, (n,))
        _check(block_table, "block_table", torch.int32)
        _check(workspace, "workspace", torch.float32)
        if workspace.numel() < n * n_heads * n_splits * (head_dim + 2):
            raise KernelError("decode attention workspace too small")
        if sinks is not None:
            _check(sinks, "sinks", torch.float32, (n_heads,))
        if keep_first or softcap or n_heads // n_kv > 16:        # this entry point also runs more than 16 heads on a kv head, in groups
            self._ok(self._lib.rb_attention_decode_bf16_opts(_ptr(q), _ptr(k_pages), _ptr(v_pages), _ptr(out), _ptr(tok_pos),
                                                             _ptr(block_table), block_table.shape[1], n, n_heads, n_kv,
                                                             head_dim, float(scale), int(window or 0), int(keep_first or 0),
                                                             float(softcap or 0.0), int(n_splits), _ptr(workspace), _ptr(sinks),
                                                             self._stream()))
            return
        self._ok(self._lib.rb_attention_decode_bf16_sinks(_ptr(q), _ptr(k_pages), _ptr(v_pages), _ptr(out), _ptr(tok_pos),
                                                          _ptr(block_table), block_table.shape[1], n, n_heads, n_kv,
                                                          head_dim, float(scale), int(window or 0), int(n_splits),
                                                          _ptr(workspace), _ptr(sinks), self._stream()))

    def attention_decode_fused_bf16(self, qkv, cos, sin, style, k_pages, v_pages, out, tok_pos, block_table,
                                    n_heads, n_kv, head_dim, scale, window, n_splits, workspace, sinks=None) -> None:
        n, n_terms, term_stride = _terms(qkv, (n_heads + 2 * n_kv) * head_dim)
        if cos is not None:
            _check(cos, "cos", torch.float32)
            _check(sin, "sin", torch.float32, cos.shape)
            if cos.shape[1] != head_dim // 2:
                raise KernelError("angle table width mismatch")
        _check(k_pages, "k_pages", torch.bfloat16)
        _check(v_pages, "v_pages", torch.bfloat16, k_pages.shape)
        if tuple(k_pages.shape[1:]) != (n_kv, self.page_size, head_dim):
            raise KernelError("cache pages do not match the head counts")
        _check(out, "out", torch.bfloat16, (n, n_heads * head_dim))
        _check(tok_pos, "tok_pos", torch.int32, (n,))
        _check(block_table, "block_table", torch.int32)
        _check(workspace, "workspace", torch.float32)
        if workspace.numel() < n * n_heads * n_splits * (head_dim + 2):
            raise KernelError("decode attention workspace too small")
        if sinks is not None:
            _check(sinks, "sinks", torch.float32, (n_heads,))
        self._ok(self._lib.rb_attention_decode_fused_bf16_sinks(
            _ptr(qkv), n_terms, term_stride, _ptr(cos), _ptr(sin), int(style), _ptr(k_pages), _ptr(v_pages), _ptr(out),
            _ptr(tok_pos),
            _ptr(block_table), block_table.shape[1], n, n_heads, n_kv, head_dim, float(scale), int(window or 0),
            int(n_splits), _ptr(workspace), _ptr(sinks), self._stream()))

    def sample(self, logits: torch.Tensor, temperature: Optional[torch.Tensor], u: Optional[torch.Tensor],
               tokens: torch.Tensor, workspace: Optional[torch.Tensor] = None) -> None:
        n, vocab = logits.shape
        _check(logits, "logits", torch.float32)
        if temperature is not None:
            _check(temperature, "temperature", torch.float32, (n,))
            _check(u, "u", torch.float32, (n,))
        _check(tokens, "tokens", torch.int32, (n,))
        need = int(self._lib.rb_sample_workspace_bytes(n, vocab))
        if workspace is None:
            workspace = torch.empty((need + 7) // 8, dtype=torch.int64, device=logits.device)
        _check(workspace, "workspace", torch.int64)
        if workspace.numel() * 8 < need:
            raise KernelError("sampling workspace too small")
        self._ok(self._lib.rb_sample(_ptr(logits), n, vocab, _ptr(temperature), _ptr(u), _ptr(tokens),
                                     _ptr(workspace), self._stream()))

    # ------------------------------------------------------------------ streams, layer norm, activations
    def embed_streams(self, table: torch.Tensor, ids: torch.Tensor, x: torch.Tensor) -> None:
        """x [S, T, E] float32: every copy s gets table[ids[t]] in row t."""
        s_, n, width = x.shape
        _check(table, "table")
        _check(ids, "ids", torch.int32, (n,))
        _check(x, "x", torch.float32)
        if table.shape[1] != width:
            raise KernelError("embedding width mismatch")
        self._ok(self._lib.rb_embed_streams(_ptr(table), dtype_code(table.dtype), _ptr(ids), _ptr(x), s_, n * width, n, width,
                                            self._stream()))

    def streams_layernorm(self, x: torch.Tensor, coef: Optional[torch.Tensor], weight: torch.Tensor,
                          bias: Optional[torch.Tensor], eps: float, rows: Optional[torch.Tensor], out: torch.Tensor,
                          delta: Optional[torch.Tensor] = None, update=None) -> None:
        """x [S, T, E] (or [T, E]: one stream) float32; out [rows or T, E]: the layer norm of sum_s coef[s] x[s].
        update (mix [S, S], out_coef [S], y [T, E], scale [E] or None): `streams_update` with these first, in the same
        pass (every row, so rows must be None)."""
        if x.dim() == 2:
            x = x.unsqueeze(0)
        s_, n, width = x.shape
        _check(x, "x", torch.float32)
        if coef is not None:
            _check(coef, "coef", torch.float32, (s_,))
        _check(weight, "weight", torch.float32, (width,))
        if bias is not None:
            _check(bias, "bias", torch.float32, (width,))
        if delta is not None:
            _check(delta, "delta", torch.float32, (n, width))
        n_rows = n
        if rows is not None:
            n_rows = rows.shape[0]
            _check(rows, "rows", torch.int32, (n_rows,))
        _check(out, "out", None, (n_rows, width))
        mix = out_coef = y = scale = None
        if update is not None:
            mix, out_coef, y, scale = update
            if rows is not None:
                raise KernelError("streams_layernorm: an update takes every row")
            _check(mix, "mix", torch.float32, (s_, s_))
            _check(out_coef, "out_coef", torch.float32, (s_,))
            _check(y, "y", torch.float32, (n, width))
            if scale is not None:
                _check(scale, "scale", torch.float32, (width,))
        self._ok(self._lib.rb_streams_update_layernorm(_ptr(x), s_, n * width, _ptr(mix), _ptr(out_coef), _ptr(y), _ptr(scale),
                                                       _ptr(coef), _ptr(delta), _ptr(weight), _ptr(bias), float(eps), _ptr(rows),
                                                       n_rows, width, _ptr(out), dtype_code(out.dtype), self._stream()))

    def streams_update(self, x: torch.Tensor, mix: torch.Tensor, out_coef: torch.Tensor, y: torch.Tensor,
                       scale: Optional[torch.Tensor]) -> None:
        """x [S, T, E] <- mix^T x + out_coef (scale * y), every copy from all the old ones."""
        s_, n, width = x.shape
        _check(x, "x", torch.float32)
        _check(mix, "mix", torch.float32, (s_, s_))
        _check(out_coef, "out_coef", torch.float32, (s_,))
        _check(y, "y", torch.float32, (n, width))
        if scale is not None:
            _check(scale, "scale", torch.float32, (width,))
        self._ok(self._lib.rb_streams_update(_ptr(x), s_, n * width, _ptr(mix), _ptr(out_coef), _ptr(y), _ptr(scale), n, width,
                                             self._stream()))

    def xielu(self, z: torch.Tensor, act: torch.Tensor, out: torch.Tensor) -> None:
        _check(z, "z", torch.float32)
        _check(act, "act", torch.float32, (2,))
        _check(out, "out", None, z.shape)
        self._ok(self._lib.rb_xielu(_ptr(z), _ptr(act), _ptr(out), dtype_code(out.dtype), z.numel(), self._stream()))

    def tanh_cap(self, x: torch.Tensor, cap: float) -> None:
        _check(x, "x", torch.float32)
        self._ok(self._lib.rb_tanh_cap(_ptr(x), float(cap), x.numel(), self._stream()))

    # ------------------------------------------------------------------ layers with a state per sequence
    def short_conv(self, x: torch.Tensor, col0: int, channels: int, w: torch.Tensor, state: Optional[torch.Tensor], ctx,
                   out: torch.Tensor, residual: bool, act: int) -> None:
        """Columns col0 .. col0 + channels of x [T, W] float32 through the causal convolution w [channels, taps];
        state [slots, taps - 1, channels] float32 holds every sequence's last inputs and is moved on by the step."""
        n, width = x.shape
        taps = w.shape[1]
        _check(x, "x", torch.float32)
        _check(w, "w", torch.float32, (channels, taps))
        if col0 < 0 or col0 + channels > width:
            raise KernelError("short_conv: the columns lie outside the rows")
        if taps > 1:
            _check(state, "state", torch.float32)
            if tuple(state.shape[1:]) != (taps - 1, channels):
                raise KernelError(f"short_conv: state of shape {tuple(state.shape)}, expected [*, {taps - 1}, {channels}]")
        _check(out, "out", None, (n, channels))
        _check(ctx.tok_pos, "tok_pos", torch.int32, (n,))
        self._ok(self._lib.rb_short_conv(x.data_ptr() + 4 * col0, width, _ptr(w), taps, _ptr(state) if taps > 1 else None,
                                         _ptr(ctx.tok_pos), _ptr(ctx.tok_seq), _ptr(ctx.cu_seqlens), _ptr(ctx.slots), _ptr(out),
                                         channels, dtype_code(out.dtype), int(bool(residual)), int(act), n, ctx.n_seqs,
                                         channels, self._stream()))

    def delta_prep(self, qkv: torch.Tensor, n_kv: int, dim: int, a: torch.Tensor, dt_bias: torch.Tensor, a_log: torch.Tensor,
                   n_heads: int, b_in: torch.Tensor, b_col: int, beta: torch.Tensor, q_scale: float, unit_eps: float) -> None:
        """In place: the q and k heads at the start of qkv's rows become unit vectors, the first H * dim columns of a
        the decays; beta [T, H] = sigmoid of columns b_col .. of b_in."""
        n, width = qkv.shape
        _check(qkv, "qkv", torch.float32)
        if width < 2 * n_kv * dim:
            raise KernelError("delta_prep: rows too short for the q and k heads")
        _check(a, "a", torch.float32)
        if a.shape[0] != n or a.shape[1] < n_heads * dim:
            raise KernelError("delta_prep: rows of a too short for the decays")
        _check(dt_bias, "dt_bias", torch.float32, (n_heads * dim,))
        _check(a_log, "a_log", torch.float32, (n_heads,))
        _check(b_in, "b_in", torch.float32)
        if b_in.shape[0] != n or b_col < 0 or b_col + n_heads > b_in.shape[1]:
            raise KernelError("delta_prep: the beta columns lie outside the rows")
        _check(beta, "beta", torch.float32, (n, n_heads))
        self._ok(self._lib.rb_delta_prep(_ptr(qkv), width, n_kv, dim, _ptr(a), a.shape[1], _ptr(dt_bias), _ptr(a_log), n_heads,
                                         b_in.data_ptr() + 4 * b_col, b_in.shape[1], _ptr(beta), float(q_scale), float(unit_eps),
                                         n, self._stream()))

    def delta_rule(self, qkv: torch.Tensor, n_kv: int, dim: int, n_heads: int, vdim: int, g: torch.Tensor,
                   beta: torch.Tensor, state: torch.Tensor, ctx, out: torch.Tensor) -> None:
        """qkv [T, >= (2 Hk dim + H vdim)] float32: q heads, k heads, v heads; state [slots, H, vdim, dim] float32 (the
        matrix S [dim, vdim] of a head, kept column by column)."""
        n, width = qkv.shape
        _check(qkv, "qkv", torch.float32)
        if width < 2 * n_kv * dim + n_heads * vdim:
            raise KernelError("delta_rule: rows too short for q, k and v")
        _check(g, "g", torch.float32)
        if g.shape[0] != n or g.shape[1] < n_heads * dim:
            raise KernelError("delta_rule: rows of g too short for the decays")
        _check(beta, "beta", torch.float32, (n, n_heads))
        _check(state, "state", torch.float32)
        if tuple(state.shape[1:]) != (n_heads, vdim, dim):
            raise KernelError(f"delta_rule: state of shape {tuple(state.shape)}, expected [*, {n_heads}, {vdim}, {dim}]")
        _check(out, "out", torch.float32, (n, n_heads * vdim))
        if ctx.n_tokens != n:
            raise KernelError("delta_rule: the step's tokens and the rows differ")
        base = qkv.data_ptr()
        self._ok(self._lib.rb_delta_rule(base, base + 4 * n_kv * dim, width, base + 8 * n_kv * dim, width, _ptr(g), g.shape[1], _ptr(beta),
                                         _ptr(state), _ptr(ctx.cu_seqlens), _ptr(ctx.slots), _ptr(out), ctx.n_seqs, n, n_heads,
                                         n_kv, dim, vdim, self._stream()))

    def gated_rmsnorm(self, o: torch.Tensor, weight: torch.Tensor, gate: torch.Tensor, gate_col: int, eps: float,
                      n_heads: int, vdim: int, out: torch.Tensor) -> None:
        n = o.shape[0]
        _check(o, "o", torch.float32, (n, n_heads * vdim))
        _check(weight, "weight", torch.float32, (vdim,))
        _check(gate, "gate", torch.float32)
        if gate.shape[0] != n or gate_col < 0 or gate_col + n_heads * vdim > gate.shape[1]:
            raise KernelError("gated_rmsnorm: the gate's columns lie outside the rows")
        _check(out, "out", None, (n, n_heads * vdim))
        self._ok(self._lib.rb_gated_rmsnorm(_ptr(o), _ptr(weight), gate.data_ptr() + 4 * gate_col, gate.shape[1], float(eps),
                                            _ptr(out), dtype_code(out.dtype), n, n_heads, vdim, self._stream()))

    # ------------------------------------------------------------------ recurrences with their choices spelled out
    def recurrence_prep(self, qkv: torch.Tensor, n_kv: int, dim: int, unit: bool, q_scale: float, unit_eps: float,
                        a: torch.Tensor, a_col: int, a_cols: int, decay: int, bias: Optional[torch.Tensor],
                        a_log: Optional[torch.Tensor], tau: float, n_heads: int, b_in: Optional[torch.Tensor] = None,
                        b_col: int = 0, beta: Optional[torch.Tensor] = None) -> None:
        """In place: the q and k heads at the start of qkv's rows (unit vectors, or q only scaled), and columns
        a_col .. a_col + a_cols of `a` turned into decays (a_cols = heads: one per head; heads * dim: per key channel;
        decay 0: exp(-exp(a_log) softplus(a + bias)), 1: sigmoid(a + bias) ^ (1 / tau)); beta [T, H] from b_in's columns."""
        n, width = qkv.shape
        _check(qkv, "qkv", torch.float32)
        if width < 2 * n_kv * dim:
            raise KernelError("recurrence_prep: rows too short for the q and k heads")
        _check(a, "a", torch.float32)
        if a.shape[0] != n or a_col < 0 or a_col + a_cols > a.shape[1] or a_cols not in (n_heads, n_heads * dim):
            raise KernelError("recurrence_prep: the decays' columns lie outside the rows, or are not one per head or channel")
        if bias is not None:
            _check(bias, "bias", torch.float32, (a_cols,))
        if decay == 0:
            _check(a_log, "a_log", torch.float32, (n_heads,))
        b_ptr, b_stride = None, 0
        if b_in is not None:
            _check(b_in, "b_in", torch.float32)
            if b_in.shape[0] != n or b_col < 0 or b_col + n_heads > b_in.shape[1]:
                raise KernelError("recurrence_prep: the beta columns lie outside the rows")
            _check(beta, "beta", torch.float32, (n, n_heads))
            b_ptr, b_stride = b_in.data_ptr() + 4 * b_col, b_in.shape[1]
        self._ok(self._lib.rb_recurrence_prep(_ptr(qkv), width, n_kv, dim, int(bool(unit)), float(q_scale), float(unit_eps),
                                              a.data_ptr() + 4 * a_col, a.shape[1], a_cols, int(decay), _ptr(bias), _ptr(a_log),
                                              float(tau), n_heads, b_ptr, b_stride, _ptr(beta), n, self._stream()))

    def linear_recurrence(self, qkv: torch.Tensor, n_kv: int, dim: int, n_heads: int, vdim: int, g: torch.Tensor, g_col: int,
                          g_per_head: bool, beta: Optional[torch.Tensor], state: torch.Tensor, ctx, out: torch.Tensor) -> None:
        """`delta_rule` with the decays at columns g_col .. of g, one per head (g_per_head) or per head and key channel,
        and, without beta, the plain rule S <- diag(g) S + k v^T."""
        n, width = qkv.shape
        _check(qkv, "qkv", torch.float32)
        if width < 2 * n_kv * dim + n_heads * vdim:
            raise KernelError("linear_recurrence: rows too short for q, k and v")
        _check(g, "g", torch.float32)
        if g.shape[0] != n or g_col < 0 or g_col + n_heads * (1 if g_per_head else dim) > g.shape[1]:
            raise KernelError("linear_recurrence: the decays' columns lie outside the rows")
        if beta is not None:
            _check(beta, "beta", torch.float32, (n, n_heads))
        _check(state, "state", torch.float32)
        if tuple(state.shape[1:]) != (n_heads, vdim, dim):
            raise KernelError(f"linear_recurrence: state of shape {tuple(state.shape)}, expected [*, {n_heads}, {vdim}, {dim}]")
        _check(out, "out", torch.float32, (n, n_heads * vdim))
        if ctx.n_tokens != n:
            raise KernelError("linear_recurrence: the step's tokens and the rows differ")
        base = qkv.data_ptr()
        self._ok(self._lib.rb_linear_recurrence(base, base + 4 * n_kv * dim, width, base + 8 * n_kv * dim, width,
                                                g.data_ptr() + 4 * g_col, g.shape[1], int(bool(g_per_head)), _ptr(beta), _ptr(state),
                                                _ptr(ctx.cu_seqlens), _ptr(ctx.slots), _ptr(out), ctx.n_seqs, n, n_heads, n_kv, dim,
                                                vdim, self._stream()))

    def gated_rmsnorm_act(self, o: torch.Tensor, weight: torch.Tensor, gate: torch.Tensor, gate_col: int, act: int, eps: float,
                          n_heads: int, vdim: int, out: torch.Tensor) -> None:
        """`gated_rmsnorm` with the gate's activation: 0 sigmoid, 1 silu."""
        n = o.shape[0]
        _check(o, "o", torch.float32, (n, n_heads * vdim))
        _check(weight, "weight", torch.float32, (vdim,))
        _check(gate, "gate", torch.float32)
        if gate.shape[0] != n or gate_col < 0 or gate_col + n_heads * vdim > gate.shape[1]:
            raise KernelError("gated_rmsnorm: the gate's columns lie outside the rows")
        _check(out, "out", None, (n, n_heads * vdim))
        self._ok(self._lib.rb_gated_rmsnorm_act(_ptr(o), _ptr(weight), gate.data_ptr() + 4 * gate_col, gate.shape[1], int(act),
                                                float(eps), _ptr(out), dtype_code(out.dtype), n, n_heads, vdim, self._stream()))

    def layernorm_residual(self, x: torch.Tensor, delta: Optional[torch.Tensor], delta2: Optional[torch.Tensor], dscale: float,
                           weight: torch.Tensor, bias: Optional[torch.Tensor], eps: float, rows: Optional[torch.Tensor],
                           out: torch.Tensor) -> None:
        """Layer norm of x [T, E] + dscale * (delta + delta2); without rows the sum is written back to x."""
        n, width = x.shape
        _check(x, "x", torch.float32)
        for name, d in (("delta", delta), ("delta2", delta2)):
            if d is not None:
                _check(d, name, torch.float32, (n, width))
        if delta is None and delta2 is not None:
            raise KernelError("layernorm_residual: a second term without a first")
        _check(weight, "weight", torch.float32, (width,))
        if bias is not None:
            _check(bias, "bias", torch.float32, (width,))
        n_rows = n
        if rows is not None:
            n_rows = rows.shape[0]
            _check(rows, "rows", torch.int32, (n_rows,))
        _check(out, "out", None, (n_rows, width))
        self._ok(self._lib.rb_layernorm_residual(_ptr(x), _ptr(delta), _ptr(delta2), float(dscale), _ptr(weight), _ptr(bias),
                                                 float(eps), _ptr(rows), n_rows, width, _ptr(out), dtype_code(out.dtype),
                                                 self._stream()))

    # ------------------------------------------------------------------ around the mixers
    def rope_store(self, qkv: torch.Tensor, cos, sin, rot: int, q_out: torch.Tensor, k_pages, v_pages, tok_pos, tok_seq,
                   block_table, n_heads: int, n_kv: int, dim: int, vdim: int, pad: int) -> None:
        """qkv [T, Hq dim (+ Hk dim + Hk vdim)] float32 -> q_out [T, Hq, pad] and the pages [*, Hk, 64, pad], the first
        `rot` numbers of every q and k head rotated (i with i + rot / 2), heads padded with zeros."""
        n, width = qkv.shape
        _check(qkv, "qkv", torch.float32)
        _check(q_out, "q_out", None, (n, n_heads, pad))
        _check(tok_pos, "tok_pos", torch.int32, (n,))
        _check(tok_seq, "tok_seq", torch.int32, (n,))
        if rot:
            _check(cos, "cos", torch.float32)
            _check(sin, "sin", torch.float32, cos.shape)
            if cos.shape[1] != rot // 2:
                raise KernelError("angle table width mismatch")
        need = n_heads * dim
        if k_pages is not None:
            need += n_kv * (dim + vdim)
            _check(block_table, "block_table", torch.int32)
            _check(k_pages, "k_pages", q_out.dtype)
            _check(v_pages, "v_pages", q_out.dtype, k_pages.shape)
            if tuple(k_pages.shape[1:]) != (n_kv, self.page_size, pad):
                raise KernelError(f"cache pages have shape {tuple(k_pages.shape)}, expected [*, {n_kv}, {self.page_size}, {pad}]")
        if width < need:
            raise KernelError("rope_store: rows too short for the heads")
        self._ok(self._lib.rb_rope_store(_ptr(qkv), width, _ptr(cos), _ptr(sin), int(rot), _ptr(q_out), _ptr(k_pages), _ptr(v_pages),
                                         dtype_code(q_out.dtype), _ptr(tok_pos), _ptr(tok_seq),
                                         _ptr(block_table) if k_pages is not None else None,
                                         block_table.shape[1] if k_pages is not None else 0, n, n_heads, n_kv if k_pages is not None else 0,
                                         dim, vdim, pad, self._stream()))

    def head_gate(self, x: torch.Tensor, gate: torch.Tensor, gate_col: int, n_heads: int, head_dim: int) -> None:
        """x [T, H * D] *= sigmoid(gate[:, gate_col + h]) per head, in place."""
        n = x.shape[0]
        _check(x, "x", None, (n, n_heads * head_dim))
        _check(gate, "gate", torch.float32)
        if gate.shape[0] != n or gate_col < 0 or gate_col + n_heads > gate.shape[1]:
            raise KernelError("head_gate: the gate's columns lie outside the rows")
        self._ok(self._lib.rb_head_gate(_ptr(x), dtype_code(x.dtype), gate.data_ptr() + 4 * gate_col, gate.shape[1], n, n_heads,
                                        head_dim, self._stream()))

    def pair_norm_mean(self, a: torch.Tensor, wa: torch.Tensor, b: torch.Tensor, wb: torch.Tensor, eps: float,
                       out: torch.Tensor) -> None:
        n, width = a.shape
        _check(a, "a", torch.float32)
        _check(b, "b", torch.float32, (n, width))
        _check(wa, "wa", torch.float32, (width,))
        _check(wb, "wb", torch.float32, (width,))
        _check(out, "out", torch.float32, (n, width))
        self._ok(self._lib.rb_pair_norm_mean(_ptr(a), _ptr(wa), _ptr(b), _ptr(wb), float(eps), _ptr(out), n, width, self._stream()))

    # ------------------------------------------------------------------ routed experts
    @staticmethod
    def routed_rows(n_tokens: int, top: int, n_experts: int) -> int:
        """Rows that the sorted pairs of a step may take: every expert's run is padded to 16."""
        return (n_tokens * top + 15) // 16 * 16 + 16 * n_experts

    def route_top(self, z: torch.Tensor, n_experts: int, top: int, sel: torch.Tensor, weight: torch.Tensor,
                  row_pair: torch.Tensor, tile_expert: torch.Tensor) -> None:
        n = z.shape[0]
        _check(z, "z", torch.float32)
        if z.shape[1] < n_experts:
            raise KernelError("route_top: rows too short for the experts")
        max_rows = row_pair.shape[0]
        if max_rows < self.routed_rows(n, top, n_experts) or max_rows % 16:
            raise KernelError("route_top: too little room for the sorted pairs")
        _check(sel, "sel", torch.int32, (n * top,))
        _check(weight, "weight", torch.float32, (n * top,))
        _check(row_pair, "row_pair", torch.int32, (max_rows,))
        _check(tile_expert, "tile_expert", torch.int32, (2 * (max_rows // 16),))
        self._ok(self._lib.rb_route_top(_ptr(z), z.shape[1], n_experts, top, _ptr(sel), _ptr(weight), _ptr(row_pair),
                                        _ptr(tile_expert), max_rows, n, self._stream()))

    def routed_experts(self, h: torch.Tensor, weight: torch.Tensor, top: int, row_pair: torch.Tensor, tile_expert: torch.Tensor,
                       w_gate: torch.Tensor, w_up: torch.Tensor, w_down: torch.Tensor, y: torch.Tensor, out: torch.Tensor,
                       limit: float, alpha: float, w_frag: bool = False) -> None:
        """w_frag: every expert's matrices are stored fragment-major (`place_rows(..., frag=True)` on each)."""
        n, width = h.shape
        n_experts, ff, _ = w_gate.shape
        max_rows = row_pair.shape[0]
        _check(h, "h")
        if weight is not None:                   # None: the experts' inputs are not scaled
            _check(weight, "weight", torch.float32, (n * top,))
        _check(row_pair, "row_pair", torch.int32)
        _check(tile_expert, "tile_expert", torch.int32, (2 * (max_rows // 16),))
        _check(w_gate, "w_gate", h.dtype, (n_experts, ff, width))
        _check(w_up, "w_up", h.dtype, (n_experts, ff, width))
        _check(w_down, "w_down", h.dtype, (n_experts, width, ff))
        _check(y, "y", h.dtype, (max_rows, ff + width))
        _check(out, "out", torch.float32, (n * top, width))
        self._ok(self._lib.rb_routed_experts(_ptr(h), dtype_code(h.dtype), _ptr(weight), top, _ptr(row_pair), _ptr(tile_expert),
                                             max_rows, _ptr(w_gate), _ptr(w_up), _ptr(w_down), int(bool(w_frag)), _ptr(y), _ptr(out),
                                             n_experts, width, ff, float(limit), float(alpha), self._stream()))

    def route_choose(self, z: torch.Tensor, n_outputs: int, n_experts: int, top: int, score: int,
                     correction: Optional[torch.Tensor], sel: torch.Tensor, weight: torch.Tensor, row_pair: torch.Tensor,
                     tile_expert: torch.Tensor) -> None:
        """`route_top` with its choices spelled out: the router's first n_experts outputs are experts with matrices, the
        rest stand for the token's own input; score 0 sigmoid, 1 softmax over all outputs with `correction` [n_outputs]
        added for the choice only."""
        n = z.shape[0]
        _check(z, "z", torch.float32)
        if z.shape[1] < n_outputs or n_experts > n_outputs:
            raise KernelError("route_choose: rows too short for the router's outputs")
        max_rows = row_pair.shape[0]
        if max_rows < self.routed_rows(n, top, n_experts) or max_rows % 16:
            raise KernelError("route_choose: too little room for the sorted pairs")
        if correction is not None:
            _check(correction, "correction", torch.float32, (n_outputs,))
        _check(sel, "sel", torch.int32, (n * top,))
        _check(weight, "weight", torch.float32, (n * top,))
        _check(row_pair, "row_pair", torch.int32, (max_rows,))
        _check(tile_expert, "tile_expert", torch.int32, (2 * (max_rows // 16),))
        self._ok(self._lib.rb_route_choose(_ptr(z), z.shape[1], n_outputs, n_experts, top, int(score), _ptr(correction), _ptr(sel),
                                           _ptr(weight), _ptr(row_pair), _ptr(tile_expert), max_rows, n, self._stream()))

    def experts_combine(self, pairs: torch.Tensor, sel: torch.Tensor, weight: torch.Tensor, top: int, n_experts: int,
                        h: torch.Tensor, shared: Optional[torch.Tensor], gate: Optional[torch.Tensor], gate_col: int,
                        out: torch.Tensor) -> None:
        """out[t] = sum_k weight * (the pair's expert output, or h[t] for an output behind the experts), plus
        sigmoid(gate[t, gate_col]) * shared[t] when there is a shared expert."""
        n, width = out.shape
        _check(pairs, "pairs", torch.float32, (n * top, width))
        _check(sel, "sel", torch.int32, (n * top,))
        _check(weight, "weight", torch.float32, (n * top,))
        _check(h, "h", None, (n, width))
        _check(out, "out", torch.float32)
        gate_ptr, stride = None, 0
        if shared is not None:
            _check(shared, "shared", torch.float32, (n, width))
            _check(gate, "gate", torch.float32)
            if gate.shape[0] != n or not 0 <= gate_col < gate.shape[1]:
                raise KernelError("experts_combine: the gate's column lies outside its rows")
            gate_ptr, stride = gate.data_ptr() + 4 * gate_col, gate.shape[1]
        self._ok(self._lib.rb_experts_combine(_ptr(pairs), _ptr(sel), _ptr(weight), top, n_experts, _ptr(h), dtype_code(h.dtype),
                                              _ptr(shared), gate_ptr, stride, _ptr(out), n, width, self._stream()))

    # ------------------------------------------------------------------ attention with mixed heads
    def embed_scaled_pos(self, table: torch.Tensor, ids: torch.Tensor, scale: float, positions: Optional[torch.Tensor],
                         tok_pos: torch.Tensor, out: torch.Tensor) -> None:
        n, width = out.shape
        _check(table, "table")
        _check(ids, "ids", torch.int32, (n,))
        _check(tok_pos, "tok_pos", torch.int32, (n,))
        _check(out, "out", torch.float32)
        if table.shape[1] != width:
            raise KernelError("embedding width mismatch")
        if positions is not None:
            _check(positions, "positions", table.dtype)
            if positions.shape[1] != width:
                raise KernelError("position table width mismatch")
        self._ok(self._lib.rb_embed_scaled_pos(_ptr(table), dtype_code(table.dtype), _ptr(ids), float(scale), _ptr(positions),
                                               _ptr(tok_pos), _ptr(out), n, width, self._stream()))

    def scale(self, x: torch.Tensor, s: float) -> None:
        _check(x, "x", torch.float32)
        self._ok(self._lib.rb_scale(_ptr(x), float(s), x.numel(), self._stream()))

    def bias_norm_store(self, qkv: torch.Tensor, bias: Optional[torch.Tensor], norm: bool, eps: float, q_out: torch.Tensor,
                        k_pages, v_pages, tok_pos, tok_seq, block_table, n_heads: int, n_kv: int, dim: int, vdim: int,
                        pad: int) -> None:
        """qkv [T, W] float32 (+ bias [W]); query and key heads divided by their root mean square when `norm`; queries to
        q_out [T, Hq, pad], keys and values to the pages [*, Hk, 64, pad] (None: the rows hold queries only)."""
        n, width = qkv.shape
        owns = k_pages is not None
        need = (n_heads + n_kv) * dim + n_kv * vdim if owns else n_heads * dim
        _check(qkv, "qkv", torch.float32)
        if width != need:
            raise KernelError(f"bias_norm_store: rows of {width} numbers, the heads take {need}")
        if bias is not None:
            _check(bias, "bias", torch.float32, (width,))
        _check(q_out, "q_out", None, (n, n_heads, pad))
        _check(tok_pos, "tok_pos", torch.int32, (n,))
        _check(tok_seq, "tok_seq", torch.int32, (n,))
        if owns:
            _check(block_table, "block_table", torch.int32)
            _check(k_pages, "k_pages", q_out.dtype)
            _check(v_pages, "v_pages", q_out.dtype, k_pages.shape)
            if tuple(k_pages.shape[1:]) != (n_kv, self.page_size, pad):
                raise KernelError(f"cache pages have shape {tuple(k_pages.shape)}, expected [*, {n_kv}, {self.page_size}, {pad}]")
        self._ok(self._lib.rb_bias_norm_store(_ptr(qkv), width, _ptr(bias), int(bool(norm)), float(eps), _ptr(q_out), _ptr(k_pages),
                                              _ptr(v_pages), dtype_code(q_out.dtype), _ptr(tok_pos), _ptr(tok_seq),
                                              _ptr(block_table) if owns else None, block_table.shape[1] if owns else 0, n,
                                              n_heads, n_kv if owns else 0, dim, vdim, pad, self._stream()))

    def attention_mixed(self, q, k_pages, v_pages, out, tok_pos, tok_seq, block_table, n_heads, n_kv, head_dim, scale, talk,
                        chunk, window) -> None:
        """All heads of a token together: scores mixed over the heads by talk [Hq, Hq] (None: none) before the softmax, keys
        limited to the token's chunk (chunk positions counted from 0; 0: no chunks) and to the last `window` (0: all)."""
        n = q.shape[0]
        _check(q, "q", None, (n, n_heads, head_dim))
        _check(k_pages, "k_pages", q.dtype)
        _check(v_pages, "v_pages", q.dtype, k_pages.shape)
        if tuple(k_pages.shape[1:]) != (n_kv, self.page_size, head_dim):
            raise KernelError("cache pages do not match the head counts")
        _check(out, "out", q.dtype, (n, n_heads * head_dim))
        _check(tok_pos, "tok_pos", torch.int32, (n,))
        _check(tok_seq, "tok_seq", torch.int32, (n,))
        _check(block_table, "block_table", torch.int32)
        if talk is not None:
            _check(talk, "talk", torch.float32, (n_heads, n_heads))
        self._ok(self._lib.rb_attention_mixed(_ptr(q), _ptr(k_pages), _ptr(v_pages), _ptr(out), dtype_code(q.dtype), _ptr(tok_pos),
                                              _ptr(tok_seq), _ptr(block_table), block_table.shape[1], n, n_heads, n_kv, head_dim,
                                              float(scale), _ptr(talk), int(chunk or 0), int(window or 0), self._stream()))

    def attention_mixed_bf16(self, q, k_pages, v_pages, out, ctx, block_table, n_heads, n_kv, head_dim, scale, talk, chunk,
                             window, n_splits: int = 1, workspace: Optional[torch.Tensor] = None) -> None:
        """attention_mixed on the matrix cores: bfloat16, head_dim 64 or 128, at most 32 heads; the step's sequences from
        ctx (cu_seqlens, past_len).  n_splits > 1: every sequence's pages are dealt out to that many workgroups, whose sums
        go through `workspace` (float32, n_splits * T * heads * (head_dim + 2))."""
        n = q.shape[0]
        _check(q, "q", torch.bfloat16, (n, n_heads, head_dim))
        _check(k_pages, "k_pages", torch.bfloat16)
        _check(v_pages, "v_pages", torch.bfloat16, k_pages.shape)
        if tuple(k_pages.shape[1:]) != (n_kv, self.page_size, head_dim):
            raise KernelError("cache pages do not match the head counts")
        if head_dim not in (64, 128) or n_heads > 32 or n_heads % n_kv:
            raise KernelError(f"attention_mixed_bf16: {n_heads} heads of {head_dim} numbers not supported (64 or 128, at most 32 heads)")
        if n != ctx.n_tokens:
            raise KernelError(f"attention_mixed_bf16: {n} rows for a step of {ctx.n_tokens} tokens")
        _check(out, "out", torch.bfloat16, (n, n_heads * head_dim))
        _check(ctx.cu_seqlens, "cu_seqlens", torch.int32, (ctx.n_seqs + 1,))
        _check(ctx.past_len, "past_len", torch.int32, (ctx.n_seqs,))
        _check(block_table, "block_table", torch.int32)
        if block_table.shape[0] < ctx.n_seqs:
            raise KernelError("attention_mixed_bf16: the block table has fewer rows than the step has sequences")
        _check(talk, "talk", torch.float32, (n_heads, n_heads))
        n_splits = int(n_splits)
        if not 1 <= n_splits <= 64:
            raise KernelError(f"attention_mixed_bf16: {n_splits} splits not supported (1 to 64)")
        if n_splits > 1:
            _check(workspace, "workspace", torch.float32)
            if workspace.numel() < n_splits * n * n_heads * (head_dim + 2):
                raise KernelError("attention_mixed_bf16: the workspace is smaller than splits * T * heads * (head_dim + 2)")
        self._ok(self._lib.rb_attention_mixed_bf16(_ptr(q), _ptr(k_pages), _ptr(v_pages), _ptr(out), _ptr(ctx.cu_seqlens),
                                                   _ptr(ctx.past_len), _ptr(block_table), block_table.shape[1], ctx.n_seqs, n,
                                                   n_heads, n_kv, head_dim, float(scale), _ptr(talk), int(chunk or 0),
                                                   int(window or 0), n_splits, _ptr(workspace) if n_splits > 1 else None,
                                                   self._stream()))

    def pairs_sum(self, pairs: torch.Tensor, top: int, out: torch.Tensor) -> None:
        n, width = out.shape
        _check(pairs, "pairs", torch.float32, (n * top, width))
        _check(out, "out", torch.float32)
        self._ok(self._lib.rb_pairs_sum(_ptr(pairs), top, _ptr(out), n, width, self._stream()))

    # ------------------------------------------------------------------ attention through a latent
    def latent_norm_store(self, proj: torch.Tensor, q_rank: int, q_gain: Optional[torch.Tensor], cq: Optional[torch.Tensor],
                          kv_rank: int, kv_gain: Optional[torch.Tensor], pages: Optional[torch.Tensor], ctx, block_table,
                          eps: float, dtype: torch.dtype) -> None:
        """proj [T, q_rank + kv_rank] float32: the two down-projections; cq [T, q_rank] and the pages
        [*, 1, 64, kv_rank] get their RMS norms (kv_rank 0: no latent is stored)."""
        n, width = proj.shape
        _check(proj, "proj", torch.float32)
        if width < q_rank + kv_rank:
            raise KernelError("latent_norm_store: rows too short for the two down-projections")
        if q_rank:
            _check(q_gain, "q_gain", torch.float32, (q_rank,))
            _check(cq, "cq", dtype, (n, q_rank))
        if kv_rank:
            _check(kv_gain, "kv_gain", torch.float32, (kv_rank,))
            _check(pages, "pages", dtype)
            if tuple(pages.shape[1:]) != (1, self.page_size, kv_rank):
                raise KernelError(f"latent pages have shape {tuple(pages.shape)}, expected [*, 1, {self.page_size}, {kv_rank}]")
            _check(block_table, "block_table", torch.int32)
        self._ok(self._lib.rb_latent_norm_store(_ptr(proj), width, q_rank, _ptr(q_gain), _ptr(cq), q_rank, kv_rank, _ptr(kv_gain),
                                                _ptr(pages) if kv_rank else None, dtype_code(dtype), _ptr(ctx.tok_pos),
                                                _ptr(ctx.tok_seq), _ptr(block_table) if kv_rank else None,
                                                block_table.shape[1] if kv_rank else 0, float(eps), n, self._stream()))

    def heads_linear(self, x: torch.Tensor, w: torch.Tensor, y: torch.Tensor) -> None:
        """y[t, h, :] = w[h]^T x[t, h, :] with w [H, K, N]; x [T, H * K], y [T, H * N]."""
        h, k, n_out = w.shape
        n = x.shape[0]
        _check(x, "x", None, (n, h * k))
        _check(w, "w")
        _check(y, "y", None, (n, h * n_out))
        self._ok(self._lib.rb_heads_linear(_ptr(x), dtype_code(x.dtype), _ptr(w), dtype_code(w.dtype), _ptr(y),
                                           dtype_code(y.dtype), n, h, n_out, k, self._stream()))

    def attention_sinks(self, q, k_pages, v_pages, out, tok_pos, tok_seq, block_table, n_heads, n_kv, head_dim,
                        scale, window, sinks) -> None:
        """`attention_generic` with a sink per query head in the softmax's denominator (sinks float32 [Hq] or None);
        v_pages may be k_pages itself."""
        n = q.shape[0]
        _check(q, "q", None, (n, n_heads, head_dim))
        _check(k_pages, "k_pages", q.dtype)
        _check(v_pages, "v_pages", q.dtype, k_pages.shape)
        if tuple(k_pages.shape[1:]) != (n_kv, self.page_size, head_dim):
            raise KernelError("cache pages do not match the head counts")
        _check(out, "out", q.dtype, (n, n_heads * head_dim))
        _check(tok_pos, "tok_pos", torch.int32, (n,))
        _check(tok_seq, "tok_seq", torch.int32, (n,))
        _check(block_table, "block_table", torch.int32)
        if sinks is not None:
            _check(sinks, "sinks", torch.float32, (n_heads,))
        self._ok(self._lib.rb_attention_generic_sinks(_ptr(q), _ptr(k_pages), _ptr(v_pages), _ptr(out), dtype_code(q.dtype),
                                                      _ptr(tok_pos), _ptr(tok_seq), _ptr(block_table), block_table.shape[1],
                                                      n, n_heads, n_kv, head_dim, float(scale), int(window or 0),
                                                      _ptr(sinks), self._stream()))

    # ------------------------------------------------------------------ layers with the norm on the sublayer's output
    def outnorm_residual(self, x: torch.Tensor, a: torch.Tensor, b: Optional[torch.Tensor], sa: float, sb: float,
                         gain: torch.Tensor, eps: float, assign: bool, h_out: Optional[torch.Tensor]) -> None:
        """x [T, E] float32 <- (assign ? 0 : x) + rmsnorm(sa a + sb b) * gain; h_out [T, E] gets the new rows in its dtype."""
        n, width = x.shape
        _check(x, "x", torch.float32)
        _check(a, "a", torch.float32, (n, width))
        if b is not None:
            _check(b, "b", torch.float32, (n, width))
        _check(gain, "gain", torch.float32, (width,))
        if h_out is not None:
            _check(h_out, "h_out", None, (n, width))
        self._ok(self._lib.rb_outnorm_residual(_ptr(x), _ptr(a), _ptr(b), float(sa), float(sb), _ptr(gain), float(eps),
                                               int(bool(assign)), _ptr(h_out), dtype_code(h_out.dtype) if h_out is not None else _F32,
                                               n, width, self._stream()))

    def clamped_glu(self, gu: torch.Tensor, out: torch.Tensor, limit: float, alpha: float) -> None:
        """gu [T, 2 F] float32 (gate, then up) -> out [T, F] = g sigmoid(alpha g) (u + 1) with g, u limited."""
        n, ff = out.shape
        _check(gu, "gu", torch.float32, (n, 2 * ff))
        _check(out, "out")
        self._ok(self._lib.rb_clamped_glu(_ptr(gu), _ptr(out), dtype_code(out.dtype), n, ff, float(limit), float(alpha), self._stream()))

    def tanh_cast(self, z: torch.Tensor, out: torch.Tensor) -> None:
        _check(z, "z", torch.float32)
        _check(out, "out", None, z.shape)
        self._ok(self._lib.rb_tanh_cast(_ptr(z), _ptr(out), dtype_code(out.dtype), z.numel(), self._stream()))

    def attention_opts(self, q, k_pages, v_pages, out, tok_pos, tok_seq, block_table, n_heads, n_kv, head_dim, scale, window,
                       keep_first, softcap, sinks) -> None:
        """`attention_sinks` with kept first keys behind the window and capped scores."""
        n = q.shape[0]
        _check(q, "q", None, (n, n_heads, head_dim))
        _check(k_pages, "k_pages", q.dtype)
        _check(v_pages, "v_pages", q.dtype, k_pages.shape)
        if tuple(k_pages.shape[1:]) != (n_kv, self.page_size, head_dim):
            raise KernelError("cache pages do not match the head counts")
        _check(out, "out", q.dtype, (n, n_heads * head_dim))
        _check(tok_pos, "tok_pos", torch.int32, (n,))
        _check(tok_seq, "tok_seq", torch.int32, (n,))
        _check(block_table, "block_table", torch.int32)
        if sinks is not None:
            _check(sinks, "sinks", torch.float32, (n_heads,))
        self._ok(self._lib.rb_attention_generic_opts(_ptr(q), _ptr(k_pages), _ptr(v_pages), _ptr(out), dtype_code(q.dtype),
                                                     _ptr(tok_pos), _ptr(tok_seq), _ptr(block_table), block_table.shape[1],
                                                     n, n_heads, n_kv, head_dim, float(scale), int(window or 0),
                                                     int(keep_first or 0), float(softcap or 0.0), _ptr(sinks), self._stream()))

    def norm_rope_store(self, qkv: torch.Tensor, cos, sin, rot: int, q_norm: torch.Tensor, k_norm: Optional[torch.Tensor], eps: float,
                        q_out: torch.Tensor, k_pages, v_pages, tok_pos, tok_seq, block_table, n_heads: int, n_kv: int, dim: int,
                        vdim: int, pad: int) -> None:
        """`rope_store` with every query and key head RMS-normed first (weights float32 [dim])."""
        n, width = qkv.shape
        _check(qkv, "qkv", torch.float32)
        _check(q_out, "q_out", None, (n, n_heads, pad))
        _check(tok_pos, "tok_pos", torch.int32, (n,))
        _check(tok_seq, "tok_seq", torch.int32, (n,))
        _check(q_norm, "q_norm", torch.float32, (dim,))
        if rot:
            _check(cos, "cos", torch.float32)
            _check(sin, "sin", torch.float32, cos.shape)
            if cos.shape[1] != rot // 2:
                raise KernelError("angle table width mismatch")
        need = n_heads * dim
        if k_pages is not None:
            need += n_kv * (dim + vdim)
            _check(k_norm, "k_norm", torch.float32, (dim,))
            _check(block_table, "block_table", torch.int32)
            _check(k_pages, "k_pages", q_out.dtype)
            _check(v_pages, "v_pages", q_out.dtype, k_pages.shape)
            if tuple(k_pages.shape[1:]) != (n_kv, self.page_size, pad):
                raise KernelError(f"cache pages have shape {tuple(k_pages.shape)}, expected [*, {n_kv}, {self.page_size}, {pad}]")
        if width < need:
            raise KernelError("norm_rope_store: rows too short for the heads")
        self._ok(self._lib.rb_norm_rope_store(_ptr(qkv), width, _ptr(cos) if rot else None, _ptr(sin) if rot else None, int(rot),
                                              _ptr(q_norm), _ptr(k_norm), float(eps), _ptr(q_out), _ptr(k_pages), _ptr(v_pages),
                                              dtype_code(q_out.dtype), _ptr(tok_pos), _ptr(tok_seq),
                                              _ptr(block_table) if k_pages is not None else None,
                                              block_table.shape[1] if k_pages is not None else 0, n, n_heads,
                                              n_kv if k_pages is not None else 0, dim, vdim, pad, self._stream()))

    def sigmoid_gate(self, x: torch.Tensor, gate: torch.Tensor) -> None:
        """x *= sigmoid(gate), in place; both [T, N], gate float32."""
        _check(x, "x")
        _check(gate, "gate", torch.float32, x.shape)
        self._ok(self._lib.rb_sigmoid_gate(_ptr(x), dtype_code(x.dtype), _ptr(gate), x.numel(), self._stream()))

    def shift_mix(self, h: torch.Tensor, state: torch.Tensor, mu: torch.Tensor, ctx, out: torch.Tensor) -> None:
        """out[m] = h + (the row before - h) * mu[m]; state [slots, E] float32 holds every sequence's last row."""
        n, width = h.shape
        m = mu.shape[0]
        _check(h, "h")
        _check(mu, "mu", torch.float32, (m, width))
        _check(state, "state", torch.float32)
        if tuple(state.shape[1:]) != (width,):
            raise KernelError(f"shift_mix: state of shape {tuple(state.shape)}, expected [*, {width}]")
        _check(out, "out", h.dtype, (m, n, width))
        if ctx.n_tokens != n:
            raise KernelError("shift_mix: the step's tokens and the rows differ")
        self._ok(self._lib.rb_shift_mix(_ptr(h), dtype_code(h.dtype), _ptr(state), _ptr(mu), m, _ptr(out), _ptr(ctx.cu_seqlens),
                                        _ptr(ctx.tok_seq), _ptr(ctx.slots), n, ctx.n_seqs, width, self._stream()))

    def short_conv_bias(self, x: torch.Tensor, col0: int, channels: int, bias: Optional[torch.Tensor], w: torch.Tensor,
                        state: Optional[torch.Tensor], ctx, out: torch.Tensor, residual: bool, act: int) -> None:
        """`short_conv` on x + bias (float32 [channels]); the state holds the inputs with their bias."""
        n, width = x.shape
        taps = w.shape[1]
        _check(x, "x", torch.float32)
        _check(w, "w", torch.float32, (channels, taps))
        if bias is not None:
            _check(bias, "bias", torch.float32, (channels,))
        if col0 < 0 or col0 + channels > width:
            raise KernelError("short_conv: the columns lie outside the rows")
        if taps > 1:
            _check(state, "state", torch.float32)
            if tuple(state.shape[1:]) != (taps - 1, channels):
                raise KernelError(f"short_conv: state of shape {tuple(state.shape)}, expected [*, {taps - 1}, {channels}]")
        _check(out, "out", None, (n, channels))
        _check(ctx.tok_pos, "tok_pos", torch.int32, (n,))
        self._ok(self._lib.rb_short_conv_bias(x.data_ptr() + 4 * col0, width, _ptr(bias), _ptr(w), taps,
                                              _ptr(state) if taps > 1 else None, _ptr(ctx.tok_pos), _ptr(ctx.tok_seq),
                                              _ptr(ctx.cu_seqlens), _ptr(ctx.slots), _ptr(out), channels, dtype_code(out.dtype),
                                              int(bool(residual)), int(act), n, ctx.n_seqs, channels, self._stream()))

    def time_mix_recurrence(self, r: torch.Tensor, k: torch.Tensor, v: torch.Tensor, decay: torch.Tensor, bonus: torch.Tensor,
                            state: torch.Tensor, ctx, out: torch.Tensor, n_heads: int, dim: int, vdim: int) -> None:
        """r, k, decay [T, H dim], v [T, H vdim] float32; bonus [H, dim]; state [slots, H, vdim, dim] float32:
        out = (S + diag(bonus) k v^T)^T r, then S <- diag(decay) S + k v^T, token after token."""
        n = r.shape[0]
        _check(r, "r", torch.float32, (n, n_heads * dim))
        _check(k, "k", torch.float32, (n, n_heads * dim))
        _check(v, "v", torch.float32, (n, n_heads * vdim))
        _check(decay, "decay", torch.float32, (n, n_heads * dim))
        _check(bonus, "bonus", torch.float32, (n_heads, dim))
        _check(state, "state", torch.float32)
        if tuple(state.shape[1:]) != (n_heads, vdim, dim):
            raise KernelError(f"time_mix_recurrence: state of shape {tuple(state.shape)}, expected [*, {n_heads}, {vdim}, {dim}]")
        _check(out, "out", torch.float32, (n, n_heads * vdim))
        if ctx.n_tokens != n:
            raise KernelError("time_mix_recurrence: the step's tokens and the rows differ")
        self._ok(self._lib.rb_linear_recurrence_bonus(_ptr(r), _ptr(k), n_heads * dim, _ptr(v), n_heads * vdim, _ptr(decay),
                                                      n_heads * dim, 0, None, _ptr(bonus), _ptr(state), _ptr(ctx.cu_seqlens),
                                                      _ptr(ctx.slots), _ptr(out), ctx.n_seqs, n, n_heads, n_heads, dim, vdim,
                                                      self._stream()))

    def decay_exp_exp(self, z: torch.Tensor, bias: torch.Tensor, n_heads: int, dim: int) -> None:
        """z [T, H dim] float32 <- exp(-exp(z + bias)), in place."""
        n = z.shape[0]
        _check(z, "z", torch.float32, (n, n_heads * dim))
        _check(bias, "bias", torch.float32, (n_heads * dim,))
        # the q and k heads are left as they are (no unit vectors, a scale of one): any valid rows serve
        self._ok(self._lib.rb_recurrence_prep(_ptr(z), n_heads * dim, 0, dim, 0, 1.0, 0.0, _ptr(z), n_heads * dim, n_heads * dim, 2,
                                              _ptr(bias), None, 1.0, n_heads, None, 0, None, n, self._stream()))

    def gated_rmsnorm_heads(self, o: torch.Tensor, weight: torch.Tensor, gate: torch.Tensor, act: int, eps: float, n_heads: int,
                            vdim: int, out: torch.Tensor) -> None:
        """`gated_rmsnorm_act` with a weight over the concatenated heads [H * vdim]; gate [T, H * vdim] float32."""
        n = o.shape[0]
        _check(o, "o", torch.float32, (n, n_heads * vdim))
        _check(weight, "weight", torch.float32, (n_heads * vdim,))
        _check(gate, "gate", torch.float32, (n, n_heads * vdim))
        _check(out, "out", None, (n, n_heads * vdim))
        self._ok(self._lib.rb_gated_rmsnorm_heads(_ptr(o), _ptr(weight), vdim, _ptr(gate), n_heads * vdim, int(act), float(eps),
                                                  _ptr(out), dtype_code(out.dtype), n, n_heads, vdim, self._stream()))

    def heads_linear_part(self, x: torch.Tensor, x_head: int, w: torch.Tensor, y: torch.Tensor, y_head: int,
                          gate: Optional[torch.Tensor] = None, gate_col: int = 0, rope=None) -> None:
        """y[t, h, :N] = w[h]^T x[t, h, :K] with w [H, K, N]; a head of x takes x_head numbers, a head of y y_head.
        gate [T, >= gate_col + H] float32: head h's outputs times sigmoid(gate[:, gate_col + h]).  rope = (x_col, rot, cos, sin,
        style, y_col, tok_pos): the rot numbers at x_col of every head of x, rotated, go to y at y_col, zeros behind them."""
        h, k, n_out = w.shape
        n = x.shape[0]
        _check(x, "x", None, (n, h * x_head))
        _check(w, "w")
        _check(y, "y", None, (n, h * y_head))
        if x_head < k or y_head < n_out:
            raise KernelError("heads_linear_part: a head is shorter than the product's sizes")
        g_ptr, g_stride = None, 0
        if gate is not None:
            _check(gate, "gate", torch.float32)
            if gate.shape[0] != n or gate_col < 0 or gate_col + h > gate.shape[1]:
                raise KernelError("heads_linear_part: the gate's columns lie outside the rows")
            g_ptr, g_stride = gate.data_ptr() + 4 * gate_col, gate.shape[1]
        rot, x_col, y_col, cos, sin, style, tok_pos = -1, 0, 0, None, None, 0, None
        if rope is not None:
            x_col, rot, cos, sin, style, y_col, tok_pos = rope
            if x.dtype != torch.float32 or x_col + rot > x_head or y_col + rot > y_head or y_col < n_out:
                raise KernelError("heads_linear_part: the rotated part lies outside a head, or x is not float32")
            _check(tok_pos, "tok_pos", torch.int32, (n,))
            if rot:
                _check(cos, "cos", torch.float32)
                _check(sin, "sin", torch.float32, cos.shape)
                if cos.shape[1] != rot // 2:
                    raise KernelError("angle table width mismatch")
        self._ok(self._lib.rb_heads_linear_more(_ptr(x), dtype_code(x.dtype), x_head, _ptr(w), dtype_code(w.dtype), _ptr(y),
                                                dtype_code(y.dtype), y_head, n, h, n_out, k, g_ptr, g_stride, int(rot), int(x_col),
                                                int(y_col), _ptr(cos) if rot > 0 else None, _ptr(sin) if rot > 0 else None, int(style),
                                                _ptr(tok_pos), self._stream()))

    def latent_norm_rope_store(self, proj: torch.Tensor, q_rank: int, q_gain, cq, kv_rank: int, kv_gain, pages, rot: int, cos, sin,
                               style: int, ctx, block_table, eps: float, dtype: torch.dtype) -> None:
        """proj [T, q_rank + kv_rank + rot] float32: cq [T, q_rank] and the pages [*, 1, 64, W >= kv_rank + rot] get the two RMS
        norms, the pages also the last `rot` numbers rotated by the position, behind the latent, and zeros up to W."""
        n, width = proj.shape
        has_kv = kv_rank > 0
        _check(proj, "proj", torch.float32)
        if width < q_rank + ((kv_rank + rot) if has_kv else 0):
            raise KernelError("latent_norm_rope_store: rows too short for the down-projections and the rotated part")
        _check(q_gain, "q_gain", torch.float32, (q_rank,))
        _check(cq, "cq", dtype, (n, q_rank))
        page_width = 0
        if has_kv:
            _check(kv_gain, "kv_gain", torch.float32, (kv_rank,))
            _check(pages, "pages", dtype)
            page_width = pages.shape[-1]
            if tuple(pages.shape[1:3]) != (1, self.page_size) or page_width < kv_rank + rot:
                raise KernelError(f"latent pages have shape {tuple(pages.shape)}, expected [*, 1, {self.page_size}, >= {kv_rank + rot}]")
            _check(block_table, "block_table", torch.int32)
            if rot:
                _check(cos, "cos", torch.float32)
                _check(sin, "sin", torch.float32, cos.shape)
                if cos.shape[1] != rot // 2:
                    raise KernelError("angle table width mismatch")
        self._ok(self._lib.rb_latent_norm_rope_store(_ptr(proj), width, q_rank, _ptr(q_gain), _ptr(cq), q_rank, kv_rank, _ptr(kv_gain),
                                                     _ptr(pages) if has_kv else None, page_width, q_rank + kv_rank, rot if has_kv else 0,
                                                     _ptr(cos) if rot else None, _ptr(sin) if rot else None, int(style),
                                                     dtype_code(dtype), _ptr(ctx.tok_pos), _ptr(ctx.tok_seq),
                                                     _ptr(block_table) if has_kv else None, block_table.shape[1] if has_kv else 0,
                                                     float(eps), n, self._stream()))

    # ------------------------------------------------------------------ recorded steps
    def plan_begin(self) -> int:
        """From here to `plan_end` every launch of this thread is noted as well as issued; returns
        the plan's handle."""
        plan = self._lib.rb_plan_begin()
        if not plan:
            raise KernelError(self._lib.rb_last_error().decode("utf-8", "replace"))
        return plan

    def plan_end(self, plan: int) -> int:
        """Ends the recording; returns the number of launches the plan holds."""
        self._ok(self._lib.rb_plan_end(plan))
        return int(self._lib.rb_plan_calls(plan))

    def plan_replay(self, plan: int) -> None:
        """Issues the plan's launches again on torch's current stream, with the arguments they were
        recorded with: the memory those name must still be the step's own."""
        self._ok(self._lib.rb_plan_replay(plan, self._stream()))

    def plan_free(self, plan: int) -> None:
        self._lib.rb_plan_free(plan)

    # ------------------------------------------------------------------ load time
    def fill_normal(self, out: torch.Tensor, key: int, mean: float, std: float) -> None:
        """out[i] = mean + std * (the standard normal number that (key, i) fixes)."""
        _check(out, "out")
        self._ok(self._lib.rb_fill_normal(_ptr(out), dtype_code(out.dtype), out.numel(), int(key) & (2**64 - 1),
                                          float(mean), float(std), self._stream()))

    def place_rows(self, src: torch.Tensor, dst: torch.Tensor, row0: int = 0, block: Optional[int] = None,
                   period: Optional[int] = None, frag: bool = False) -> None:
        """Row r of src goes, cast to dst's dtype, to row row0 + (r // block) * period + r % block
        of dst (block: all rows, so that they follow one another from row0).  frag: dst is stored
        fragment-major (the matrix-core products' other layout of W; rows % 16 == 0, width % 32 == 0)."""
        _check(src, "src")
        _check(dst, "dst")
        if src.dim() != 2 or dst.dim() != 2 or src.shape[1] != dst.shape[1]:
            raise KernelError(f"place_rows: {tuple(src.shape)} does not fit into {tuple(dst.shape)}")
        n = src.shape[0]
        block = max(1, n) if block is None else int(block)
        period = block if period is None else int(period)
        self._ok(self._lib.rb_place_rows(_ptr(src), dtype_code(src.dtype), _ptr(dst), dtype_code(dst.dtype),
                                         int(bool(frag)), n, src.shape[1], dst.shape[0], int(row0), block, period,
                                         self._stream()))

    # ------------------------------------------------------------------ probes
    def probe_read(self, buf: torch.Tensor, sink: torch.Tensor, blocks: int = 2048, pieces: bool = False) -> None:
        """Reads every byte of `buf` once with `blocks` workgroups (see probe.hip).  pieces: every
        workgroup walks pieces of its own with non-temporal loads, as the decode products do."""
        _check(buf, "buf")
        _check(sink, "sink", torch.float32)
        nbytes = buf.numel() * buf.element_size()
        if nbytes % 16 != 0 or buf.data_ptr() % 16 != 0:
            raise KernelError("probe buffer must be 16-byte aligned and a multiple of 16 bytes long")
        self._ok(self._lib.rb_probe_read(_ptr(buf), nbytes, int(blocks), int(bool(pieces)), _ptr(sink), self._stream()))

    def probe_mfma(self, waves: int, iters: int, sink: torch.Tensor) -> float:
        """Runs the MFMA loop; returns the floating-point operations it performs."""
        _check(sink, "sink", torch.float32)
        self._ok(self._lib.rb_probe_mfma(int(waves), int(iters), _ptr(sink), self._stream()))
        return float(waves) * iters * 4 * 2 * 32 * 32 * 16


_lock = threading.Lock()
_instance: Optional[Kernels] = None


def kernels() -> Kernels:
    """The process-wide library, loaded (and built, if it is not) at first use."""
    global _instance
    with _lock:
        if _instance is None:
            _instance = Kernels()
        return _instance
