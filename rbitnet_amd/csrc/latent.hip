// Attention through a latent: every token leaves one vector c of kv_rank numbers in the cache, and each head's
// keys and values are products of c with matrices of that head.  The products are moved to the query's side, so that
// attention runs over the cached latents themselves, as one key/value head of size kv_rank that all query heads share:
//   score = q . (Wk c) = (Wk^T q) . c,      out = Wv (sum_j p_j c_j)
// Here: the RMS norms of the two down-projections with the cache write, and the per-head products on either side
// of attention.  float32 arithmetic; storage float32 or bfloat16.
#include <math.h>

#include "api.h"
#include "common.h"

// proj [T, stride] float32 holds, per token, q_rank numbers at column 0 and kv_rank numbers at column kv_col.
// cq[t] = rmsnorm(proj[t, 0:q_rank]) * q_gain; c = rmsnorm(proj[t, kv_col:kv_col + kv_rank]) * kv_gain goes into the
// token's place of the cache pages [pages, 1, 64, kv_rank].  Either half may be absent (rank 0).
template <typename TC>
__global__ void latent_norm_store_kernel(const float* __restrict__ proj, size_t stride, int q_rank,
                                         const float* __restrict__ q_gain, TC* __restrict__ cq, int kv_col, int kv_rank,
                                         const float* __restrict__ kv_gain, TC* __restrict__ pages, int page_width,
                                         const int32_t* __restrict__ tok_pos, const int32_t* __restrict__ tok_seq,
                                         const int32_t* __restrict__ block_table, int bt_stride, float eps, int rot_col = 0,
                                         int rot = 0, const float* __restrict__ cos_t = nullptr,
                                         const float* __restrict__ sin_t = nullptr, int style = 0) {
  __shared__ float scratch[16];
  const int t = blockIdx.x;
  const float* row = proj + (size_t)t * stride;
  if (q_rank > 0) {
    float ss = 0.f;
    for (int j = threadIdx.x; j < q_rank; j += blockDim.x) ss = fmaf(row[j], row[j], ss);
    const float f = 1.0f / sqrtf(block_sum(ss, scratch) / (float)q_rank + eps);
    for (int j = threadIdx.x; j < q_rank; j += blockDim.x) Num<TC>::store(cq + (size_t)t * q_rank + j, row[j] * f * q_gain[j]);
  }
  if (kv_rank > 0) {
    const int pos = tok_pos[t];
    const int page = block_table[(size_t)tok_seq[t] * bt_stride + pos / RB_PAGE];
    TC* dst = pages + ((size_t)page * RB_PAGE + (size_t)(pos % RB_PAGE)) * page_width;
    const float* src = row + kv_col;
    float ss = 0.f;
    for (int j = threadIdx.x; j < kv_rank; j += blockDim.x) ss = fmaf(src[j], src[j], ss);
    const float f = 1.0f / sqrtf(block_sum(ss, scratch) / (float)kv_rank + eps);
    for (int j = threadIdx.x; j < kv_rank; j += blockDim.x) Num<TC>::store(dst + j, src[j] * f * kv_gain[j]);
    // behind the latent: the row's `rot` numbers at rot_col rotated by the position (not normed), then zeros up to page_width
    if (page_width > kv_rank) {
      const int half = rot / 2;
      const float* rsrc = row + rot_col;
      const float* cr = cos_t + (size_t)pos * half;
      const float* sr = sin_t + (size_t)pos * half;
      TC* rdst = dst + kv_rank;
      for (int i = threadIdx.x; i < half; i += blockDim.x) {
        const int a = style == 0 ? 2 * i : i, b = style == 0 ? 2 * i + 1 : i + half;
        float y0, y1;
        rotate_pair(rsrc[a], rsrc[b], cr[i], sr[i], y0, y1);
        Num<TC>::store(rdst + a, y0);
        Num<TC>::store(rdst + b, y1);
      }
      for (int i = rot + threadIdx.x; i < page_width - kv_rank; i += blockDim.x) Num<TC>::store(rdst + i, 0.f);
    }
  }
}

extern "C" int rb_latent_norm_store(const float* proj, long long stride, int q_rank, const float* q_gain, void* cq,
                                    int kv_col, int kv_rank, const float* kv_gain, void* pages, int dtype,
                                    const int32_t* tok_pos, const int32_t* tok_seq, const int32_t* block_table,
                                    int bt_stride, float eps, int n_tokens, void* stream) {
  RB_RECORDED(rb_latent_norm_store(proj, stride, q_rank, q_gain, cq, kv_col, kv_rank, kv_gain, pages, dtype, tok_pos, tok_seq,
                                   block_table, bt_stride, eps, n_tokens, stream));
  RB_REQUIRE(n_tokens >= 0 && q_rank >= 0 && kv_rank >= 0 && kv_col >= 0, "rb_latent_norm_store: bad sizes");
  RB_REQUIRE(stride >= q_rank && stride >= (long long)kv_col + kv_rank, "rb_latent_norm_store: the row stride is too short");
  RB_REQUIRE(kv_rank == 0 || (pages && block_table), "rb_latent_norm_store: a latent needs cache pages");
  if (n_tokens == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  if (dtype == RB_F32)
    latent_norm_store_kernel<float><<<n_tokens, 256, 0, s>>>(proj, (size_t)stride, q_rank, q_gain, (float*)cq, kv_col, kv_rank,
                                                             kv_gain, (float*)pages, kv_rank, tok_pos, tok_seq, block_table, bt_stride, eps);
  else if (dtype == RB_BF16)
    latent_norm_store_kernel<bf16_t><<<n_tokens, 256, 0, s>>>(proj, (size_t)stride, q_rank, q_gain, (bf16_t*)cq, kv_col, kv_rank,
                                                              kv_gain, (bf16_t*)pages, kv_rank, tok_pos, tok_seq, block_table, bt_stride, eps);
  else
    RB_REQUIRE(false, "rb_latent_norm_store: unknown dtype %d", dtype);
  RB_LAUNCH_CHECK();
  return 0;
}

// ---------------------------------------------------------------- a product per head
// y[t, h, n] = sum_k w[h, k, n] * x[t, h, k]: H small matrices, stored [H, K, N] (the output index runs fastest, so
// that neighbouring lanes read neighbouring weights).  A workgroup of four waves takes HL_TOKENS tokens and 64 output
// columns of one head: the tokens' inputs in LDS, a lane per column with one sum per token; the waves share the inner
// index (wave w takes k = w, w + 4, ...), sixteen weights in flight per lane (the scheduler is told not to move a load
// down to its use: it would trade the registers for a trip to memory per weight), and add up through LDS in a fixed order.
#define HL_TOKENS 16
#define HL_WAVES 4
template <typename TX, typename TW, typename TY>
__global__ __launch_bounds__(RB_WAVE * HL_WAVES) void heads_linear_kernel(const TX* __restrict__ x, const TW* __restrict__ w,
                                                                          TY* __restrict__ y, int n_tokens, int n_heads, int n, int k,
                                                                          size_t x_hs, size_t y_hs, const float* __restrict__ gate,
                                                                          size_t gate_stride, int rot, int x_rot_col, int y_rot_col,
                                                                          const float* __restrict__ cos_t,
                                                                          const float* __restrict__ sin_t, int style,
                                                                          const int32_t* __restrict__ tok_pos, int n_col_tiles) {
  extern __shared__ float xs[];                  // [HL_TOKENS][k], then [HL_WAVES - 1][HL_TOKENS][64] partial sums
  float* part = xs + HL_TOKENS * k;
  const int t0 = blockIdx.x * HL_TOKENS, h = blockIdx.y;
  const int lane = threadIdx.x & (RB_WAVE - 1), wave = threadIdx.x / RB_WAVE;
  const int nt = n_tokens - t0 < HL_TOKENS ? n_tokens - t0 : HL_TOKENS;
  if ((int)blockIdx.z == n_col_tiles) {
    // one more workgroup per (tokens, head): the `rot` numbers at x_rot_col of the head, rotated by the token's position, go to
    // y at y_rot_col, and what lies behind them in the head of y becomes zero
    const int half = rot / 2, tail = (int)y_hs - y_rot_col - rot, per = half + tail;
    for (int idx = threadIdx.x; idx < nt * per; idx += blockDim.x) {
      const int tt = idx / per, i = idx - tt * per;
      const TX* src = x + ((size_t)(t0 + tt) * n_heads + h) * x_hs + x_rot_col;
      TY* dst = y + ((size_t)(t0 + tt) * n_heads + h) * y_hs + y_rot_col;
      if (i < half) {
        const size_t at = (size_t)tok_pos[t0 + tt] * half + i;
        const int a = style == 0 ? 2 * i : i, b = style == 0 ? 2 * i + 1 : i + half;
        float y0, y1;
        rotate_pair(Num<TX>::load(src + a), Num<TX>::load(src + b), cos_t[at], sin_t[at], y0, y1);
        Num<TY>::store(dst + a, y0);
        Num<TY>::store(dst + b, y1);
      } else {
        Num<TY>::store(dst + rot + (i - half), 0.f);
      }
    }
    return;
  }
  // the tokens' inputs, eight loads in flight per lane (a step of few tokens is a chain of trips to memory otherwise)
  for (int base = 0; base < HL_TOKENS * k; base += 8 * RB_WAVE * HL_WAVES) {
    float v[8];
#pragma unroll
    for (int it = 0; it < 8; ++it) {
      const int idx = base + it * RB_WAVE * HL_WAVES + threadIdx.x;
      const int tt = idx / k, kk = idx - tt * k;
      v[it] = (idx < HL_TOKENS * k && tt < nt) ? Num<TX>::load(x + ((size_t)(t0 + tt) * n_heads + h) * x_hs + kk) : 0.f;
    }
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int it = 0; it < 8; ++it) {
      const int idx = base + it * RB_WAVE * HL_WAVES + threadIdx.x;
      if (idx < HL_TOKENS * k) xs[idx] = v[it];
    }
  }
  __syncthreads();
  const int col = blockIdx.z * RB_WAVE + lane;
  const bool on = col < n;
  const TW* wh = w + (size_t)h * k * n + (on ? col : 0);
  float acc[HL_TOKENS];
#pragma unroll
  for (int tt = 0; tt < HL_TOKENS; ++tt) acc[tt] = 0.f;
  int kk = wave;
  for (; kk + 15 * HL_WAVES < k; kk += 16 * HL_WAVES) {
    float wv[16];
#pragma unroll
    for (int j = 0; j < 16; ++j) wv[j] = Num<TW>::load(wh + (size_t)(kk + j * HL_WAVES) * n);
    __builtin_amdgcn_sched_barrier(0);          // all sixteen loads are issued before the first is waited for
#pragma unroll
    for (int j = 0; j < 16; ++j)
#pragma unroll
      for (int tt = 0; tt < HL_TOKENS; ++tt) acc[tt] = fmaf(wv[j], xs[tt * k + kk + j * HL_WAVES], acc[tt]);
  }
  for (; kk < k; kk += HL_WAVES) {
    const float wv = Num<TW>::load(wh + (size_t)kk * n);
#pragma unroll
    for (int tt = 0; tt < HL_TOKENS; ++tt) acc[tt] = fmaf(wv, xs[tt * k + kk], acc[tt]);
  }
  if (wave > 0) {
#pragma unroll
    for (int tt = 0; tt < HL_TOKENS; ++tt) part[((wave - 1) * HL_TOKENS + tt) * RB_WAVE + lane] = acc[tt];
  }
  __syncthreads();
  if (wave > 0 || !on) return;
#pragma unroll
  for (int tt = 0; tt < HL_TOKENS; ++tt) {
    float v = acc[tt];
#pragma unroll
    for (int ww = 0; ww < HL_WAVES - 1; ++ww) v += part[(ww * HL_TOKENS + tt) * RB_WAVE + lane];
    if (tt < nt) {
      if (gate) v *= 1.0f / (1.0f + expf(-gate[(size_t)(t0 + tt) * gate_stride + h]));      // a gate per head on the way out
      Num<TY>::store(y + ((size_t)(t0 + tt) * n_heads + h) * y_hs + col, v);
    }
  }
}

struct HeadsLinearMore {      // what rides in the same launch: a gate per head on the outputs, a rotated part beside them
  const float* gate = nullptr;
  size_t gate_stride = 0;
  int rot = 0, x_rot_col = 0, y_rot_col = 0, style = 0;
  const float* cos_t = nullptr;
  const float* sin_t = nullptr;
  const int32_t* tok_pos = nullptr;
  bool has_rot = false;
};
template <typename TX, typename TW, typename TY>
static void launch_heads_linear(const void* x, const void* w, void* y, int n_tokens, int n_heads, int n, int k, size_t x_hs,
                                size_t y_hs, hipStream_t s, const HeadsLinearMore& m = HeadsLinearMore()) {
  const int n_col_tiles = (n + RB_WAVE - 1) / RB_WAVE;
  dim3 grid((n_tokens + HL_TOKENS - 1) / HL_TOKENS, n_heads, n_col_tiles + (m.has_rot ? 1 : 0));
  const size_t lds = ((size_t)HL_TOKENS * k + (size_t)(HL_WAVES - 1) * HL_TOKENS * RB_WAVE) * sizeof(float);
  heads_linear_kernel<TX, TW, TY><<<grid, RB_WAVE * HL_WAVES, lds, s>>>((const TX*)x, (const TW*)w, (TY*)y, n_tokens, n_heads, n, k, x_hs,
                                                                        y_hs, m.gate, m.gate_stride, m.rot, m.x_rot_col, m.y_rot_col,
                                                                        m.cos_t, m.sin_t, m.style, m.tok_pos, n_col_tiles);
}

extern "C" int rb_heads_linear(const void* x, int x_dtype, const void* w, int w_dtype, void* y, int y_dtype, int n_tokens,
                               int n_heads, int n, int k, void* stream) {
  RB_RECORDED(rb_heads_linear(x, x_dtype, w, w_dtype, y, y_dtype, n_tokens, n_heads, n, k, stream));
  return rb_heads_linear_strided(x, x_dtype, k, w, w_dtype, y, y_dtype, n, n_tokens, n_heads, n, k, stream);
}

// The same with a head of x taking x_head_stride numbers (the first k of them are read) and a head of y y_head_stride
// (the first n are written): products on a part of every head, into a part of every head.
extern "C" int rb_heads_linear_strided(const void* x, int x_dtype, long long x_head_stride, const void* w, int w_dtype, void* y,
                                       int y_dtype, long long y_head_stride, int n_tokens, int n_heads, int n, int k, void* stream) {
  RB_RECORDED(rb_heads_linear_strided(x, x_dtype, x_head_stride, w, w_dtype, y, y_dtype, y_head_stride, n_tokens, n_heads, n, k,
                                      stream));
  return rb_heads_linear_more(x, x_dtype, x_head_stride, w, w_dtype, y, y_dtype, y_head_stride, n_tokens, n_heads, n, k, nullptr, 0,
                              -1, 0, 0, nullptr, nullptr, 0, nullptr, stream);
}

// The same with two things in the same launch.  gate (float32, rows gate_stride apart; null: none): head h's outputs of token t
// are multiplied by sigmoid(gate[t * gate_stride + h]).  rot >= 0 (rot < 0: none): the `rot` numbers at x_rot_col of every head
// of x, rotated by the token's position (cos, sin [positions, rot / 2]; style 0: 2i with 2i + 1, 1: i with i + rot / 2), go to
// y at y_rot_col, and what lies behind them in a head of y becomes zero.
extern "C" int rb_heads_linear_more(const void* x, int x_dtype, long long x_head_stride, const void* w, int w_dtype, void* y,
                                    int y_dtype, long long y_head_stride, int n_tokens, int n_heads, int n, int k, const float* gate,
                                    long long gate_stride, int rot, int x_rot_col, int y_rot_col, const float* cos, const float* sin,
                                    int style, const int32_t* tok_pos, void* stream) {
  RB_RECORDED(rb_heads_linear_more(x, x_dtype, x_head_stride, w, w_dtype, y, y_dtype, y_head_stride, n_tokens, n_heads, n, k, gate,
                                   gate_stride, rot, x_rot_col, y_rot_col, cos, sin, style, tok_pos, stream));
  HeadsLinearMore more;
  more.gate = gate;
  more.gate_stride = (size_t)gate_stride;
  RB_REQUIRE(gate == nullptr || gate_stride >= n_heads, "rb_heads_linear: the gate's rows are shorter than the heads");
  if (rot >= 0) {
    RB_REQUIRE(rot % 2 == 0 && x_rot_col >= 0 && y_rot_col >= n && x_head_stride >= (long long)x_rot_col + rot &&
                   y_head_stride >= (long long)y_rot_col + rot,
               "rb_heads_linear: the rotated part lies outside a head, or over the product's outputs");
    RB_REQUIRE(rot == 0 || (cos && sin && tok_pos && (style == 0 || style == 1)), "rb_heads_linear: a rotation needs its tables");
    more.has_rot = y_head_stride > y_rot_col;
    more.rot = rot;
    more.x_rot_col = x_rot_col;
    more.y_rot_col = y_rot_col;
    more.style = style;
    more.cos_t = cos;
    more.sin_t = sin;
    more.tok_pos = tok_pos;
  }
  RB_REQUIRE(n_tokens >= 0 && n_heads > 0 && n_heads <= 65535 && n > 0 && n <= 65535 * 64 && k > 0, "rb_heads_linear: bad sizes");
  RB_REQUIRE(k <= 768, "rb_heads_linear: inner size %d not supported (at most 768)", k);
  RB_REQUIRE(x_head_stride >= k && y_head_stride >= n, "rb_heads_linear: a head's stride is shorter than the head");
  if (n_tokens == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  const size_t xs = (size_t)x_head_stride, ys = (size_t)y_head_stride;
  const int key = x_dtype * 4 + w_dtype * 2 + y_dtype;
  switch (key) {
    case 0: launch_heads_linear<float, float, float>(x, w, y, n_tokens, n_heads, n, k, xs, ys, s, more); break;
    case 3: launch_heads_linear<float, bf16_t, bf16_t>(x, w, y, n_tokens, n_heads, n, k, xs, ys, s, more); break;
    case 6: launch_heads_linear<bf16_t, bf16_t, float>(x, w, y, n_tokens, n_heads, n, k, xs, ys, s, more); break;
    case 7: launch_heads_linear<bf16_t, bf16_t, bf16_t>(x, w, y, n_tokens, n_heads, n, k, xs, ys, s, more); break;
    case 2: launch_heads_linear<float, bf16_t, float>(x, w, y, n_tokens, n_heads, n, k, xs, ys, s, more); break;
    default: RB_REQUIRE(false, "rb_heads_linear: this combination of types is not built (x %d, w %d, y %d)", x_dtype, w_dtype, y_dtype);
  }
  RB_LAUNCH_CHECK();
  return 0;
}

// ---------------------------------------------------------------- a rotated part beside the latent
// Where a head's key is a part made from the latent beside a rotated part that all heads share, the cache holds per token
// the latent c and, behind it, that rotated part: one key/value head of page_width >= kv_rank + rot numbers (the rest
// zeros), and a query is [Wk^T q_unrotated, rotate(q_rotated)] in the same layout.
// rb_latent_norm_store with that: the `rot` numbers at rot_col of a row of proj are rotated by the token's position
// (style 0: 2i with 2i + 1; 1: i with i + rot / 2; cos, sin [positions, rot / 2]) and stored behind the latent, by the same
// launch.
extern "C" int rb_latent_norm_rope_store(const float* proj, long long stride, int q_rank, const float* q_gain, void* cq, int kv_col,
                                         int kv_rank, const float* kv_gain, void* pages, int page_width, int rot_col, int rot,
                                         const float* cos, const float* sin, int style, int dtype, const int32_t* tok_pos,
                                         const int32_t* tok_seq, const int32_t* block_table, int bt_stride, float eps, int n_tokens,
                                         void* stream) {
  RB_RECORDED(rb_latent_norm_rope_store(proj, stride, q_rank, q_gain, cq, kv_col, kv_rank, kv_gain, pages, page_width, rot_col, rot,
                                        cos, sin, style, dtype, tok_pos, tok_seq, block_table, bt_stride, eps, n_tokens, stream));
  RB_REQUIRE(n_tokens >= 0 && q_rank >= 0 && kv_rank >= 0 && kv_col >= 0 && rot >= 0 && rot % 2 == 0 && rot_col >= 0,
             "rb_latent_norm_rope_store: bad sizes");
  RB_REQUIRE(stride >= q_rank && stride >= (long long)kv_col + kv_rank && stride >= (long long)rot_col + rot,
             "rb_latent_norm_rope_store: the row stride is too short");
  RB_REQUIRE(kv_rank == 0 || (pages && block_table && page_width >= kv_rank + rot),
             "rb_latent_norm_rope_store: a latent needs cache pages that hold it and the rotated part");
  RB_REQUIRE(rot == 0 || kv_rank == 0 || (cos && sin && (style == 0 || style == 1)), "rb_latent_norm_rope_store: a rotation needs its tables");
  RB_REQUIRE(dtype == RB_F32 || dtype == RB_BF16, "rb_latent_norm_rope_store: unknown dtype %d", dtype);
  if (n_tokens == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  if (dtype == RB_F32)
    latent_norm_store_kernel<float><<<n_tokens, 256, 0, s>>>(proj, (size_t)stride, q_rank, q_gain, (float*)cq, kv_col, kv_rank,
                                                             kv_gain, (float*)pages, page_width, tok_pos, tok_seq, block_table,
                                                             bt_stride, eps, rot_col, rot, cos, sin, style);
  else
    latent_norm_store_kernel<bf16_t><<<n_tokens, 256, 0, s>>>(proj, (size_t)stride, q_rank, q_gain, (bf16_t*)cq, kv_col, kv_rank,
                                                              kv_gain, (bf16_t*)pages, page_width, tok_pos, tok_seq, block_table,
                                                              bt_stride, eps, rot_col, rot, cos, sin, style);
  RB_LAUNCH_CHECK();
  return 0;
}
