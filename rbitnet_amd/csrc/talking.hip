// Attention whose heads' scores are mixed before the softmax, and what stands around it.
//
//   rb_embed_scaled_pos   x[t] = table[id[t]] * scale + positions[pos[t]]
//   rb_scale              x <- s x
//   rb_bias_norm_store    q, k, v of a step: + bias; q and k heads / sqrt(mean(head^2) + eps); q to q_out, k and v to the pages
//   rb_attention_mixed    score[g, j] = q_g . k_kv(g),j * scale;  mixed[h, j] = sum_g talk[h, g] score[g, j];  softmax over the
//                         keys that the token sees (causal, optionally the token's chunk of `chunk` positions counted from
//                         position 0, optionally the last `window` keys);  out_h = sum_j p[h, j] v_kv(h),j
// All arithmetic in float32; storage float32 or bfloat16.  One workgroup takes a token and all of its heads, since every
// head's weights need every head's scores: the keys go by in tiles of 64 (a page), the scores of all heads for a tile
// lie in LDS, are mixed there, and go through an online softmax per head.  The same kernel serves a prompt's tokens and
// single tokens, so a token's result does not depend on how its sequence was cut into steps.
#include <math.h>

#include "api.h"
#include "common.h"

// ---------------------------------------------------------------- embedding with a scale and learned positions
template <typename T>
__global__ void embed_scaled_pos_kernel(const T* __restrict__ table, const int32_t* __restrict__ ids, float scale,
                                        const T* __restrict__ positions, const int32_t* __restrict__ tok_pos,
                                        float* __restrict__ x, int width) {
  const int t = blockIdx.x;
  const T* row = table + (size_t)ids[t] * width;
  const T* pr = positions ? positions + (size_t)tok_pos[t] * width : nullptr;
  float* dst = x + (size_t)t * width;
  for (int j = threadIdx.x; j < width; j += blockDim.x) {
    const float e = Num<T>::load(row + j) * scale;
    dst[j] = pr ? e + Num<T>::load(pr + j) : e;
  }
}

extern "C" int rb_embed_scaled_pos(const void* table, int table_dtype, const int32_t* ids, float scale, const void* positions,
                                   const int32_t* tok_pos, float* x, int n_tokens, int width, void* stream) {
  RB_RECORDED(rb_embed_scaled_pos(table, table_dtype, ids, scale, positions, tok_pos, x, n_tokens, width, stream));
  RB_REQUIRE(n_tokens >= 0 && width > 0, "rb_embed_scaled_pos: bad sizes %d x %d", n_tokens, width);
  RB_REQUIRE(positions == nullptr || tok_pos != nullptr, "rb_embed_scaled_pos: a table of positions needs the tokens' positions");
  if (n_tokens == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  const int threads = width >= 256 ? 256 : 64;
  if (table_dtype == RB_F32)
    embed_scaled_pos_kernel<float><<<n_tokens, threads, 0, s>>>((const float*)table, ids, scale, (const float*)positions, tok_pos, x, width);
  else if (table_dtype == RB_BF16)
    embed_scaled_pos_kernel<bf16_t><<<n_tokens, threads, 0, s>>>((const bf16_t*)table, ids, scale, (const bf16_t*)positions, tok_pos, x, width);
  else
    RB_REQUIRE(false, "rb_embed_scaled_pos: unknown dtype %d", table_dtype);
  RB_LAUNCH_CHECK();
  return 0;
}

__global__ void scale_kernel(float* __restrict__ x, float s, size_t n) {
  for (size_t e = (size_t)blockIdx.x * blockDim.x + threadIdx.x; e < n; e += (size_t)gridDim.x * blockDim.x) x[e] *= s;
}

extern "C" int rb_scale(float* x, float s, long long n, void* stream) {
  RB_RECORDED(rb_scale(x, s, n, stream));
  RB_REQUIRE(n >= 0, "rb_scale: bad size");
  if (n == 0) return 0;
  const size_t blocks = ((size_t)n + 255) / 256;
  scale_kernel<<<(int)(blocks < 65535 ? blocks : 65535), 256, 0, (hipStream_t)stream>>>(x, s, (size_t)n);
  RB_LAUNCH_CHECK();
  return 0;
}

// ---------------------------------------------------------------- bias, unit root mean square per head, pages
// A row of qkv (row_width floats apart) holds Hq query heads and Hk key heads of `dim` numbers and Hk value heads of
// `vdim`; without pages of its own (k_pages null) only the query heads.  A wave takes a head: the row's numbers plus
// their bias, and for query and key heads (norm != 0) divided by sqrt(mean of their squares + eps).  Heads are laid
// out with `pad` numbers, zeros behind their own.
template <typename TC>
__global__ void bias_norm_store_kernel(const float* __restrict__ qkv, size_t row_width, const float* __restrict__ bias, int norm,
                                       float eps, TC* __restrict__ q_out, TC* __restrict__ k_pages, TC* __restrict__ v_pages,
                                       const int32_t* __restrict__ tok_pos, const int32_t* __restrict__ tok_seq,
                                       const int32_t* __restrict__ block_table, int bt_stride, int n_heads, int n_kv, int dim,
                                       int vdim, int pad) {
  const int t = blockIdx.x;
  const int lane = threadIdx.x & (RB_WAVE - 1), wave = threadIdx.x / RB_WAVE, n_waves = blockDim.x / RB_WAVE;
  const int pos = tok_pos[t];
  const float* src = qkv + (size_t)t * row_width;
  size_t page_base = 0;
  if (k_pages) {
    const int page = block_table[(size_t)tok_seq[t] * bt_stride + pos / RB_PAGE];
    page_base = ((size_t)page * n_kv) * RB_PAGE * pad + (size_t)(pos % RB_PAGE) * pad;
  }
  const int n_all = n_heads + (k_pages ? 2 * n_kv : 0);
  for (int h = wave; h < n_all; h += n_waves) {
    const bool is_v = h >= n_heads + n_kv;
    const int size = is_v ? vdim : dim;
    const size_t col = is_v ? (size_t)(n_heads + n_kv) * dim + (size_t)(h - n_heads - n_kv) * vdim : (size_t)h * dim;
    TC* dst = h < n_heads ? q_out + ((size_t)t * n_heads + h) * pad
              : !is_v     ? k_pages + page_base + (size_t)(h - n_heads) * RB_PAGE * pad
                          : v_pages + page_base + (size_t)(h - n_heads - n_kv) * RB_PAGE * pad;
    float factor = 1.0f;
    if (norm && !is_v) {
      float ss = 0.f;
      for (int d = lane; d < size; d += RB_WAVE) {
        const float v = src[col + d] + (bias ? bias[col + d] : 0.f);
        ss = fmaf(v, v, ss);
      }
      ss = wave_sum(ss);
      factor = 1.0f / sqrtf(ss / (float)size + eps);
    }
    for (int d = lane; d < pad; d += RB_WAVE) {
      float v = 0.f;
      if (d < size) v = (src[col + d] + (bias ? bias[col + d] : 0.f)) * factor;
      Num<TC>::store(dst + d, v);
    }
  }
}

extern "C" int rb_bias_norm_store(const float* qkv, long long row_width, const float* bias, int norm, float eps, void* q_out,
                                  void* k_pages, void* v_pages, int cache_dtype, const int32_t* tok_pos, const int32_t* tok_seq,
                                  const int32_t* block_table, int bt_stride, int n_tokens, int n_heads, int n_kv_heads, int dim,
                                  int vdim, int pad, void* stream) {
  RB_RECORDED(rb_bias_norm_store(qkv, row_width, bias, norm, eps, q_out, k_pages, v_pages, cache_dtype, tok_pos, tok_seq, block_table,
                                 bt_stride, n_tokens, n_heads, n_kv_heads, dim, vdim, pad, stream));
  RB_REQUIRE(n_tokens >= 0 && n_heads > 0 && n_kv_heads >= 0 && dim > 0 && vdim > 0 && pad >= dim && pad >= vdim,
             "rb_bias_norm_store: bad sizes T=%d Hq=%d Hk=%d dim=%d vdim=%d pad=%d", n_tokens, n_heads, n_kv_heads, dim, vdim, pad);
  RB_REQUIRE((k_pages == nullptr) == (v_pages == nullptr), "rb_bias_norm_store: keys and values go to pages together");
  const long long need = k_pages ? (long long)(n_heads + n_kv_heads) * dim + (long long)n_kv_heads * vdim : (long long)n_heads * dim;
  RB_REQUIRE(row_width >= need, "rb_bias_norm_store: a row of %lld numbers does not hold the heads (%lld)", row_width, need);
  RB_REQUIRE(k_pages == nullptr || (block_table != nullptr && tok_seq != nullptr && n_kv_heads > 0), "rb_bias_norm_store: pages need a table");
  if (n_tokens == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  if (cache_dtype == RB_F32)
    bias_norm_store_kernel<float><<<n_tokens, 256, 0, s>>>(qkv, (size_t)row_width, bias, norm, eps, (float*)q_out, (float*)k_pages,
                                                           (float*)v_pages, tok_pos, tok_seq, block_table, bt_stride, n_heads,
                                                           n_kv_heads, dim, vdim, pad);
  else if (cache_dtype == RB_BF16)
    bias_norm_store_kernel<bf16_t><<<n_tokens, 256, 0, s>>>(qkv, (size_t)row_width, bias, norm, eps, (bf16_t*)q_out, (bf16_t*)k_pages,
                                                            (bf16_t*)v_pages, tok_pos, tok_seq, block_table, bt_stride, n_heads,
                                                            n_kv_heads, dim, vdim, pad);
  else
    RB_REQUIRE(false, "rb_bias_norm_store: unknown dtype %d", cache_dtype);
  RB_LAUNCH_CHECK();
  return 0;
}

// ---------------------------------------------------------------- attention with mixed heads, any sizes
#define TK_TILE 64          // keys a tile: a page
#define TK_THREADS 256
#define TK_MAX_ACC 32       // outputs a thread: heads * pad <= TK_THREADS * TK_MAX_ACC
#define TK_MAX_HEADS 64

// first and last key that the token at `pos` sees
__device__ __forceinline__ void visible_range(int pos, int chunk, int window, int& lo, int& hi) {
  lo = 0;
  hi = pos;
  if (chunk > 0) lo = pos / chunk * chunk;
  if (window > 0 && pos - window + 1 > lo) lo = pos - window + 1;
}

template <typename TC>
__global__ __launch_bounds__(TK_THREADS) void attention_mixed_kernel(
    const TC* __restrict__ q, const TC* __restrict__ k_pages, const TC* __restrict__ v_pages, TC* __restrict__ out,
    const int32_t* __restrict__ tok_pos, const int32_t* __restrict__ tok_seq, const int32_t* __restrict__ block_table, int bt_stride,
    int n_heads, int n_kv, int pad, float scale, const float* __restrict__ talk, int chunk, int window) {
  extern __shared__ float lds[];
  float* qs = lds;                                   // [H, pad]
  float* raw = qs + (size_t)n_heads * pad;           // [H, 64]: the heads' own scores of a tile
  float* mixed = raw + n_heads * TK_TILE;            // [H, 64]: mixed scores, then the weights
  float* tk = mixed + n_heads * TK_TILE;             // [H, H]
  float* alpha = tk + n_heads * n_heads;             // [H]: what a head's sums so far are multiplied by
  float* denom = alpha + n_heads;                    // [H]
  const int t = blockIdx.x, tid = threadIdx.x;
  const int lane = tid & (RB_WAVE - 1), wave = tid / RB_WAVE;
  const int pos = tok_pos[t];
  const int group = n_heads / n_kv;
  int lo, hi;
  visible_range(pos, chunk, window, lo, hi);
  for (int i = tid; i < n_heads * pad; i += TK_THREADS) qs[i] = Num<TC>::load(q + (size_t)t * n_heads * pad + i);
  for (int i = tid; i < n_heads * n_heads; i += TK_THREADS) tk[i] = talk ? talk[i] : ((i / n_heads == i % n_heads) ? 1.f : 0.f);
  float acc[TK_MAX_ACC];
#pragma unroll
  for (int i = 0; i < TK_MAX_ACC; ++i) acc[i] = 0.f;
  // heads wave, wave + 4, ...: their running maxima and sums live in this wave's registers (the same in every lane)
  float run_max[TK_MAX_HEADS / 4], run_sum[TK_MAX_HEADS / 4];
#pragma unroll
  for (int i = 0; i < TK_MAX_HEADS / 4; ++i) {
    run_max[i] = -INFINITY;
    run_sum[i] = 0.f;
  }
  const int32_t* bt = block_table + (size_t)tok_seq[t] * bt_stride;
  const size_t head_stride = (size_t)RB_PAGE * pad;
  __syncthreads();
  for (int tile = lo / TK_TILE; tile <= hi / TK_TILE; ++tile) {
    const size_t page_base = (size_t)bt[tile] * n_kv * head_stride;
    const int j0 = tile * TK_TILE;
    // ---- the heads' own scores
    for (int idx = tid; idx < n_heads * TK_TILE; idx += TK_THREADS) {
      const int g = idx / TK_TILE, j = idx - g * TK_TILE;
      float s = 0.f;
      if (j0 + j >= lo && j0 + j <= hi) {
        const TC* kr = k_pages + page_base + (size_t)(g / group) * head_stride + (size_t)j * pad;
        const float* qr = qs + (size_t)g * pad;
        for (int d = 0; d < pad; ++d) s = fmaf(qr[d], Num<TC>::load(kr + d), s);
        s *= scale;
      }
      raw[idx] = s;
    }
    __syncthreads();
    // ---- mixed over the heads
    for (int idx = tid; idx < n_heads * TK_TILE; idx += TK_THREADS) {
      const int h = idx / TK_TILE, j = idx - h * TK_TILE;
      float s = -INFINITY;
      if (j0 + j >= lo && j0 + j <= hi) {
        s = 0.f;
        for (int g = 0; g < n_heads; ++g) s = fmaf(tk[h * n_heads + g], raw[g * TK_TILE + j], s);
      }
      mixed[idx] = s;
    }
    __syncthreads();
    // ---- online softmax, a wave a head: lane j holds key j of the tile
#pragma unroll
    for (int i = 0; i < TK_MAX_HEADS / 4; ++i) {
      const int h = wave + 4 * i;
      if (h < n_heads) {
        const float s = mixed[h * TK_TILE + lane];
        const float m_new = fmaxf(run_max[i], wave_max(s));          // a tile holds at least one visible key
        const float p = s == -INFINITY ? 0.f : expf(s - m_new);
        const float a = run_max[i] == -INFINITY ? 0.f : expf(run_max[i] - m_new);
        run_sum[i] = run_sum[i] * a + wave_sum(p);
        run_max[i] = m_new;
        mixed[h * TK_TILE + lane] = p;
        if (lane == 0) {
          alpha[h] = a;
          denom[h] = run_sum[i];
        }
      }
    }
    __syncthreads();
    // ---- weighted sums of the values
    const int j_first = lo > j0 ? lo - j0 : 0, j_last = hi - j0 < TK_TILE - 1 ? hi - j0 : TK_TILE - 1;
#pragma unroll
    for (int i = 0; i < TK_MAX_ACC; ++i) {
      const int idx = tid + TK_THREADS * i;
      if (idx < n_heads * pad) {
        const int h = idx / pad, d = idx - h * pad;
        const TC* vr = v_pages + page_base + (size_t)(h / group) * head_stride + d;
        const float* pr = mixed + h * TK_TILE;
        float a = acc[i] * alpha[h];
        for (int j = j_first; j <= j_last; ++j) a = fmaf(pr[j], Num<TC>::load(vr + (size_t)j * pad), a);
        acc[i] = a;
      }
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < TK_MAX_ACC; ++i) {
    const int idx = tid + TK_THREADS * i;
    if (idx < n_heads * pad) Num<TC>::store(out + (size_t)t * n_heads * pad + idx, acc[i] / denom[idx / pad]);
  }
}

extern "C" int rb_attention_mixed(const void* q, const void* k_pages, const void* v_pages, void* out, int dtype,
                                  const int32_t* tok_pos, const int32_t* tok_seq, const int32_t* block_table, int bt_stride,
                                  int n_tokens, int n_heads, int n_kv_heads, int head_dim, float scale, const float* talk, int chunk,
                                  int window, void* stream) {
  RB_RECORDED(rb_attention_mixed(q, k_pages, v_pages, out, dtype, tok_pos, tok_seq, block_table, bt_stride, n_tokens, n_heads,
                                 n_kv_heads, head_dim, scale, talk, chunk, window, stream));
  RB_REQUIRE(n_tokens >= 0 && n_heads > 0 && n_kv_heads > 0 && n_heads % n_kv_heads == 0 && head_dim > 0 && chunk >= 0 && window >= 0,
             "rb_attention_mixed: bad sizes T=%d Hq=%d Hk=%d D=%d", n_tokens, n_heads, n_kv_heads, head_dim);
  RB_REQUIRE(n_heads <= TK_MAX_HEADS && (long long)n_heads * head_dim <= (long long)TK_THREADS * TK_MAX_ACC,
             "rb_attention_mixed: %d heads of %d numbers are more than a workgroup takes (at most %d heads, %d numbers in all)",
             n_heads, head_dim, TK_MAX_HEADS, TK_THREADS * TK_MAX_ACC);
  if (n_tokens == 0) return 0;
  const size_t lds = sizeof(float) * ((size_t)n_heads * head_dim + 2 * (size_t)n_heads * TK_TILE + (size_t)n_heads * n_heads + 2 * n_heads);
  RB_REQUIRE(lds <= 160 * 1024, "rb_attention_mixed: %zu bytes of LDS are more than a workgroup has", lds);
  hipStream_t s = (hipStream_t)stream;
  if (dtype == RB_F32) {
    if (lds > 64 * 1024)
      RB_REQUIRE(hipFuncSetAttribute((const void*)attention_mixed_kernel<float>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) == hipSuccess,
                 "rb_attention_mixed: cannot have %zu bytes of LDS", lds);
    attention_mixed_kernel<float><<<n_tokens, TK_THREADS, lds, s>>>((const float*)q, (const float*)k_pages, (const float*)v_pages, (float*)out,
                                                                    tok_pos, tok_seq, block_table, bt_stride, n_heads, n_kv_heads, head_dim,
                                                                    scale, talk, chunk, window);
  } else if (dtype == RB_BF16) {
    if (lds > 64 * 1024)
      RB_REQUIRE(hipFuncSetAttribute((const void*)attention_mixed_kernel<bf16_t>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) == hipSuccess,
                 "rb_attention_mixed: cannot have %zu bytes of LDS", lds);
    attention_mixed_kernel<bf16_t><<<n_tokens, TK_THREADS, lds, s>>>((const bf16_t*)q, (const bf16_t*)k_pages, (const bf16_t*)v_pages,
                                                                     (bf16_t*)out, tok_pos, tok_seq, block_table, bt_stride, n_heads,
                                                                     n_kv_heads, head_dim, scale, talk, chunk, window);
  } else {
    RB_REQUIRE(false, "rb_attention_mixed: unknown dtype %d", dtype);
  }
  RB_LAUNCH_CHECK();
  return 0;
}
