// What stands around attention when a head's keys and values differ in size or only a part of a head is rotated, a
// gate per head on attention's output, and the mean of two mixers' outputs after a norm of each.  float32 arithmetic.
#include <math.h>

#include "api.h"
#include "common.h"

// ---------------------------------------------------------------- rotation of a part of a head, heads padded for the cache
// A row of qkv holds Hq query heads and Hk key heads of `dim` numbers and Hk value heads of `vdim`.  Of every query and
// key head the first `rot` numbers are rotated, i paired with i + rot / 2, by the angles of the token's position
// (cos, sin [positions, rot / 2]); the rest pass.  Queries go to q_out [T, Hq, pad], keys and values to the token's
// place in pages [*, Hk, 64, pad]; what lies beyond a head's own size is zero, so that a kernel made for one head size
// `pad` computes the same scores and the same sums.
template <typename TC>
__global__ void rope_store_kernel(const float* __restrict__ qkv, size_t row_width, const float* __restrict__ cos_t,
                                  const float* __restrict__ sin_t, int rot, TC* __restrict__ q_out, TC* __restrict__ k_pages,
                                  TC* __restrict__ v_pages, const int32_t* __restrict__ tok_pos,
                                  const int32_t* __restrict__ tok_seq, const int32_t* __restrict__ block_table, int bt_stride,
                                  int n_heads, int n_kv, int dim, int vdim, int pad) {
  const int t = blockIdx.x;
  const int pos = tok_pos[t];
  const int half = rot / 2;
  const float* src = qkv + (size_t)t * row_width;
  const float* cr = cos_t + (size_t)pos * half;
  const float* sr = sin_t + (size_t)pos * half;
  size_t page_base = 0;
  if (k_pages) {
    const int page = block_table[(size_t)tok_seq[t] * bt_stride + pos / RB_PAGE];
    page_base = ((size_t)page * n_kv) * RB_PAGE * pad + (size_t)(pos % RB_PAGE) * pad;
  }
  const int n_rot_heads = n_heads + (k_pages ? n_kv : 0);
  for (int idx = threadIdx.x; idx < n_rot_heads * pad; idx += blockDim.x) {
    const int h = idx / pad, d = idx - h * pad;
    const float* hp = src + (size_t)h * dim;
    float y = 0.f;
    if (d < half) {
      float y1;
      rotate_pair(hp[d], hp[d + half], cr[d], sr[d], y, y1);
    } else if (d < rot) {
      float y0;
      rotate_pair(hp[d - half], hp[d], cr[d - half], sr[d - half], y0, y);
    } else if (d < dim) {
      y = hp[d];
    }
    TC* dst = h < n_heads ? q_out + ((size_t)t * n_heads + h) * pad
                          : k_pages + page_base + (size_t)(h - n_heads) * RB_PAGE * pad;
    Num<TC>::store(dst + d, y);
  }
  if (v_pages) {
    const float* vsrc = src + (size_t)(n_heads + n_kv) * dim;
    for (int idx = threadIdx.x; idx < n_kv * pad; idx += blockDim.x) {
      const int h = idx / pad, d = idx - h * pad;
      Num<TC>::store(v_pages + page_base + (size_t)h * RB_PAGE * pad + d, d < vdim ? vsrc[(size_t)h * vdim + d] : 0.f);
    }
  }
}

// The same with four numbers a thread (16-byte loads, 8- or 16-byte stores), for sizes that are multiples of 4 and a
// rotated part that is a multiple of 8: a group of four lies wholly in the first half of the rotated part, in its
// second half, behind it, or in the padding.
__device__ __forceinline__ void store4(float* p, float a, float b, float c, float d) { *reinterpret_cast<float4*>(p) = make_float4(a, b, c, d); }
__device__ __forceinline__ void store4(bf16_t* p, float a, float b, float c, float d) {
  *reinterpret_cast<uint2*>(p) = make_uint2(pack_bf16x2(a, b), pack_bf16x2(c, d));
}
template <typename TC>
__global__ void rope_store_vec_kernel(const float* __restrict__ qkv, size_t row_width, const float* __restrict__ cos_t,
                                      const float* __restrict__ sin_t, int rot, TC* __restrict__ q_out, TC* __restrict__ k_pages,
                                      TC* __restrict__ v_pages, const int32_t* __restrict__ tok_pos,
                                      const int32_t* __restrict__ tok_seq, const int32_t* __restrict__ block_table, int bt_stride,
                                      int n_heads, int n_kv, int dim, int vdim, int pad) {
  const int t = blockIdx.x;
  const int pos = tok_pos[t];
  const int half = rot / 2;
  const float* src = qkv + (size_t)t * row_width;
  const float* cr = cos_t + (size_t)pos * half;
  const float* sr = sin_t + (size_t)pos * half;
  size_t page_base = 0;
  if (k_pages) {
    const int page = block_table[(size_t)tok_seq[t] * bt_stride + pos / RB_PAGE];
    page_base = ((size_t)page * n_kv) * RB_PAGE * pad + (size_t)(pos % RB_PAGE) * pad;
  }
  const int n_rot_heads = n_heads + (k_pages ? n_kv : 0);
  const int quads = pad / 4;
  for (int idx = threadIdx.x; idx < n_rot_heads * quads; idx += blockDim.x) {
    const int h = idx / quads, d = 4 * (idx - h * quads);
    const float* hp = src + (size_t)h * dim;
    float4 y = make_float4(0.f, 0.f, 0.f, 0.f);
    if (d < rot) {
      const bool first = d < half;
      const int i = first ? d : d - half;                       // the pairs' index
      const float4 a = *reinterpret_cast<const float4*>(hp + i), b = *reinterpret_cast<const float4*>(hp + i + half);
      const float4 c = *reinterpret_cast<const float4*>(cr + i), sn = *reinterpret_cast<const float4*>(sr + i);
      float y0[4], y1[4];
      rotate_pair(a.x, b.x, c.x, sn.x, y0[0], y1[0]);
      rotate_pair(a.y, b.y, c.y, sn.y, y0[1], y1[1]);
      rotate_pair(a.z, b.z, c.z, sn.z, y0[2], y1[2]);
      rotate_pair(a.w, b.w, c.w, sn.w, y0[3], y1[3]);
      y = first ? make_float4(y0[0], y0[1], y0[2], y0[3]) : make_float4(y1[0], y1[1], y1[2], y1[3]);
    } else if (d < dim) {
      y = *reinterpret_cast<const float4*>(hp + d);
    }
    TC* dst = h < n_heads ? q_out + ((size_t)t * n_heads + h) * pad
                          : k_pages + page_base + (size_t)(h - n_heads) * RB_PAGE * pad;
    store4(dst + d, y.x, y.y, y.z, y.w);
  }
  if (v_pages) {
    const float* vsrc = src + (size_t)(n_heads + n_kv) * dim;
    for (int idx = threadIdx.x; idx < n_kv * quads; idx += blockDim.x) {
      const int h = idx / quads, d = 4 * (idx - h * quads);
      const float4 v = d < vdim ? *reinterpret_cast<const float4*>(vsrc + (size_t)h * vdim + d) : make_float4(0.f, 0.f, 0.f, 0.f);
      store4(v_pages + page_base + (size_t)h * RB_PAGE * pad + d, v.x, v.y, v.z, v.w);
    }
  }
}

extern "C" int rb_rope_store(const float* qkv, long long row_width, const float* cos, const float* sin, int rot, void* q_out,
                             void* k_pages, void* v_pages, int cache_dtype, const int32_t* tok_pos, const int32_t* tok_seq,
                             const int32_t* block_table, int bt_stride, int n_tokens, int n_heads, int n_kv_heads, int dim,
                             int vdim, int pad, void* stream) {
  RB_RECORDED(rb_rope_store(qkv, row_width, cos, sin, rot, q_out, k_pages, v_pages, cache_dtype, tok_pos, tok_seq, block_table,
                            bt_stride, n_tokens, n_heads, n_kv_heads, dim, vdim, pad, stream));
  RB_REQUIRE(n_tokens >= 0 && n_heads > 0 && n_kv_heads >= 0 && dim > 0 && vdim > 0 && pad >= dim && pad >= vdim,
             "rb_rope_store: bad sizes T=%d Hq=%d Hk=%d dim=%d vdim=%d pad=%d", n_tokens, n_heads, n_kv_heads, dim, vdim, pad);
  RB_REQUIRE(rot >= 0 && rot % 2 == 0 && rot <= dim, "rb_rope_store: %d rotated numbers in a head of %d", rot, dim);
  RB_REQUIRE(rot == 0 || (cos != nullptr && sin != nullptr), "rb_rope_store: a rotation needs its tables");
  RB_REQUIRE((k_pages == nullptr) == (v_pages == nullptr), "rb_rope_store: k and v pages go together");
  const long long need = (long long)n_heads * dim + (k_pages ? (long long)n_kv_heads * (dim + vdim) : 0);
  RB_REQUIRE(row_width >= need, "rb_rope_store: rows of %lld numbers, %lld needed", row_width, need);
  if (n_tokens == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  auto aligned = [](const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; };
  const bool vec = dim % 4 == 0 && vdim % 4 == 0 && pad % 4 == 0 && rot % 8 == 0 && row_width % 4 == 0 && aligned(qkv) &&
                   aligned(cos) && aligned(sin) && aligned(q_out) && aligned(k_pages) && aligned(v_pages);
  if (vec && cache_dtype == RB_F32)
    rope_store_vec_kernel<float><<<n_tokens, 256, 0, s>>>(qkv, (size_t)row_width, cos, sin, rot, (float*)q_out, (float*)k_pages,
                                                          (float*)v_pages, tok_pos, tok_seq, block_table, bt_stride, n_heads,
                                                          n_kv_heads, dim, vdim, pad);
  else if (vec && cache_dtype == RB_BF16)
    rope_store_vec_kernel<bf16_t><<<n_tokens, 256, 0, s>>>(qkv, (size_t)row_width, cos, sin, rot, (bf16_t*)q_out, (bf16_t*)k_pages,
                                                           (bf16_t*)v_pages, tok_pos, tok_seq, block_table, bt_stride, n_heads,
                                                           n_kv_heads, dim, vdim, pad);
  else if (cache_dtype == RB_F32)
    rope_store_kernel<float><<<n_tokens, 256, 0, s>>>(qkv, (size_t)row_width, cos, sin, rot, (float*)q_out, (float*)k_pages,
                                                      (float*)v_pages, tok_pos, tok_seq, block_table, bt_stride, n_heads,
                                                      n_kv_heads, dim, vdim, pad);
  else if (cache_dtype == RB_BF16)
    rope_store_kernel<bf16_t><<<n_tokens, 256, 0, s>>>(qkv, (size_t)row_width, cos, sin, rot, (bf16_t*)q_out, (bf16_t*)k_pages,
                                                       (bf16_t*)v_pages, tok_pos, tok_seq, block_table, bt_stride, n_heads,
                                                       n_kv_heads, dim, vdim, pad);
  else
    RB_REQUIRE(false, "rb_rope_store: unknown dtype %d", cache_dtype);
  RB_LAUNCH_CHECK();
  return 0;
}

// ---------------------------------------------------------------- a gate per head
// x[t, h, :] *= sigmoid(gate[t * gate_stride + h]), in place; x [T, H, D] of dtype.
template <typename TC>
__global__ void head_gate_kernel(TC* __restrict__ x, const float* __restrict__ gate, size_t gate_stride, int n_heads, int d,
                                 size_t n) {
  for (size_t e = (size_t)blockIdx.x * blockDim.x + threadIdx.x; e < n; e += (size_t)gridDim.x * blockDim.x) {
    const size_t th = e / d;
    const size_t t = th / n_heads;
    const int h = (int)(th - t * n_heads);
    const float g = 1.0f / (1.0f + expf(-gate[t * gate_stride + h]));
    Num<TC>::store(x + e, Num<TC>::load(x + e) * g);
  }
}

// The same with 16 bytes a lane, for head sizes that are multiples of 8: a group of values lies within one head.
template <typename TC>
__global__ void head_gate_vec_kernel(TC* __restrict__ x, const float* __restrict__ gate, size_t gate_stride, int n_heads, int d,
                                     size_t n_groups) {
  constexpr int E = 16 / sizeof(TC);
  for (size_t gi = (size_t)blockIdx.x * blockDim.x + threadIdx.x; gi < n_groups; gi += (size_t)gridDim.x * blockDim.x) {
    const size_t e = gi * E;
    const size_t th = e / d;
    const size_t t = th / n_heads;
    const int h = (int)(th - t * n_heads);
    const float g = 1.0f / (1.0f + expf(-gate[t * gate_stride + h]));
    uint4 raw = *reinterpret_cast<const uint4*>(x + e);
    if (sizeof(TC) == 4) {
      float4 v = *reinterpret_cast<float4*>(&raw);
      v = make_float4(v.x * g, v.y * g, v.z * g, v.w * g);
      *reinterpret_cast<float4*>(x + e) = v;
    } else {
      raw = make_uint4(pack_bf16x2(bf16_bits_to_f32(raw.x & 0xffffu) * g, bf16_bits_to_f32(raw.x >> 16) * g),
                       pack_bf16x2(bf16_bits_to_f32(raw.y & 0xffffu) * g, bf16_bits_to_f32(raw.y >> 16) * g),
                       pack_bf16x2(bf16_bits_to_f32(raw.z & 0xffffu) * g, bf16_bits_to_f32(raw.z >> 16) * g),
                       pack_bf16x2(bf16_bits_to_f32(raw.w & 0xffffu) * g, bf16_bits_to_f32(raw.w >> 16) * g));
      *reinterpret_cast<uint4*>(x + e) = raw;
    }
  }
}

extern "C" int rb_head_gate(void* x, int dtype, const float* gate, long long gate_stride, int n_tokens, int n_heads, int head_dim,
                            void* stream) {
  RB_RECORDED(rb_head_gate(x, dtype, gate, gate_stride, n_tokens, n_heads, head_dim, stream));
  RB_REQUIRE(n_tokens >= 0 && n_heads > 0 && head_dim > 0 && gate_stride >= n_heads, "rb_head_gate: bad sizes");
  if (n_tokens == 0) return 0;
  const size_t n = (size_t)n_tokens * n_heads * head_dim;
  hipStream_t s = (hipStream_t)stream;
  if (head_dim % 8 == 0 && (reinterpret_cast<uintptr_t>(x) & 15) == 0 && (dtype == RB_F32 || dtype == RB_BF16)) {
    const size_t groups = n / (dtype == RB_F32 ? 4 : 8);
    const size_t vb = (groups + 255) / 256;
    const int vgrid = (int)(vb < 65535 ? vb : 65535);
    if (dtype == RB_F32)
      head_gate_vec_kernel<float><<<vgrid, 256, 0, s>>>((float*)x, gate, (size_t)gate_stride, n_heads, head_dim, groups);
    else
      head_gate_vec_kernel<bf16_t><<<vgrid, 256, 0, s>>>((bf16_t*)x, gate, (size_t)gate_stride, n_heads, head_dim, groups);
    RB_LAUNCH_CHECK();
    return 0;
  }
  const size_t blocks = (n + 255) / 256;
  const int grid = (int)(blocks < 65535 ? blocks : 65535);
  if (dtype == RB_F32)
    head_gate_kernel<float><<<grid, 256, 0, s>>>((float*)x, gate, (size_t)gate_stride, n_heads, head_dim, n);
  else if (dtype == RB_BF16)
    head_gate_kernel<bf16_t><<<grid, 256, 0, s>>>((bf16_t*)x, gate, (size_t)gate_stride, n_heads, head_dim, n);
  else
    RB_REQUIRE(false, "rb_head_gate: unknown dtype %d", dtype);
  RB_LAUNCH_CHECK();
  return 0;
}

// ---------------------------------------------------------------- the mean of two normed outputs
// out[t, :] = (a / sqrt(mean a^2 + eps) * wa + b / sqrt(mean b^2 + eps) * wb) / 2; one workgroup a row.
__global__ void pair_norm_mean_kernel(const float* __restrict__ a, const float* __restrict__ wa, const float* __restrict__ b,
                                      const float* __restrict__ wb, float eps, float* __restrict__ out, int width) {
  __shared__ float scratch[16];
  const size_t r = blockIdx.x;
  const float* ar = a + r * width;
  const float* br = b + r * width;
  float sa = 0.f, sb = 0.f;
  for (int j = threadIdx.x; j < width; j += blockDim.x) {
    sa = fmaf(ar[j], ar[j], sa);
    sb = fmaf(br[j], br[j], sb);
  }
  const float fa = 1.0f / sqrtf(block_sum(sa, scratch) / (float)width + eps);
  const float fb = 1.0f / sqrtf(block_sum(sb, scratch) / (float)width + eps);
  for (int j = threadIdx.x; j < width; j += blockDim.x)
    out[r * width + j] = 0.5f * (ar[j] * fa * wa[j] + br[j] * fb * wb[j]);
}

// The same with 16-byte accesses for widths that are multiples of 4, the rows kept in registers between the two passes
// when 1024 threads hold them (widths up to 4096), else read again.
__global__ __launch_bounds__(1024) void pair_norm_mean_vec_kernel(const float* __restrict__ a, const float* __restrict__ wa,
                                                                  const float* __restrict__ b, const float* __restrict__ wb, float eps,
                                                                  float* __restrict__ out, int width) {
  __shared__ float scratch[16];
  const size_t r = blockIdx.x;
  const float* ar = a + r * width;
  const float* br = b + r * width;
  const int j0 = 4 * threadIdx.x;
  float4 va = make_float4(0.f, 0.f, 0.f, 0.f), vb = va;
  float sa = 0.f, sb = 0.f;
  for (int j = j0; j < width; j += 4 * blockDim.x) {
    const float4 x = *reinterpret_cast<const float4*>(ar + j), y = *reinterpret_cast<const float4*>(br + j);
    if (j == j0) {
      va = x;
      vb = y;
    }
    sa += (x.x * x.x + x.y * x.y) + (x.z * x.z + x.w * x.w);
    sb += (y.x * y.x + y.y * y.y) + (y.z * y.z + y.w * y.w);
  }
  const float fa = 1.0f / sqrtf(block_sum(sa, scratch) / (float)width + eps);
  const float fb = 1.0f / sqrtf(block_sum(sb, scratch) / (float)width + eps);
  for (int j = j0; j < width; j += 4 * blockDim.x) {
    const float4 x = j == j0 ? va : *reinterpret_cast<const float4*>(ar + j);
    const float4 y = j == j0 ? vb : *reinterpret_cast<const float4*>(br + j);
    const float4 p = *reinterpret_cast<const float4*>(wa + j), q = *reinterpret_cast<const float4*>(wb + j);
    *reinterpret_cast<float4*>(out + r * width + j) =
        make_float4(0.5f * (x.x * fa * p.x + y.x * fb * q.x), 0.5f * (x.y * fa * p.y + y.y * fb * q.y),
                    0.5f * (x.z * fa * p.z + y.z * fb * q.z), 0.5f * (x.w * fa * p.w + y.w * fb * q.w));
  }
}

extern "C" int rb_pair_norm_mean(const float* a, const float* wa, const float* b, const float* wb, float eps, float* out,
                                 int n_tokens, int width, void* stream) {
  RB_RECORDED(rb_pair_norm_mean(a, wa, b, wb, eps, out, n_tokens, width, stream));
  RB_REQUIRE(n_tokens >= 0 && width > 0, "rb_pair_norm_mean: bad sizes %d x %d", n_tokens, width);
  if (n_tokens == 0) return 0;
  auto aligned = [](const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; };
  if (width % 4 == 0 && aligned(a) && aligned(b) && aligned(wa) && aligned(wb) && aligned(out)) {
    int threads = ((width / 4 + RB_WAVE - 1) / RB_WAVE) * RB_WAVE;
    if (threads > 1024) threads = 1024;
    pair_norm_mean_vec_kernel<<<n_tokens, threads, 0, (hipStream_t)stream>>>(a, wa, b, wb, eps, out, width);
    RB_LAUNCH_CHECK();
    return 0;
  }
  const int threads = width >= 1024 ? 1024 : (width >= 256 ? 256 : 64);
  pair_norm_mean_kernel<<<n_tokens, threads, 0, (hipStream_t)stream>>>(a, wa, b, wb, eps, out, width);
  RB_LAUNCH_CHECK();
  return 0;
}

// ---------------------------------------------------------------- a norm per head in front of the rotation
// rb_rope_store with every query and key head first RMS-normed over its `dim` numbers with a weight of that size shared by
// the heads (q_norm, k_norm; plain weights): x / sqrt(mean(x^2) + eps) * w, in float32, then the rotation of the head's
// first `rot` numbers, the padding and the cache write as there.  A wave takes a head.
#define NRS_MAX_DIM 512
#define NRS_MAX_WAVES 16
template <typename TC>
__global__ void norm_rope_store_kernel(const float* __restrict__ qkv, size_t row_width, const float* __restrict__ cos_t,
                                       const float* __restrict__ sin_t, int rot, const float* __restrict__ q_norm,
                                       const float* __restrict__ k_norm, float eps, TC* __restrict__ q_out,
                                       TC* __restrict__ k_pages, TC* __restrict__ v_pages, const int32_t* __restrict__ tok_pos,
                                       const int32_t* __restrict__ tok_seq, const int32_t* __restrict__ block_table,
                                       int bt_stride, int n_heads, int n_kv, int dim, int vdim, int pad) {
  // a wave reads its head once (whole lines), leaves the normed head in an LDS row of its own and rotates from there
  __shared__ float stage[NRS_MAX_WAVES][NRS_MAX_DIM];
  const int t = blockIdx.x;
  const int pos = tok_pos[t];
  const int half = rot / 2;
  const int lane = threadIdx.x & (RB_WAVE - 1), wave = threadIdx.x / RB_WAVE, n_waves = blockDim.x / RB_WAVE;
  const float* src = qkv + (size_t)t * row_width;
  const float* cr = cos_t + (size_t)pos * half;
  const float* sr = sin_t + (size_t)pos * half;
  float* mine = stage[wave];
  size_t page_base = 0;
  if (k_pages) {
    const int page = block_table[(size_t)tok_seq[t] * bt_stride + pos / RB_PAGE];
    page_base = ((size_t)page * n_kv) * RB_PAGE * pad + (size_t)(pos % RB_PAGE) * pad;
  }
  const int n_rot_heads = n_heads + (k_pages ? n_kv : 0);
  for (int h = wave; h < n_rot_heads; h += n_waves) {
    const float* hp = src + (size_t)h * dim;
    const float* w = h < n_heads ? q_norm : k_norm;
    float xv[NRS_MAX_DIM / RB_WAVE];
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < NRS_MAX_DIM / RB_WAVE; ++i) {
      const int d = lane + RB_WAVE * i;
      xv[i] = d < dim ? hp[d] : 0.f;
      ss = fmaf(xv[i], xv[i], ss);
    }
    const float f = 1.0f / sqrtf(wave_sum(ss) / (float)dim + eps);
#pragma unroll
    for (int i = 0; i < NRS_MAX_DIM / RB_WAVE; ++i) {
      const int d = lane + RB_WAVE * i;
      if (d < dim) mine[d] = xv[i] * f * w[d];
    }
    __builtin_amdgcn_wave_barrier();          // the row is this wave's alone; a wave's LDS accesses complete in order
    TC* dst = h < n_heads ? q_out + ((size_t)t * n_heads + h) * pad
                          : k_pages + page_base + (size_t)(h - n_heads) * RB_PAGE * pad;
    for (int d = lane; d < pad; d += RB_WAVE) {
      float y = 0.f;
      if (d < half) {
        float y1;
        rotate_pair(mine[d], mine[d + half], cr[d], sr[d], y, y1);
      } else if (d < rot) {
        float y0;
        rotate_pair(mine[d - half], mine[d], cr[d - half], sr[d - half], y0, y);
      } else if (d < dim) {
        y = mine[d];
      }
      Num<TC>::store(dst + d, y);
    }
    __builtin_amdgcn_wave_barrier();
  }
  if (v_pages) {
    const float* vsrc = src + (size_t)(n_heads + n_kv) * dim;
    for (int idx = threadIdx.x; idx < n_kv * pad; idx += blockDim.x) {
      const int h = idx / pad, d = idx - h * pad;
      Num<TC>::store(v_pages + page_base + (size_t)h * RB_PAGE * pad + d, d < vdim ? vsrc[(size_t)h * vdim + d] : 0.f);
    }
  }
}

extern "C" int rb_norm_rope_store(const float* qkv, long long row_width, const float* cos, const float* sin, int rot,
                                  const float* q_norm, const float* k_norm, float eps, void* q_out, void* k_pages, void* v_pages,
                                  int cache_dtype, const int32_t* tok_pos, const int32_t* tok_seq, const int32_t* block_table,
                                  int bt_stride, int n_tokens, int n_heads, int n_kv_heads, int dim, int vdim, int pad,
                                  void* stream) {
  RB_RECORDED(rb_norm_rope_store(qkv, row_width, cos, sin, rot, q_norm, k_norm, eps, q_out, k_pages, v_pages, cache_dtype, tok_pos,
                                 tok_seq, block_table, bt_stride, n_tokens, n_heads, n_kv_heads, dim, vdim, pad, stream));
  RB_REQUIRE(n_tokens >= 0 && n_heads > 0 && n_kv_heads >= 0 && dim > 0 && vdim > 0 && pad >= dim && pad >= vdim,
             "rb_norm_rope_store: bad sizes T=%d Hq=%d Hk=%d dim=%d vdim=%d pad=%d", n_tokens, n_heads, n_kv_heads, dim, vdim, pad);
  RB_REQUIRE(rot >= 0 && rot % 2 == 0 && rot <= dim, "rb_norm_rope_store: %d rotated numbers in a head of %d", rot, dim);
  RB_REQUIRE(dim <= NRS_MAX_DIM, "rb_norm_rope_store: head size %d not supported (at most %d)", dim, NRS_MAX_DIM);
  RB_REQUIRE(rot == 0 || (cos != nullptr && sin != nullptr), "rb_norm_rope_store: a rotation needs its tables");
  RB_REQUIRE(q_norm != nullptr && (k_pages == nullptr || k_norm != nullptr), "rb_norm_rope_store: the norms' weights are needed");
  RB_REQUIRE((k_pages == nullptr) == (v_pages == nullptr), "rb_norm_rope_store: k and v pages go together");
  const long long need = (long long)n_heads * dim + (k_pages ? (long long)n_kv_heads * (dim + vdim) : 0);
  RB_REQUIRE(row_width >= need, "rb_norm_rope_store: rows of %lld numbers, %lld needed", row_width, need);
  if (n_tokens == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  // a wave a head, up to 16 waves a token: a wave's heads are a chain of trips to memory
  int waves = n_heads + (k_pages ? n_kv_heads : 0);
  const int most = n_tokens < 2 * rb_compute_units() ? NRS_MAX_WAVES : 8;
  waves = waves > most ? most : (waves < 4 ? 4 : waves);
  const int threads = RB_WAVE * waves;
  if (cache_dtype == RB_F32)
    norm_rope_store_kernel<float><<<n_tokens, threads, 0, s>>>(qkv, (size_t)row_width, cos, sin, rot, q_norm, k_norm, eps, (float*)q_out,
                                                           (float*)k_pages, (float*)v_pages, tok_pos, tok_seq, block_table,
                                                           bt_stride, n_heads, n_kv_heads, dim, vdim, pad);
  else if (cache_dtype == RB_BF16)
    norm_rope_store_kernel<bf16_t><<<n_tokens, threads, 0, s>>>(qkv, (size_t)row_width, cos, sin, rot, q_norm, k_norm, eps,
                                                            (bf16_t*)q_out, (bf16_t*)k_pages, (bf16_t*)v_pages, tok_pos, tok_seq,
                                                            block_table, bt_stride, n_heads, n_kv_heads, dim, vdim, pad);
  else
    RB_REQUIRE(false, "rb_norm_rope_store: unknown dtype %d", cache_dtype);
  RB_LAUNCH_CHECK();
  return 0;
}

// ---------------------------------------------------------------- a gate on every number
// x[e] *= sigmoid(gate[e]), in place; x of dtype and gate float32 laid out alike, n numbers.
template <typename TC>
__global__ void sigmoid_gate_kernel(TC* __restrict__ x, const float* __restrict__ gate, size_t n) {
  for (size_t e = (size_t)blockIdx.x * blockDim.x + threadIdx.x; e < n; e += (size_t)gridDim.x * blockDim.x)
    Num<TC>::store(x + e, Num<TC>::load(x + e) / (1.0f + expf(-gate[e])));
}

extern "C" int rb_sigmoid_gate(void* x, int dtype, const float* gate, long long n, void* stream) {
  RB_RECORDED(rb_sigmoid_gate(x, dtype, gate, n, stream));
  RB_REQUIRE(n >= 0, "rb_sigmoid_gate: bad size");
  if (n == 0) return 0;
  const size_t blocks = ((size_t)n + 255) / 256;
  const int grid = (int)(blocks < 65535 ? blocks : 65535);
  hipStream_t s = (hipStream_t)stream;
  if (dtype == RB_F32)
    sigmoid_gate_kernel<float><<<grid, 256, 0, s>>>((float*)x, gate, (size_t)n);
  else if (dtype == RB_BF16)
    sigmoid_gate_kernel<bf16_t><<<grid, 256, 0, s>>>((bf16_t*)x, gate, (size_t)n);
  else
    RB_REQUIRE(false, "rb_sigmoid_gate: unknown dtype %d", dtype);
  RB_LAUNCH_CHECK();
  return 0;
}

// ---------------------------------------------------------------- the token before, mixed in
// out[m, t, :] = h[t] + (h[t - 1] - h[t]) * mu[m], m < n_mix, where the row before a step's first comes from the sequence's
// state [slots, E] (float32; zeros for a fresh slot) and the state then holds the step's last row.  float32 arithmetic; h and
// out of dtype.  A workgroup a token; the one that takes a sequence's first row of the step is also the one that writes
// the state, after it has read it.
template <typename TC>
__global__ void shift_mix_kernel(const TC* __restrict__ h, float* __restrict__ state, const float* __restrict__ mu, int n_mix,
                                 TC* __restrict__ out, const int32_t* __restrict__ cu_seqlens, const int32_t* __restrict__ tok_seq,
                                 const int32_t* __restrict__ slots, int n_tokens, int width) {
  const int t = blockIdx.x;
  const int b = tok_seq[t];
  const int row0 = cu_seqlens[b], last = cu_seqlens[b + 1] - 1;
  const bool first = t == row0;
  float* st = state + (size_t)slots[b] * width;
  for (int j = threadIdx.x; j < width; j += blockDim.x) {
    const float cur = Num<TC>::load(h + (size_t)t * width + j);
    const float before = first ? st[j] : Num<TC>::load(h + (size_t)(t - 1) * width + j);
    const float d = before - cur;
    for (int m = 0; m < n_mix; ++m)
      Num<TC>::store(out + ((size_t)m * n_tokens + t) * width + j, fmaf(d, mu[(size_t)m * width + j], cur));
    if (first) st[j] = last == t ? cur : Num<TC>::load(h + (size_t)last * width + j);
  }
}

extern "C" int rb_shift_mix(const void* h, int dtype, float* state, const float* mu, int n_mix, void* out,
                            const int32_t* cu_seqlens, const int32_t* tok_seq, const int32_t* slots, int n_tokens, int n_seqs,
                            int width, void* stream) {
  RB_RECORDED(rb_shift_mix(h, dtype, state, mu, n_mix, out, cu_seqlens, tok_seq, slots, n_tokens, n_seqs, width, stream));
  RB_REQUIRE(n_tokens >= 0 && n_seqs >= 0 && width > 0 && n_mix > 0, "rb_shift_mix: bad sizes");
  RB_REQUIRE(h && state && mu && out, "rb_shift_mix: a pointer is missing");
  if (n_tokens == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  const int threads = width >= 1024 ? 1024 : 256;
  if (dtype == RB_F32)
    shift_mix_kernel<float><<<n_tokens, threads, 0, s>>>((const float*)h, state, mu, n_mix, (float*)out, cu_seqlens, tok_seq, slots,
                                                        n_tokens, width);
  else if (dtype == RB_BF16)
    shift_mix_kernel<bf16_t><<<n_tokens, threads, 0, s>>>((const bf16_t*)h, state, mu, n_mix, (bf16_t*)out, cu_seqlens, tok_seq,
                                                         slots, n_tokens, width);
  else
    RB_REQUIRE(false, "rb_shift_mix: unknown dtype %d", dtype);
  RB_LAUNCH_CHECK();
  return 0;
}
