// Attention whose heads' scores are mixed before the softmax, on the matrix cores: bfloat16, heads of 64 or 128
// numbers, at most 32 query heads.  The same kernel takes a prompt's tokens and single tokens.
//
// A workgroup of 4 waves takes 16 consecutive queries of one sequence and ALL heads, since every head's weights need
// every head's scores.  The keys go by in tiles of 64 (a page).  Per tile:
//   1. scores      S[g, i, j] = q_gi . k_j * scale for every head g: bfloat16 MFMA 16x16x32, operands straight from memory
//                  (a query's and a key's 8 numbers are 16 bytes in a row); a wave takes a quarter of the heads, keeps
//                  their queries in registers for all tiles where they fit, and asks for a kv head's 64 keys at once;
//                  float32 into LDS, zero where j is not seen
//   2. mixing      S[h, i, j] <- sum_g talk[h, g] S[g, i, j]: float32 MFMA 16x16x4 (float32 inputs and sums), talk in
//                  registers, 16 (i, j) columns at a time, in place
//   3. softmax     online, per (h, i) row in float32; the weights leave as TWO bfloat16 numbers (p = hi + lo, which holds
//                  16 bits of p), written over the row's scores
//   4. values      per kv head: V^T of the tile through LDS, O_h += P_hi V + P_lo V (bfloat16 MFMA, float32 sums); a wave
//                  owns 16 (or 32) of a head's output numbers for all heads; the next kv head's (or tile's) values are on
//                  their way from memory while the products of this one run
// What a row has seen so far (maximum, sum) lives in registers of the wave that does the row's softmax.
#include <math.h>

#include "api.h"
#include "mfma.h"

#define TM_Q 16                           // queries a workgroup
#define TM_ROW 68                         // floats a (head, query) row of scores: 64 keys + 4, so rows start at 16 bytes
#define TM_HEAD (TM_Q * TM_ROW + 20)      // floats a head: 20 banks on, so that 4 heads' reads and writes spread
#define TM_VLD 72                         // bfloat16 a row of V^T: 64 keys + 8
#define TM_THREADS 256
#define TM_MAX_HEADS 32

__device__ __forceinline__ int tm_first_key(int pos, int chunk, int window) {
  int lo = 0;
  if (chunk > 0) lo = pos / chunk * chunk;
  if (window > 0 && pos - window + 1 > lo) lo = pos - window + 1;
  return lo;
}

// D: head size; HB: heads rounded up to 8, 16 or 32
template <int D, int HB>
__global__ __launch_bounds__(TM_THREADS) void attention_mixed_mfma_kernel(
    const bf16_t* __restrict__ q, const bf16_t* __restrict__ k_pages, const bf16_t* __restrict__ v_pages, bf16_t* __restrict__ out,
    const int32_t* __restrict__ cu_seqlens, const int32_t* __restrict__ past_len, const int32_t* __restrict__ block_table,
    int bt_stride, int n_seqs, int n_heads, int n_kv, float scale, const float* __restrict__ talk, int chunk, int window) {
  constexpr int RB = (HB + 15) / 16;      // blocks of 16 mixed heads
  constexpr int DS = HB / 4;              // depth steps of the mixing: 4 heads each
  constexpr int HW = HB / 4;              // heads whose softmax a wave does
  constexpr int DB = D / 64;              // blocks of 16 output numbers a wave owns
  extern __shared__ __attribute__((aligned(16))) float tm_lds[];
  float* S = tm_lds;                                          // [H][TM_HEAD]
  float* alpha = S + (size_t)n_heads * TM_HEAD;               // [H][16]: what a row's sums so far are multiplied by
  bf16_t* vt = reinterpret_cast<bf16_t*>(alpha + n_heads * TM_Q);      // [D][TM_VLD]

  // ---- which sequence, which 16 queries
  int wg = blockIdx.x, b = 0, q0 = -1, seq_start = 0, q_len = 0;
  for (b = 0; b < n_seqs; ++b) {
    seq_start = cu_seqlens[b];
    q_len = cu_seqlens[b + 1] - seq_start;
    const int tiles = (q_len + TM_Q - 1) / TM_Q;
    if (wg < tiles) {
      q0 = wg * TM_Q;
      break;
    }
    wg -= tiles;
  }
  if (q0 < 0) return;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int l16 = lane & 15, lg = lane >> 4;
  const int group = n_heads / n_kv;
  const int past = past_len[b];
  const int n_valid = q_len - q0 < TM_Q ? q_len - q0 : TM_Q;
  const int pos_first = past + q0, pos_last = past + q0 + n_valid - 1;
  const int kv_last = past + q_len - 1;                       // the last key the sequence holds
  const int32_t* bt = block_table + (size_t)b * bt_stride;
  const int first_tile = tm_first_key(pos_first, chunk, window) / RB_PAGE, last_tile = pos_last / RB_PAGE;

  // rows of an MFMA result that this lane holds: queries 4 * lg + r
  int lo_r[4];
#pragma unroll
  for (int r = 0; r < 4; ++r) lo_r[r] = tm_first_key(pos_first + 4 * lg + r, chunk, window);
  // the row whose softmax this lane shares in: query lane / 4, keys 16 * (lane % 4) ...
  const int si = lane >> 2, sq = lane & 3;
  const int s_pos = pos_first + si, s_lo = tm_first_key(s_pos, chunk, window);

  // ---- the mixing matrix as A operands: row h = 16 rb + l16, depth g = 4 s + lg
  float ta[RB][DS];
#pragma unroll
  for (int rb = 0; rb < RB; ++rb)
#pragma unroll
    for (int s = 0; s < DS; ++s) {
      const int h = 16 * rb + l16, g = 4 * s + lg;
      ta[rb][s] = (h < n_heads && g < n_heads) ? talk[h * n_heads + g] : 0.f;
    }

  float m_run[HW], l_run[HW];
#pragma unroll
  for (int k = 0; k < HW; ++k) {
    m_run[k] = -INFINITY;
    l_run[k] = 0.f;
  }
  f32x4_t oacc[HB][DB];
#pragma unroll
  for (int h = 0; h < HB; ++h)
#pragma unroll
    for (int d = 0; d < DB; ++d) oacc[h][d] = f32x4_t{0.f, 0.f, 0.f, 0.f};

  // ---- the heads whose scores this wave computes, and their queries (rows past the sequence's end read its last row)
  constexpr bool QR = HW * (D / 32) <= 16;      // the queries stay in registers
  const int hpw = (n_heads + 3) / 4;
  const int h_lo = wave * hpw, h_hi = h_lo + hpw < n_heads ? h_lo + hpw : n_heads;
  const size_t q_row = ((size_t)(seq_start + q0 + (l16 < n_valid ? l16 : n_valid - 1)) * n_heads) * D + lg * 8;
  Frag8 qres[QR ? HW * (D / 32) : 1];
  if (QR) {
#pragma unroll
    for (int k = 0; k < HW; ++k)
#pragma unroll
      for (int s = 0; s < D / 32; ++s)
        qres[k * (D / 32) + s].u = h_lo + k < h_hi ? load16(q + q_row + (size_t)(h_lo + k) * D + s * 32) : zero16();
  }

  // ---- V^T of a tile and kv head: a thread takes 4 keys in a row and 8 numbers of each, and writes 8 times 4 keys
  const int v_kq = tid & 15, v_dc = tid >> 4;
  const bool v_on = tid < 16 * (D / 8);
  uint4 vreg[4];
  auto load_v = [&](int kt, int g) {
    if (!v_on) return;
    const bf16_t* src = v_pages + ((size_t)bt[kt] * n_kv + g) * RB_PAGE * D + (size_t)(4 * v_kq) * D + v_dc * 8;
#pragma unroll
    for (int e = 0; e < 4; ++e)      // what lies beyond the sequence may be anything, even NaN: zeros
      vreg[e] = kt * RB_PAGE + 4 * v_kq + e <= kv_last ? load16(src + (size_t)e * D) : zero16();
  };
  auto store_v = [&]() {
    if (!v_on) return;
    const uint32_t w[4][4] = {{vreg[0].x, vreg[1].x, vreg[2].x, vreg[3].x}, {vreg[0].y, vreg[1].y, vreg[2].y, vreg[3].y},
                              {vreg[0].z, vreg[1].z, vreg[2].z, vreg[3].z}, {vreg[0].w, vreg[1].w, vreg[2].w, vreg[3].w}};
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      uint2 even, odd;
      even.x = (w[c][0] & 0xffffu) | (w[c][1] << 16);
      even.y = (w[c][2] & 0xffffu) | (w[c][3] << 16);
      odd.x = (w[c][0] >> 16) | (w[c][1] & 0xffff0000u);
      odd.y = (w[c][2] >> 16) | (w[c][3] & 0xffff0000u);
      *reinterpret_cast<uint2*>(vt + (v_dc * 8 + 2 * c) * TM_VLD + 4 * v_kq) = even;
      *reinterpret_cast<uint2*>(vt + (v_dc * 8 + 2 * c + 1) * TM_VLD + 4 * v_kq) = odd;
    }
  };
  load_v(first_tile, 0);

  for (int kt = first_tile; kt <= last_tile; ++kt) {
    const size_t page_base = (size_t)bt[kt] * n_kv * RB_PAGE * D;
    const int key0 = kt * RB_PAGE;
    // ---------------------------------------------------------------- 1. scores
    {
      Frag8 kf[4][D / 32];
      int g_have = -1;
#pragma unroll
      for (int k = 0; k < HW; ++k) {
        const int h = h_lo + k;
        if (h < h_hi) {
          const int g = h / group;
          if (g != g_have) {           // the 64 keys of this kv head, asked for together
            const bf16_t* krow = k_pages + page_base + ((size_t)g * RB_PAGE + l16) * D + lg * 8;
#pragma unroll
            for (int kb = 0; kb < 4; ++kb)
#pragma unroll
              for (int s = 0; s < D / 32; ++s) kf[kb][s].u = load16(krow + (size_t)kb * 16 * D + s * 32);
            g_have = g;
          }
          Frag8 qf[D / 32];
#pragma unroll
          for (int s = 0; s < D / 32; ++s) {
            if (QR)
              qf[s] = qres[k * (D / 32) + s];
            else
              qf[s].u = load16(q + q_row + (size_t)h * D + s * 32);
          }
          float* dst = S + (size_t)h * TM_HEAD + l16;
#pragma unroll
          for (int kb = 0; kb < 4; ++kb) {
            f32x4_t acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int s = 0; s < D / 32; ++s) acc = mfma16(qf[s], kf[kb][s], acc);
            const int key = key0 + kb * 16 + l16;
#pragma unroll
            for (int r = 0; r < 4; ++r) {
              const int i = 4 * lg + r;
              const bool seen = i < n_valid && key <= pos_first + i && key >= lo_r[r];
              dst[i * TM_ROW + kb * 16] = seen ? acc[r] * scale : 0.f;       // a select: a key beyond the sequence may be anything
            }
          }
        }
      }
    }
    __syncthreads();
    // ---------------------------------------------------------------- 2. mixing over the heads
    if (talk) {
      for (int cb = wave; cb < TM_Q * 4; cb += 4) {
        const int i = cb >> 2, jb = cb & 3;
        if (i >= n_valid || key0 + jb * 16 > pos_first + i) continue;          // nothing seen in these 16 columns
        float* col = S + i * TM_ROW + jb * 16 + l16;
        float bv[DS];
#pragma unroll
        for (int s = 0; s < DS; ++s) {
          const int g = 4 * s + lg;
          bv[s] = col[(size_t)(g < n_heads ? g : n_heads - 1) * TM_HEAD];
        }
#pragma unroll
        for (int rb = 0; rb < RB; ++rb) {
          f32x4_t acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
          for (int s = 0; s < DS; ++s) acc = __builtin_amdgcn_mfma_f32_16x16x4f32(ta[rb][s], bv[s], acc, 0, 0, 0);
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            const int h = 16 * rb + 4 * lg + r;
            if (h < n_heads) col[(size_t)h * TM_HEAD] = acc[r];
          }
        }
      }
      __syncthreads();
    }
    // ---------------------------------------------------------------- 3. softmax, a wave a head, 4 lanes a row
#pragma unroll
    for (int k = 0; k < HW; ++k) {
      const int h = wave + 4 * k;
      if (h < n_heads) {
        float* row = S + (size_t)h * TM_HEAD + si * TM_ROW;
        float p[16];
#pragma unroll
        for (int v = 0; v < 4; ++v) {
          const float4 f = *reinterpret_cast<const float4*>(row + sq * 16 + 4 * v);
          p[4 * v + 0] = f.x;
          p[4 * v + 1] = f.y;
          p[4 * v + 2] = f.z;
          p[4 * v + 3] = f.w;
        }
        float mx = -INFINITY;
#pragma unroll
        for (int e = 0; e < 16; ++e) {
          const int key = key0 + sq * 16 + e;
          const bool seen = si < n_valid && key <= s_pos && key >= s_lo;
          p[e] = seen ? p[e] : -INFINITY;
          mx = fmaxf(mx, p[e]);
        }
        mx = fmaxf(mx, __shfl_xor(mx, 1, 64));
        mx = fmaxf(mx, __shfl_xor(mx, 2, 64));
        const float m_new = fmaxf(m_run[k], mx);
        const float m_safe = m_new == -INFINITY ? 0.f : m_new;
        float sum = 0.f;
#pragma unroll
        for (int e = 0; e < 16; ++e) {
          p[e] = p[e] == -INFINITY ? 0.f : expf(p[e] - m_safe);
          sum += p[e];
        }
        sum += __shfl_xor(sum, 1, 64);
        sum += __shfl_xor(sum, 2, 64);
        const float a = m_run[k] == -INFINITY ? 0.f : expf(m_run[k] - m_safe);
        l_run[k] = l_run[k] * a + sum;
        m_run[k] = m_new;
        if (sq == 0) alpha[h * TM_Q + si] = a;
        // the weights as hi + lo, over the row's scores: hi in the row's first 128 bytes, lo in the next
        uint32_t hi[8], lo[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const float a0 = p[2 * e], a1 = p[2 * e + 1];
          const uint32_t w = pack_bf16x2(a0, a1);
          hi[e] = w;
          lo[e] = pack_bf16x2(a0 - __uint_as_float(w << 16), a1 - __uint_as_float(w & 0xffff0000u));
        }
        uint4* ph = reinterpret_cast<uint4*>(reinterpret_cast<bf16_t*>(row) + sq * 16);
        uint4* pl = reinterpret_cast<uint4*>(reinterpret_cast<bf16_t*>(row) + 64 + sq * 16);
        ph[0] = make_uint4(hi[0], hi[1], hi[2], hi[3]);
        ph[1] = make_uint4(hi[4], hi[5], hi[6], hi[7]);
        pl[0] = make_uint4(lo[0], lo[1], lo[2], lo[3]);
        pl[1] = make_uint4(lo[4], lo[5], lo[6], lo[7]);
      }
    }
    __syncthreads();
    // ---------------------------------------------------------------- 4. values, one kv head after the other
    for (int g = 0; g < n_kv; ++g) {
      store_v();
      if (g + 1 < n_kv)
        load_v(kt, g + 1);
      else if (kt < last_tile)
        load_v(kt + 1, 0);
      __syncthreads();
#pragma unroll
      for (int h = 0; h < HB; ++h) {
        if (h < n_heads && h / group == g) {
          float a_r[4];
#pragma unroll
          for (int r = 0; r < 4; ++r) a_r[r] = alpha[h * TM_Q + 4 * lg + r];
#pragma unroll
          for (int d = 0; d < DB; ++d)
#pragma unroll
            for (int r = 0; r < 4; ++r) oacc[h][d][r] *= a_r[r];
          const bf16_t* prow = reinterpret_cast<const bf16_t*>(S + (size_t)h * TM_HEAD + l16 * TM_ROW) + lg * 8;
#pragma unroll
          for (int ks = 0; ks < 2; ++ks) {
            Frag8 p_hi, p_lo;
            p_hi.u = *reinterpret_cast<const uint4*>(prow + ks * 32);
            p_lo.u = *reinterpret_cast<const uint4*>(prow + 64 + ks * 32);
#pragma unroll
            for (int d = 0; d < DB; ++d) {
              Frag8 vf;
              vf.u = *reinterpret_cast<const uint4*>(vt + ((wave + 4 * d) * 16 + l16) * TM_VLD + ks * 32 + lg * 8);
              oacc[h][d] = mfma16(p_hi, vf, oacc[h][d]);
              oacc[h][d] = mfma16(p_lo, vf, oacc[h][d]);
            }
          }
        }
      }
      __syncthreads();
    }
  }

  // ---- the rows' sums to everyone, and out
#pragma unroll
  for (int k = 0; k < HW; ++k) {
    const int h = wave + 4 * k;
    if (h < n_heads && sq == 0) alpha[h * TM_Q + si] = l_run[k];
  }
  __syncthreads();
#pragma unroll
  for (int h = 0; h < HB; ++h) {
    if (h < n_heads) {
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int i = 4 * lg + r;
        if (i < n_valid) {
          const float l = alpha[h * TM_Q + i];
          const float inv = l > 0.f ? 1.0f / l : 0.f;
          bf16_t* dst = out + ((size_t)(seq_start + q0 + i) * n_heads + h) * D + l16;
#pragma unroll
          for (int d = 0; d < DB; ++d) Num<bf16_t>::store(dst + (wave + 4 * d) * 16, oacc[h][d][r] * inv);
        }
      }
    }
  }
}

template <int D, int HB>
static int launch_mixed_mfma(const void* q, const void* k_pages, const void* v_pages, void* out, const int32_t* cu_seqlens,
                             const int32_t* past_len, const int32_t* block_table, int bt_stride, int n_seqs, int n_tokens,
                             int n_heads, int n_kv, float scale, const float* talk, int chunk, int window, hipStream_t s) {
  const size_t lds = sizeof(float) * ((size_t)n_heads * TM_HEAD + (size_t)n_heads * TM_Q) + sizeof(bf16_t) * (size_t)D * TM_VLD;
  RB_REQUIRE(lds <= 160 * 1024, "rb_attention_mixed_bf16: %zu bytes of LDS are more than a workgroup has", lds);
  auto kernel = attention_mixed_mfma_kernel<D, HB>;
  if (lds > 64 * 1024) {
    static bool raised = false;          // per instantiation
    if (!raised) {
      RB_REQUIRE(hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024) == hipSuccess,
                 "rb_attention_mixed_bf16: cannot have %zu bytes of LDS", lds);
      raised = true;
    }
  }
  // an upper bound of the 16-query tiles that depends on the step's shape alone: workgroups past the last tile leave
  const int grid = n_tokens / TM_Q + n_seqs;
  kernel<<<grid, TM_THREADS, lds, s>>>((const bf16_t*)q, (const bf16_t*)k_pages, (const bf16_t*)v_pages, (bf16_t*)out, cu_seqlens,
                                       past_len, block_table, bt_stride, n_seqs, n_heads, n_kv, scale, talk, chunk, window);
  RB_LAUNCH_CHECK();
  return 0;
}

extern "C" int rb_attention_mixed_bf16(const void* q, const void* k_pages, const void* v_pages, void* out,
                                       const int32_t* cu_seqlens, const int32_t* past_len, const int32_t* block_table,
                                       int bt_stride, int n_seqs, int n_tokens, int n_heads, int n_kv_heads, int head_dim,
                                       float scale, const float* talk, int chunk, int window, void* stream) {
  RB_RECORDED(rb_attention_mixed_bf16(q, k_pages, v_pages, out, cu_seqlens, past_len, block_table, bt_stride, n_seqs, n_tokens,
                                      n_heads, n_kv_heads, head_dim, scale, talk, chunk, window, stream));
  RB_REQUIRE(n_seqs >= 0 && n_tokens >= 0 && n_heads > 0 && n_kv_heads > 0 && n_heads % n_kv_heads == 0 && chunk >= 0 && window >= 0,
             "rb_attention_mixed_bf16: bad sizes B=%d T=%d Hq=%d Hk=%d", n_seqs, n_tokens, n_heads, n_kv_heads);
  RB_REQUIRE(head_dim == 64 || head_dim == 128, "rb_attention_mixed_bf16: head_dim %d not supported (64 or 128; use rb_attention_mixed)",
             head_dim);
  RB_REQUIRE(n_heads <= TM_MAX_HEADS, "rb_attention_mixed_bf16: %d heads are more than a workgroup takes (%d; use rb_attention_mixed)",
             n_heads, TM_MAX_HEADS);
  RB_REQUIRE(talk != nullptr, "rb_attention_mixed_bf16: no mixing matrix (the identity, if the heads are not mixed)");
  if (n_seqs == 0 || n_tokens == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
#define TM_LAUNCH(D_, HB_)                                                                                                     \
  return launch_mixed_mfma<D_, HB_>(q, k_pages, v_pages, out, cu_seqlens, past_len, block_table, bt_stride, n_seqs, n_tokens, \
                                    n_heads, n_kv_heads, scale, talk, chunk, window, s)
  if (head_dim == 64) {
    if (n_heads <= 8) TM_LAUNCH(64, 8);
    if (n_heads <= 16) TM_LAUNCH(64, 16);
    TM_LAUNCH(64, 32);
  }
  if (n_heads <= 8) TM_LAUNCH(128, 8);
  if (n_heads <= 16) TM_LAUNCH(128, 16);
  TM_LAUNCH(128, 32);
#undef TM_LAUNCH
}
