// Attention whose heads' scores are mixed before the softmax, on the matrix cores: bfloat16, heads of 64 or 128
// numbers, at most 32 query heads.  The same kernel takes a prompt's tokens and single tokens.
//
// A workgroup of 8 waves takes 16 consecutive queries of one sequence and ALL heads, since every head's weights need
// every head's scores.  The keys go by in tiles of 64 (a page); a step of single tokens deals a sequence's tiles out to
// several workgroups, whose sums a second kernel puts together.  Every phase of a tile is a chain of LDS round trips, so
// the tile's time falls with the number of waves that share it, which is why there are so many.  Per tile:
//   1. scores      S[g, i, j] = q_gi . k_j * scale for every head g: bfloat16 MFMA 16x16x32, operands straight from memory
//                  (a query's and a key's 8 numbers are 16 bytes in a row); a wave takes its share of the heads, keeps
//                  their queries in registers for all tiles, and asks for a kv head's 64 keys at once;
//                  float32 into LDS, zero where j is not seen
//   2. mixing      S[h, i, j] <- sum_g talk[h, g] S[g, i, j]: float32 MFMA 16x16x4 (float32 inputs and sums), talk in
//                  registers, 16 (i, j) columns at a time, in place
//   3. softmax     online, per (h, i) row in float32; the weights leave as TWO bfloat16 numbers (p = hi + lo, which holds
//                  16 bits of p), written over the row's scores
//   4. values      per kv head: V^T of the tile through LDS, O_h += P_hi V + P_lo V (bfloat16 MFMA, float32 sums); a wave
//                  owns 16 of the output numbers of every head, or of some heads; the next kv head's (or tile's) values are on
//                  their way from memory while the products of this one run
// What a row has seen so far (maximum, sum) lives in registers of the wave that does the row's softmax.
#include <math.h>

#include "api.h"
#include "mfma.h"

#define TM_Q 16                           // queries a workgroup
#define TM_ROW 68                         // floats a (head, query) row of scores: 64 keys + 4, so rows start at 16 bytes
#define TM_HEAD (TM_Q * TM_ROW + 20)      // floats a head: 20 banks on, so that 4 heads' reads and writes spread
#define TM_VLD 72                         // bfloat16 a row of V^T: 64 keys + 8
#define TM_MAX_HEADS 32

__device__ __forceinline__ int tm_first_key(int pos, int chunk, int window) {
  int lo = 0;
  if (chunk > 0) lo = pos / chunk * chunk;
  if (window > 0 && pos - window + 1 > lo) lo = pos - window + 1;
  return lo;
}

// D: head size; HB: heads rounded up to 8, 16 or 32; NW: waves.  gridDim.y workgroups share a 16-query tile's key tiles;
// with more than one, each leaves its sums unnormalised in part_o [splits, T, H, D] and (maximum, sum) in part_ml
// [splits, T, H, 2].
template <int D, int HB, int NW>
__global__ __launch_bounds__(64 * NW) void attention_mixed_mfma_kernel(
    const bf16_t* __restrict__ q, const bf16_t* __restrict__ k_pages, const bf16_t* __restrict__ v_pages, bf16_t* __restrict__ out,
    const int32_t* __restrict__ cu_seqlens, const int32_t* __restrict__ past_len, const int32_t* __restrict__ block_table,
    int bt_stride, int n_seqs, int n_heads, int n_kv, float scale, const float* __restrict__ talk, int chunk, int window,
    float* __restrict__ part_o, float* __restrict__ part_ml, int n_tokens, int gv) {
  constexpr int RB = (HB + 15) / 16;                // blocks of 16 mixed heads
  constexpr int DS = HB / 4;                        // depth steps of the mixing: 4 heads each
  constexpr int HW = HB / NW > 0 ? HB / NW : 1;     // heads whose scores and softmax a wave does
  constexpr int NDB = D / 16;                       // blocks of 16 output numbers
  constexpr int HS = NW / NDB;                      // waves that share a block: each takes the heads h % HS == its own
  constexpr int HA = HB / HS > 0 ? HB / HS : 1;     // heads whose sums a wave holds
  static_assert(NW % NDB == 0 && NW >= NDB, "a wave owns one block of 16 output numbers");
  extern __shared__ __attribute__((aligned(16))) float tm_lds[];
  float* S = tm_lds;                                          // [H][TM_HEAD]
  float* alpha = S + (size_t)n_heads * TM_HEAD;               // [H][16]: what a row's sums so far are multiplied by
  bf16_t* vt = reinterpret_cast<bf16_t*>(alpha + n_heads * TM_Q);      // [gv][D][TM_VLD]: V^T of gv kv heads at a time

  // ---- which sequence, which 16 queries
  int wg = blockIdx.x, b = 0, q0 = -1, seq_start = 0, q_len = 0;
  for (b = 0; b < n_seqs; ++b) {
    seq_start = cu_seqlens[b];
    q_len = cu_seqlens[b + 1] - seq_start;
    const int tiles = (q_len + TM_Q - 1) / TM_Q;
    if (wg < tiles) {
      q0 = (tiles - 1 - wg) * TM_Q;        // a sequence's last queries walk the most pages: they start first
      break;
    }
    wg -= tiles;
  }
  if (q0 < 0) return;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int l16 = lane & 15, lg = lane >> 4;
  const int group = n_heads / n_kv;
  // scores are kept in units of log 2 (the mixing is linear, so the factor goes through it): the softmax is 2^(s - m)
  const float scale_log2 = scale * 1.4426950408889634f;
  const int past = past_len[b];
  const int n_valid = q_len - q0 < TM_Q ? q_len - q0 : TM_Q;
  const int pos_first = past + q0, pos_last = past + q0 + n_valid - 1;
  const int kv_last = past + q_len - 1;                       // the last key the sequence holds
  const int32_t* bt = block_table + (size_t)b * bt_stride;
  const int n_splits = gridDim.y;
  const int first_tile = tm_first_key(pos_first, chunk, window) / RB_PAGE + blockIdx.y, last_tile = pos_last / RB_PAGE;
  const int o_db = wave % NDB, o_hp = wave / NDB;          // this wave's block of output numbers, and which heads

  // rows of an MFMA result that this lane holds: queries 4 * lg + r
  int lo_r[4];
#pragma unroll
  for (int r = 0; r < 4; ++r) lo_r[r] = tm_first_key(pos_first + 4 * lg + r, chunk, window);
  // the row whose softmax this lane shares in: query lane / 4, keys 16 * (lane % 4) ...
  const int si = lane >> 2, sq = lane & 3;
  const int s_pos = pos_first + si, s_lo = tm_first_key(s_pos, chunk, window);
  const int lo_last = tm_first_key(pos_last, chunk, window);       // the latest first key of all rows

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
  f32x4_t oacc[HA];
#pragma unroll
  for (int a = 0; a < HA; ++a) oacc[a] = f32x4_t{0.f, 0.f, 0.f, 0.f};

  // ---- the heads whose scores this wave computes, and their queries (rows past the sequence's end read its last row)
  const int hpw = (n_heads + NW - 1) / NW;
  const int h_lo = wave * hpw, h_hi = h_lo + hpw < n_heads ? h_lo + hpw : n_heads;
  const size_t q_row = ((size_t)(seq_start + q0 + (l16 < n_valid ? l16 : n_valid - 1)) * n_heads) * D + lg * 8;
  constexpr bool QRES = HW * (D / 32) <= 4;        // the wave's queries stay in registers for all tiles
  Frag8 qres[QRES ? HW * (D / 32) : 1];
  if (QRES) {
#pragma unroll
    for (int k = 0; k < HW; ++k)
#pragma unroll
      for (int s = 0; s < D / 32; ++s)
        qres[k * (D / 32) + s].u = h_lo + k < h_hi ? load16(q + q_row + (size_t)(h_lo + k) * D + s * 32) : zero16();
  }

  // ---- V^T of a tile and gv kv heads: a thread takes 4 keys in a row and 8 numbers of each, and writes 8 times 4 keys
  constexpr int VU = 16 * (D / 8);                  // threads a kv head
  const int v_g = tid / VU, v_kq = tid & 15, v_dc = (tid % VU) >> 4;
  uint4 vreg[4];
  auto load_v = [&](int kt, int g0) {
    if (v_g >= gv || g0 + v_g >= n_kv) return;
    const bf16_t* src = v_pages + ((size_t)bt[kt] * n_kv + g0 + v_g) * RB_PAGE * D + (size_t)(4 * v_kq) * D + v_dc * 8;
#pragma unroll
    for (int e = 0; e < 4; ++e)      // what lies beyond the sequence may be anything, even NaN: zeros
      vreg[e] = kt * RB_PAGE + 4 * v_kq + e <= kv_last ? load16(src + (size_t)e * D) : zero16();
  };
  auto store_v = [&](int g0) {
    if (v_g >= gv || g0 + v_g >= n_kv) return;
    bf16_t* dst = vt + (size_t)v_g * D * TM_VLD + 4 * v_kq;
    const uint32_t w[4][4] = {{vreg[0].x, vreg[1].x, vreg[2].x, vreg[3].x}, {vreg[0].y, vreg[1].y, vreg[2].y, vreg[3].y},
                              {vreg[0].z, vreg[1].z, vreg[2].z, vreg[3].z}, {vreg[0].w, vreg[1].w, vreg[2].w, vreg[3].w}};
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      uint2 even, odd;
      even.x = (w[c][0] & 0xffffu) | (w[c][1] << 16);
      even.y = (w[c][2] & 0xffffu) | (w[c][3] << 16);
      odd.x = (w[c][0] >> 16) | (w[c][1] & 0xffff0000u);
      odd.y = (w[c][2] >> 16) | (w[c][3] & 0xffff0000u);
      *reinterpret_cast<uint2*>(dst + (v_dc * 8 + 2 * c) * TM_VLD) = even;
      *reinterpret_cast<uint2*>(dst + (v_dc * 8 + 2 * c + 1) * TM_VLD) = odd;
    }
  };
  // ---- the 64 keys of a tile and kv head as B operands, asked for together; where registers allow (heads of 64), those
  // of the wave's first kv head are asked for a tile ahead
  constexpr bool KP = D == 64;
  constexpr int KBL = KP ? 4 : 1;                  // key blocks of 16 asked for together
  Frag8 kf[KBL][D / 32];
  int g_have = -1;
  auto load_k = [&](int kt, int g, int kb0) {
    const bf16_t* krow = k_pages + (((size_t)bt[kt] * n_kv + g) * RB_PAGE + kb0 * 16 + l16) * D + lg * 8;
#pragma unroll
    for (int kb = 0; kb < KBL; ++kb)
#pragma unroll
      for (int s = 0; s < D / 32; ++s) kf[kb][s].u = load16(krow + (size_t)kb * 16 * D + s * 32);
    g_have = g;
  };
  if (KP && first_tile <= last_tile && h_lo < h_hi) load_k(first_tile, h_lo / group, 0);
  if (first_tile <= last_tile) load_v(first_tile, 0);

  for (int kt = first_tile; kt <= last_tile; kt += n_splits) {
    const size_t page_base = (size_t)bt[kt] * n_kv * RB_PAGE * D;
    const int key0 = kt * RB_PAGE;
    // every query of the workgroup sees every key of the tile: no masks
    const bool full = n_valid == TM_Q && key0 + RB_PAGE - 1 <= pos_first && key0 >= lo_last;
    // ---------------------------------------------------------------- 1. scores
    {
      if (!KP) g_have = -1;
#pragma unroll
      for (int k = 0; k < HW; ++k) {
        const int h = h_lo + k;
        if (h < h_hi) {
          const int g = h / group;
          if (KP && g != g_have) load_k(kt, g, 0);
          Frag8 qf[D / 32];
#pragma unroll
          for (int s = 0; s < D / 32; ++s) {
            if (QRES)
              qf[s] = qres[k * (D / 32) + s];
            else
              qf[s].u = load16(q + q_row + (size_t)h * D + s * 32);
          }
          float* dst = S + (size_t)h * TM_HEAD + l16;
#pragma unroll
          for (int kb = 0; kb < 4; ++kb) {
            if (!KP) load_k(kt, g, kb);
            f32x4_t acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int s = 0; s < D / 32; ++s) acc = mfma16(qf[s], kf[KP ? kb : 0][s], acc);
            if (full) {
#pragma unroll
              for (int r = 0; r < 4; ++r) dst[(4 * lg + r) * TM_ROW + kb * 16] = acc[r] * scale_log2;
            } else {
              const int key = key0 + kb * 16 + l16;
#pragma unroll
              for (int r = 0; r < 4; ++r) {
                const int i = 4 * lg + r;
                const bool seen = i < n_valid && key <= pos_first + i && key >= lo_r[r];
                dst[i * TM_ROW + kb * 16] = seen ? acc[r] * scale_log2 : 0.f;       // a select: a key beyond the sequence may be anything
              }
            }
          }
        }
      }
      if (KP && kt + n_splits <= last_tile && h_lo < h_hi) load_k(kt + n_splits, h_lo / group, 0);
    }
    __syncthreads();
    // ---------------------------------------------------------------- 2. mixing over the heads
    if (talk) {
      for (int cb = wave; cb < TM_Q * 4; cb += NW) {
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
      const int h = wave + NW * k;
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
        if (!full) {
#pragma unroll
          for (int e = 0; e < 16; ++e) {
            const int key = key0 + sq * 16 + e;
            const bool seen = si < n_valid && key <= s_pos && key >= s_lo;
            p[e] = seen ? p[e] : -INFINITY;
          }
        }
        float mx = fmaxf(p[0], p[1]);
#pragma unroll
        for (int e = 2; e < 16; e += 2) mx = fmaxf(mx, fmaxf(p[e], p[e + 1]));
        mx = fmaxf(mx, __shfl_xor(mx, 1, 64));
        mx = fmaxf(mx, __shfl_xor(mx, 2, 64));
        const float m_new = fmaxf(m_run[k], mx);
        const float m_safe = m_new == -INFINITY ? 0.f : m_new;
        float sum = 0.f;
#pragma unroll
        for (int e = 0; e < 16; ++e) {
          p[e] = __builtin_amdgcn_exp2f(p[e] - m_safe);        // 2^(-inf) = 0
          sum += p[e];
        }
        sum += __shfl_xor(sum, 1, 64);
        sum += __shfl_xor(sum, 2, 64);
        const float a = __builtin_amdgcn_exp2f(m_run[k] - m_safe);      // nothing seen so far: 0
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
    for (int g0 = 0; g0 < n_kv; g0 += gv) {
      store_v(g0);
      if (g0 + gv < n_kv)
        load_v(kt, g0 + gv);
      else if (kt + n_splits <= last_tile)
        load_v(kt + n_splits, 0);
      __syncthreads();
#pragma unroll
      for (int a = 0; a < HA; ++a) {
        const int h = a * HS + o_hp;
        const int kvh = h / group - g0;
        if (h < n_heads && kvh >= 0 && kvh < gv) {
          const bf16_t* vrow = vt + (size_t)kvh * D * TM_VLD + (o_db * 16 + l16) * TM_VLD + lg * 8;
          float a_r[4];
#pragma unroll
          for (int r = 0; r < 4; ++r) a_r[r] = alpha[h * TM_Q + 4 * lg + r];
#pragma unroll
          for (int r = 0; r < 4; ++r) oacc[a][r] *= a_r[r];
          const bf16_t* prow = reinterpret_cast<const bf16_t*>(S + (size_t)h * TM_HEAD + l16 * TM_ROW) + lg * 8;
#pragma unroll
          for (int ks = 0; ks < 2; ++ks) {
            Frag8 p_hi, p_lo, vf;
            p_hi.u = *reinterpret_cast<const uint4*>(prow + ks * 32);
            p_lo.u = *reinterpret_cast<const uint4*>(prow + 64 + ks * 32);
            vf.u = *reinterpret_cast<const uint4*>(vrow + ks * 32);
            oacc[a] = mfma16(p_hi, vf, oacc[a]);
            oacc[a] = mfma16(p_lo, vf, oacc[a]);
          }
        }
      }
      __syncthreads();
    }
  }

  // ---- the rows' sums (and maxima) to everyone, and out
  float* m_all = S;                           // [H][16]: the scores are done with
#pragma unroll
  for (int k = 0; k < HW; ++k) {
    const int h = wave + NW * k;
    if (h < n_heads && sq == 0) {
      alpha[h * TM_Q + si] = l_run[k];
      m_all[h * TM_Q + si] = m_run[k];
    }
  }
  __syncthreads();
  if (n_splits == 1) {
#pragma unroll
    for (int a = 0; a < HA; ++a) {
      const int h = a * HS + o_hp;
      if (h < n_heads) {
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int i = 4 * lg + r;
          if (i < n_valid) {
            const float l = alpha[h * TM_Q + i];
            Num<bf16_t>::store(out + ((size_t)(seq_start + q0 + i) * n_heads + h) * D + o_db * 16 + l16,
                               oacc[a][r] * (l > 0.f ? 1.0f / l : 0.f));
          }
        }
      }
    }
    return;
  }
  const size_t part_row = (size_t)blockIdx.y * n_tokens + seq_start + q0;
#pragma unroll
  for (int a = 0; a < HA; ++a) {
    const int h = a * HS + o_hp;
    if (h < n_heads) {
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int i = 4 * lg + r;
        if (i < n_valid) part_o[((part_row + i) * n_heads + h) * D + o_db * 16 + l16] = oacc[a][r];
      }
    }
  }
  for (int e = tid; e < n_heads * TM_Q; e += 64 * NW) {
    const int h = e / TM_Q, i = e % TM_Q;
    if (i < n_valid) {
      float* ml = part_ml + ((part_row + i) * n_heads + h) * 2;
      ml[0] = m_all[e];
      ml[1] = alpha[e];
    }
  }
}

// out[t, h, :] = sum_s o_s 2^(m_s - m) / sum_s l_s 2^(m_s - m), m the largest m_s (maxima in units of log 2): a wave a
// (token, head)
template <int D>
__global__ __launch_bounds__(256) void attention_mixed_combine_kernel(const float* __restrict__ part_o, const float* __restrict__ part_ml,
                                                                       bf16_t* __restrict__ out, int n_rows, int n_splits) {
  const int row = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
  if (row >= n_rows) return;
  float m = -INFINITY;
  for (int s = 0; s < n_splits; ++s) m = fmaxf(m, part_ml[((size_t)s * n_rows + row) * 2]);
  float l = 0.f, acc[D / 64];
#pragma unroll
  for (int d = 0; d < D / 64; ++d) acc[d] = 0.f;
  for (int s = 0; s < n_splits; ++s) {
    const float* ml = part_ml + ((size_t)s * n_rows + row) * 2;
    const float w = ml[0] == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(ml[0] - m);
    l = fmaf(ml[1], w, l);
    const float* o = part_o + ((size_t)s * n_rows + row) * D + lane;
#pragma unroll
    for (int d = 0; d < D / 64; ++d) acc[d] = fmaf(o[64 * d], w, acc[d]);
  }
  const float inv = l > 0.f ? 1.0f / l : 0.f;
#pragma unroll
  for (int d = 0; d < D / 64; ++d) Num<bf16_t>::store(out + (size_t)row * D + 64 * d + lane, acc[d] * inv);
}

template <int D, int HB, int NW>
static int launch_mixed_mfma(const void* q, const void* k_pages, const void* v_pages, void* out, const int32_t* cu_seqlens,
                             const int32_t* past_len, const int32_t* block_table, int bt_stride, int n_seqs, int n_tokens,
                             int n_heads, int n_kv, float scale, const float* talk, int chunk, int window, int n_splits,
                             float* workspace, hipStream_t s) {
  // V^T of as many kv heads at a time as LDS holds beside the scores and the workgroup's threads fetch at once
  const size_t fixed = sizeof(float) * ((size_t)n_heads * TM_HEAD + (size_t)n_heads * TM_Q), one = sizeof(bf16_t) * (size_t)D * TM_VLD;
  RB_REQUIRE(fixed + one <= 160 * 1024, "rb_attention_mixed_bf16: %zu bytes of LDS are more than a workgroup has", fixed + one);
  int gv = (int)((160 * 1024 - fixed) / one);
  if (gv > n_kv) gv = n_kv;
  if (gv > 64 * NW / (16 * (D / 8))) gv = 64 * NW / (16 * (D / 8));
  const size_t lds = fixed + gv * one;
  auto kernel = attention_mixed_mfma_kernel<D, HB, NW>;
  if (lds > 64 * 1024) {
    static bool raised = false;          // per instantiation
    if (!raised) {
      RB_REQUIRE(hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024) == hipSuccess,
                 "rb_attention_mixed_bf16: cannot have %zu bytes of LDS", lds);
      raised = true;
    }
  }
  // an upper bound of the 16-query tiles that depends on the step's shape alone: workgroups past the last tile leave
  const int tiles = n_tokens / TM_Q + n_seqs;
  float* part_o = workspace;
  float* part_ml = workspace ? workspace + (size_t)n_splits * n_tokens * n_heads * D : nullptr;
  kernel<<<dim3(tiles, n_splits), 64 * NW, lds, s>>>((const bf16_t*)q, (const bf16_t*)k_pages, (const bf16_t*)v_pages, (bf16_t*)out,
                                                      cu_seqlens, past_len, block_table, bt_stride, n_seqs, n_heads, n_kv, scale, talk,
                                                      chunk, window, part_o, part_ml, n_tokens, gv);
  RB_LAUNCH_CHECK();
  if (n_splits > 1) {
    const int rows = n_tokens * n_heads;
    attention_mixed_combine_kernel<D><<<(rows + 3) / 4, 256, 0, s>>>(part_o, part_ml, (bf16_t*)out, rows, n_splits);
    RB_LAUNCH_CHECK();
  }
  return 0;
}

extern "C" int rb_attention_mixed_bf16(const void* q, const void* k_pages, const void* v_pages, void* out,
                                       const int32_t* cu_seqlens, const int32_t* past_len, const int32_t* block_table,
                                       int bt_stride, int n_seqs, int n_tokens, int n_heads, int n_kv_heads, int head_dim,
                                       float scale, const float* talk, int chunk, int window, int n_splits, float* workspace,
                                       void* stream) {
  RB_RECORDED(rb_attention_mixed_bf16(q, k_pages, v_pages, out, cu_seqlens, past_len, block_table, bt_stride, n_seqs, n_tokens,
                                      n_heads, n_kv_heads, head_dim, scale, talk, chunk, window, n_splits, workspace, stream));
  RB_REQUIRE(n_seqs >= 0 && n_tokens >= 0 && n_heads > 0 && n_kv_heads > 0 && n_heads % n_kv_heads == 0 && chunk >= 0 && window >= 0,
             "rb_attention_mixed_bf16: bad sizes B=%d T=%d Hq=%d Hk=%d", n_seqs, n_tokens, n_heads, n_kv_heads);
  RB_REQUIRE(head_dim == 64 || head_dim == 128, "rb_attention_mixed_bf16: head_dim %d not supported (64 or 128; use rb_attention_mixed)",
             head_dim);
  RB_REQUIRE(n_heads <= TM_MAX_HEADS, "rb_attention_mixed_bf16: %d heads are more than a workgroup takes (%d; use rb_attention_mixed)",
             n_heads, TM_MAX_HEADS);
  RB_REQUIRE(talk != nullptr, "rb_attention_mixed_bf16: no mixing matrix (the identity, if the heads are not mixed)");
  RB_REQUIRE(n_splits >= 1 && n_splits <= 64 && (n_splits == 1 || workspace != nullptr),
             "rb_attention_mixed_bf16: %d splits need a workspace of splits * T * Hq * (head_dim + 2) numbers", n_splits);
  if (n_seqs == 0 || n_tokens == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
#define TM_LAUNCH(D_, HB_, NW_)                                                                                                    \
  return launch_mixed_mfma<D_, HB_, NW_>(q, k_pages, v_pages, out, cu_seqlens, past_len, block_table, bt_stride, n_seqs, n_tokens, \
                                         n_heads, n_kv_heads, scale, talk, chunk, window, n_splits, workspace, s)
  if (head_dim == 64) {
    if (n_heads <= 8) TM_LAUNCH(64, 8, 8);
    if (n_heads <= 16) TM_LAUNCH(64, 16, 8);
    TM_LAUNCH(64, 32, 8);
  }
  if (n_heads <= 8) TM_LAUNCH(128, 8, 8);
  if (n_heads <= 16) TM_LAUNCH(128, 16, 8);
  TM_LAUNCH(128, 32, 8);
#undef TM_LAUNCH
}
