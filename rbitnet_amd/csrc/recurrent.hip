// Layers that carry a fixed-size state from token to token: the short causal convolution over time
// (per channel, a few taps) and the gated delta rule (per head a matrix S [key dim, value dim] that
// decays per key channel, is corrected towards the new value along the new key, and is read with the
// query).  States are float32 and live in the cache's per-slot storage; a step brings any number of
// tokens per sequence on top of what the state holds.  All arithmetic here is float32.
#include <math.h>

#include "api.h"
#include "common.h"

__device__ __forceinline__ float rb_sigmoid(float v) { return 1.0f / (1.0f + expf(-v)); }
__device__ __forceinline__ float rb_softplus(float v) { return v > 20.0f ? v : log1pf(expf(v)); }

// ---------------------------------------------------------------- short convolution
// y[t, c] = (residual ? x[t, c] : 0) + sum_d w[c, taps - 1 - d] * x[t - d, c], d = 0 .. taps - 1, where rows
// before the step's first come from the sequence's state (its last taps - 1 inputs, oldest first) and rows
// before the sequence's start are zero (the state of a fresh slot is zero).  act 1: silu on the result.
// Afterwards the state holds the last taps - 1 inputs again.  One launch: workgroups that walk 16 rows each of the
// tokens that need rows of the step only, and a workgroup per sequence that walks the step's first taps - 1 tokens with
// the old state in registers and then writes the new state, so that whoever reads the state is also who writes it.
#define SC_MAX_TAPS 16
#define SC_TILE 16             // rows of the step that a workgroup walks
template <typename TO>
__global__ void short_conv_kernel(const float* __restrict__ x, size_t x_stride, const float* __restrict__ bias,
                                  const float* __restrict__ w, int taps,
                                  float* __restrict__ state, const int32_t* __restrict__ tok_pos,
                                  const int32_t* __restrict__ tok_seq, const int32_t* __restrict__ cu_seqlens,
                                  const int32_t* __restrict__ slots, TO* __restrict__ out, size_t out_stride,
                                  int residual, int act, int channels, int n_tokens, int n_tiles) {
  const int keep = taps - 1;
  if ((int)blockIdx.x < n_tiles) {
    // SC_TILE rows of the packed step, walked with the window (the last taps - 1 inputs) in registers: one new row a
    // token.  Rows that are among a sequence's first taps - 1 of the step belong to the sequence's workgroup; after such
    // a row (and at the tile's start) the window is read anew.
    const int r0 = blockIdx.x * SC_TILE;
    const int r1 = r0 + SC_TILE < n_tokens ? r0 + SC_TILE : n_tokens;
    for (int c = blockIdx.y * blockDim.x + threadIdx.x; c < channels; c += gridDim.y * blockDim.x) {
      float win[SC_MAX_TAPS], wt[SC_MAX_TAPS];
#pragma unroll
      for (int j = 0; j < SC_MAX_TAPS; ++j) {
        win[j] = 0.f;
        wt[j] = j < keep ? w[(size_t)c * taps + j] : 0.f;
      }
      const float w_cur = w[(size_t)c * taps + keep];
      const float bc = bias ? bias[c] : 0.f;
      bool have = false;
      for (int t = r0; t < r1; ++t) {
        if (t - cu_seqlens[tok_seq[t]] < keep) {             // the sequence's workgroup takes it
          have = false;
          continue;
        }
        if (!have) {
#pragma unroll
          for (int j = 0; j < SC_MAX_TAPS; ++j)
            if (j < keep) win[j] = x[(size_t)(t - keep + j) * x_stride + c] + bc;
          have = true;
        }
        const float cur = x[(size_t)t * x_stride + c] + bc;
        float acc = residual ? cur : 0.f;
        acc = fmaf(w_cur, cur, acc);
#pragma unroll
        for (int j = 0; j < SC_MAX_TAPS; ++j) acc = fmaf(wt[j], win[j], acc);
#pragma unroll
        for (int j = 0; j < SC_MAX_TAPS - 1; ++j) win[j] = j + 1 < keep ? win[j + 1] : win[j];
#pragma unroll
        for (int j = 0; j < SC_MAX_TAPS; ++j)
          if (j == keep - 1) win[j] = cur;
        if (act == 1) acc = acc * rb_sigmoid(acc);
        Num<TO>::store(out + (size_t)t * out_stride + c, acc);
      }
    }
    return;
  }
  const int b = blockIdx.x - n_tiles;
  const int row0 = cu_seqlens[b], n = cu_seqlens[b + 1] - row0;
  float* st = state + (size_t)slots[b] * keep * channels;
  const int first = n < keep ? n : keep;
  for (int c = blockIdx.y * blockDim.x + threadIdx.x; c < channels; c += gridDim.y * blockDim.x) {
    float win[SC_MAX_TAPS], wt[SC_MAX_TAPS];                 // the last `keep` inputs, oldest first; their weights
#pragma unroll
    for (int j = 0; j < SC_MAX_TAPS; ++j) {
      win[j] = j < keep ? st[(size_t)j * channels + c] : 0.f;
      wt[j] = j < keep ? w[(size_t)c * taps + j] : 0.f;
    }
    const float w_cur = w[(size_t)c * taps + keep];
    const float bc = bias ? bias[c] : 0.f;
    float nxt = first > 0 ? x[(size_t)row0 * x_stride + c] + bc : 0.f;
    __builtin_amdgcn_sched_barrier(0);                       // state, weights and the first row: one trip to memory together
    for (int i = 0; i < first; ++i) {
      const float cur = nxt;
      if (i + 1 < first) nxt = x[(size_t)(row0 + i + 1) * x_stride + c] + bc;
      float acc = residual ? cur : 0.f;
      acc = fmaf(w_cur, cur, acc);
#pragma unroll
      for (int j = 0; j < SC_MAX_TAPS; ++j) acc = fmaf(wt[j], win[j], acc);
#pragma unroll
      for (int j = 0; j < SC_MAX_TAPS - 1; ++j) win[j] = j + 1 < keep ? win[j + 1] : win[j];
#pragma unroll
      for (int j = 0; j < SC_MAX_TAPS; ++j)
        if (j == keep - 1) win[j] = cur;
      if (act == 1) acc = acc * rb_sigmoid(acc);
      Num<TO>::store(out + (size_t)(row0 + i) * out_stride + c, acc);
    }
#pragma unroll
    for (int j = 0; j < SC_MAX_TAPS; ++j)
      if (j < keep) st[(size_t)j * channels + c] = n > keep ? x[(size_t)(row0 + n - keep + j) * x_stride + c] + bc : win[j];
  }
}

extern "C" int rb_short_conv(const float* x, long long x_stride, const float* w, int taps, float* state,
                             const int32_t* tok_pos, const int32_t* tok_seq, const int32_t* cu_seqlens,
                             const int32_t* slots, void* out, long long out_stride, int out_dtype, int residual,
                             int act, int n_tokens, int n_seqs, int channels, void* stream) {
  RB_RECORDED(rb_short_conv(x, x_stride, w, taps, state, tok_pos, tok_seq, cu_seqlens, slots, out, out_stride, out_dtype,
                            residual, act, n_tokens, n_seqs, channels, stream));
  return rb_short_conv_bias(x, x_stride, nullptr, w, taps, state, tok_pos, tok_seq, cu_seqlens, slots, out, out_stride, out_dtype,
                            residual, act, n_tokens, n_seqs, channels, stream);
}

// The same on x + bias (bias float32 [C], null: none): the bias belongs to the inputs, so the state holds them with it and
// rows before a sequence's start stay zero.
extern "C" int rb_short_conv_bias(const float* x, long long x_stride, const float* bias, const float* w, int taps, float* state,
                                  const int32_t* tok_pos, const int32_t* tok_seq, const int32_t* cu_seqlens,
                                  const int32_t* slots, void* out, long long out_stride, int out_dtype, int residual,
                                  int act, int n_tokens, int n_seqs, int channels, void* stream) {
  RB_RECORDED(rb_short_conv_bias(x, x_stride, bias, w, taps, state, tok_pos, tok_seq, cu_seqlens, slots, out, out_stride, out_dtype,
                                 residual, act, n_tokens, n_seqs, channels, stream));
  RB_REQUIRE(n_tokens >= 0 && n_seqs >= 0 && channels > 0 && taps >= 1 && taps - 1 <= SC_MAX_TAPS,
             "rb_short_conv: bad sizes T=%d B=%d C=%d taps=%d (at most %d)", n_tokens, n_seqs, channels, taps, SC_MAX_TAPS + 1);
  RB_REQUIRE(x_stride >= channels && out_stride >= channels, "rb_short_conv: a row stride is shorter than the channels");
  RB_REQUIRE(taps == 1 || state != nullptr, "rb_short_conv: %d taps need a state", taps);
  RB_REQUIRE(act == 0 || act == 1, "rb_short_conv: unknown activation %d", act);
  if (n_tokens == 0) return 0;
  const int n_tiles = (n_tokens + SC_TILE - 1) / SC_TILE;
  dim3 grid(n_tiles + (taps > 1 ? n_seqs : 0), (channels + 255) / 256 < 64 ? (channels + 255) / 256 : 64);
  hipStream_t s = (hipStream_t)stream;
  if (out_dtype == RB_F32)
    short_conv_kernel<float><<<grid, 256, 0, s>>>(x, (size_t)x_stride, bias, w, taps, state, tok_pos, tok_seq, cu_seqlens, slots,
                                                  (float*)out, (size_t)out_stride, residual, act, channels, n_tokens, n_tiles);
  else if (out_dtype == RB_BF16)
    short_conv_kernel<bf16_t><<<grid, 256, 0, s>>>(x, (size_t)x_stride, bias, w, taps, state, tok_pos, tok_seq, cu_seqlens, slots,
                                                   (bf16_t*)out, (size_t)out_stride, residual, act, channels, n_tokens, n_tiles);
  else
    RB_REQUIRE(false, "rb_short_conv: unknown dtype %d", out_dtype);
  RB_LAUNCH_CHECK();
  return 0;
}

// ---------------------------------------------------------------- what enters a recurrence
// Per token, in place.  The q and k heads (n_kv of each, `dim` numbers): unit 1 makes each a unit vector,
// x / sqrt(sum x^2 + unit_eps); q is also multiplied by q_scale (unit 0: only that).  The a_cols numbers of a row of
// `a` become decays, a_cols being H (one per head) or H * dim (one per head and key channel), h = i / (a_cols / H):
//   decay 0:  exp(-exp(a_log[h]) * softplus(a + bias[i]))
//   decay 1:  sigmoid(a + bias[i]) ^ (1 / tau), computed as exp(-softplus(-(a + bias[i])) / tau)
//   decay 2:  exp(-exp(a + bias[i]))
// beta[t, h] = sigmoid(b[t, h]) where b_in is given.
__global__ __launch_bounds__(1024) void recurrence_prep_kernel(float* __restrict__ qk, size_t qk_stride, int n_kv, int dim, int unit,
                                  float* __restrict__ a, size_t a_stride, int a_cols, int decay, const float* __restrict__ bias,
                                  const float* __restrict__ a_log, float tau, int n_heads,
                                  const float* __restrict__ b_in, size_t b_stride, float* __restrict__ beta,
                                  float q_scale, float unit_eps) {
  const int t = blockIdx.x;
  const int lane = threadIdx.x & (RB_WAVE - 1);
  const int wave = threadIdx.x / RB_WAVE, n_waves = blockDim.x / RB_WAVE;
  float* row = qk + (size_t)t * qk_stride;
  if (unit) {
    for (int v = wave; v < 2 * n_kv; v += n_waves) {           // the q heads, then the k heads
      float* p = row + (size_t)v * dim;
      float ss = 0.f;
      for (int i = lane; i < dim; i += RB_WAVE) ss = fmaf(p[i], p[i], ss);
      ss = wave_sum(ss);
      const float f = (v < n_kv ? q_scale : 1.0f) / sqrtf(ss + unit_eps);
      for (int i = lane; i < dim; i += RB_WAVE) p[i] *= f;
    }
  } else if (q_scale != 1.0f) {
    for (int i = threadIdx.x; i < n_kv * dim; i += blockDim.x) row[i] *= q_scale;
  }
  float* ar = a + (size_t)t * a_stride;
  const int per_head = a_cols / n_heads;
  for (int i = threadIdx.x; i < a_cols; i += blockDim.x) {
    const float z = ar[i] + (bias ? bias[i] : 0.f);
    if (decay == 0)
      ar[i] = expf(-expf(a_log[i / per_head]) * rb_softplus(z));
    else if (decay == 1)
      ar[i] = expf(-rb_softplus(-z) / tau);
    else
      ar[i] = expf(-expf(z));
  }
  if (b_in)
    for (int h = threadIdx.x; h < n_heads; h += blockDim.x) beta[(size_t)t * n_heads + h] = rb_sigmoid(b_in[(size_t)t * b_stride + h]);
}

extern "C" int rb_recurrence_prep(float* qk, long long qk_stride, int n_kv_heads, int dim, int unit, float q_scale, float unit_eps,
                                  float* a, long long a_stride, int a_cols, int decay, const float* bias, const float* a_log,
                                  float tau, int n_heads, const float* b_in, long long b_stride, float* beta, int n_tokens,
                                  void* stream) {
  RB_RECORDED(rb_recurrence_prep(qk, qk_stride, n_kv_heads, dim, unit, q_scale, unit_eps, a, a_stride, a_cols, decay, bias, a_log,
                                 tau, n_heads, b_in, b_stride, beta, n_tokens, stream));
  RB_REQUIRE(n_tokens >= 0 && n_kv_heads >= 0 && n_heads > 0 && dim > 0, "rb_recurrence_prep: bad sizes");      // no q/k heads: the decays alone
  RB_REQUIRE(a_cols == n_heads || a_cols == n_heads * dim, "rb_recurrence_prep: %d decays a token for %d heads of %d", a_cols,
             n_heads, dim);
  RB_REQUIRE(qk_stride >= 2LL * n_kv_heads * dim && a_stride >= a_cols && (b_in == nullptr || b_stride >= n_heads),
             "rb_recurrence_prep: a row stride is too short");
  RB_REQUIRE((decay == 0 && a_log != nullptr) || (decay == 1 && tau > 0.f) || decay == 2,
             "rb_recurrence_prep: decay %d lacks its constants", decay);
  RB_REQUIRE(b_in == nullptr || beta != nullptr, "rb_recurrence_prep: beta has nowhere to go");
  if (n_tokens == 0) return 0;
  // a step of few tokens has few workgroups, and a token's heads are a chain of trips to memory for each wave: more waves then
  const int threads = n_tokens < 2 * rb_compute_units() ? 1024 : 256;
  recurrence_prep_kernel<<<n_tokens, threads, 0, (hipStream_t)stream>>>(qk, (size_t)qk_stride, n_kv_heads, dim, unit, a, (size_t)a_stride,
                                                                    a_cols, decay, bias, a_log, tau, n_heads, b_in, (size_t)b_stride,
                                                                    beta, q_scale, unit_eps);
  RB_LAUNCH_CHECK();
  return 0;
}

// The gated delta rule with a decay per key channel: unit vectors, decay 0 on H * dim numbers, beta.
extern "C" int rb_delta_prep(float* qk, long long qk_stride, int n_kv_heads, int dim, float* a, long long a_stride, const float* dt_bias,
                             const float* a_log, int n_heads, const float* b_in, long long b_stride, float* beta,
                             float q_scale, float unit_eps, int n_tokens, void* stream) {
  RB_RECORDED(rb_delta_prep(qk, qk_stride, n_kv_heads, dim, a, a_stride, dt_bias, a_log, n_heads, b_in, b_stride, beta, q_scale,
                            unit_eps, n_tokens, stream));
  return rb_recurrence_prep(qk, qk_stride, n_kv_heads, dim, 1, q_scale, unit_eps, a, a_stride, n_heads * dim, 0, dt_bias, a_log, 1.0f,
                            n_heads, b_in, b_stride, beta, n_tokens, stream);
}

// ---------------------------------------------------------------- gated delta rule: the recurrence
// Per sequence and head, token after token:
//   S <- diag(g) S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q
// The columns of S (one per value channel) do not meet: a column is held by RG lanes, each with DKL of its rows in
// registers; the dot products over the rows are finished among the RG lanes by moves inside a row of lanes.  A workgroup is one wave
// and holds 64 / RG columns.  Tokens go by in chunks of CH: q, k, g, v and beta of a chunk lie in LDS for all lanes, and
// the next chunk's loads are in flight (in registers) while the current one is computed, so that a token costs its
// arithmetic and no trip to memory; the chunk's outputs leave through LDS as whole rows.  The state is read once and
// written once.
// The sum over each group of RG neighbouring lanes (RG = 4, 8 or 16), in every lane of the group, by moves inside a
// row of 16 lanes (no trip through LDS): the two swaps inside a quad, then the mirror of a half row, then of a row.
template <int RG>
__device__ __forceinline__ float lanes_sum(float v) {
  static_assert(RG == 4 || RG == 8 || RG == 16, "groups of 4, 8 or 16 lanes");
  v += __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, v), 0xB1, 0xF, 0xF, true));   // quad_perm [1,0,3,2]
  v += __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, v), 0x4E, 0xF, 0xF, true));   // quad_perm [2,3,0,1]
  if (RG >= 8) v += __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, v), 0x141, 0xF, 0xF, true));   // row_half_mirror
  if (RG >= 16) v += __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, v), 0x140, 0xF, 0xF, true));  // row_mirror
  return v;
}

template <int DKL, int RG, int CH, bool BONUS>
__global__ __launch_bounds__(RB_WAVE) void delta_rule_kernel(
    const float* __restrict__ q, const float* __restrict__ k, size_t qk_stride, const float* __restrict__ v,
    size_t v_stride, const float* __restrict__ g, size_t g_stride, const float* __restrict__ beta, float* __restrict__ state,
    const int32_t* __restrict__ cu_seqlens, const int32_t* __restrict__ slots, float* __restrict__ out, int n_heads,
    int n_kv, int dim, int vdim, int g_per_head, const float* __restrict__ bonus) {
  constexpr int COLS = RB_WAVE / RG;
  constexpr int DK = DKL * RG;               // rows held, >= dim; rows beyond dim stay zero
  constexpr int NQ = DK * CH / RB_WAVE;      // q (or k, or g) values of a chunk per lane
  constexpr int NV = (COLS * CH + RB_WAVE - 1) / RB_WAVE;
  __shared__ float sq[CH][DK], sk[CH][DK], sg[CH][DK], sv[CH][COLS], so[CH][COLS], sb[CH];
  const int b = blockIdx.x, h = blockIdx.y;
  const int lane = threadIdx.x;
  const int col0 = blockIdx.z * COLS;
  const int col = col0 + lane / RG;
  const int rg = lane % RG;
  const bool on = col < vdim;
  const int kvh = h / (n_heads / n_kv);
  const int row0 = cu_seqlens[b], n = cu_seqlens[b + 1] - row0;
  // the state is kept column by column, [slots, H, vdim, dim]: a lane's rows are DKL numbers in a row and a wave's
  // columns one piece of memory (with S as rows a wave of four columns used a quarter of every line it touched)
  float* S = state + (((size_t)slots[b] * n_heads + h) * vdim + (on ? col : 0)) * dim;
  float s[DKL];
  const bool quads = dim % 4 == 0 && DKL % 4 == 0 && (reinterpret_cast<uintptr_t>(state) & 15) == 0;
  if (quads) {
#pragma unroll
    for (int i = 0; i < DKL; i += 4) {
      const int r = rg * DKL + i;
      const float4 v4 = (on && r < dim) ? *reinterpret_cast<const float4*>(S + r) : make_float4(0.f, 0.f, 0.f, 0.f);
      s[i] = v4.x;
      s[i + 1] = v4.y;
      s[i + 2] = v4.z;
      s[i + 3] = v4.w;
    }
  } else {
#pragma unroll
    for (int i = 0; i < DKL; ++i) {
      const int r = rg * DKL + i;
      s[i] = (on && r < dim) ? S[r] : 0.f;
    }
  }
  // BONUS: the read-out sees the state as it was before the token, and the token's own k v^T times a weight per key
  // channel: o = S^T q + v sum_i bonus_i k_i q_i;  then S <- diag(g) S + k v^T
  float ub[DKL];
#pragma unroll
  for (int i = 0; i < DKL; ++i) {
    const int r = rg * DKL + i;
    ub[i] = (BONUS && r < dim) ? bonus[(size_t)h * dim + r] : 0.f;
  }
  float rq[NQ], rk[NQ], rgt[NQ], rv[NV], rb = 0.f;
  auto fetch = [&](int t0) {
    const int nt = n - t0 < CH ? n - t0 : CH;
#pragma unroll
    for (int j = 0; j < NQ; ++j) {
      const int e = lane + RB_WAVE * j, tt = e / DK, i = e - tt * DK;
      const bool in = tt < nt && i < dim;
      const size_t t = (size_t)(row0 + t0 + tt);
      rq[j] = in ? q[t * qk_stride + (size_t)kvh * dim + i] : 0.f;
      rk[j] = in ? k[t * qk_stride + (size_t)kvh * dim + i] : 0.f;
      rgt[j] = in ? (g_per_head ? g[t * g_stride + h] : g[t * g_stride + (size_t)h * dim + i]) : 0.f;
    }
#pragma unroll
    for (int j = 0; j < NV; ++j) {
      const int e = lane + RB_WAVE * j, tt = e / COLS, c = e - tt * COLS;
      rv[j] = (tt < nt && col0 + c < vdim) ? v[(size_t)(row0 + t0 + tt) * v_stride + (size_t)h * vdim + col0 + c] : 0.f;
    }
    rb = (beta && lane < nt) ? beta[(size_t)(row0 + t0 + lane) * n_heads + h] : 0.f;
  };
  if (n > 0) fetch(0);
  for (int t0 = 0; t0 < n; t0 += CH) {
    const int nt = n - t0 < CH ? n - t0 : CH;
    __syncthreads();                                   // the chunk before has been read and its outputs are out
#pragma unroll
    for (int j = 0; j < NQ; ++j) {
      const int e = lane + RB_WAVE * j, tt = e / DK, i = e - tt * DK;
      sq[tt][i] = rq[j];
      sk[tt][i] = rk[j];
      sg[tt][i] = rgt[j];
    }
#pragma unroll
    for (int j = 0; j < NV; ++j) {
      const int e = lane + RB_WAVE * j;
      if (e < COLS * CH) sv[e / COLS][e % COLS] = rv[j];
    }
    if (lane < CH) sb[lane] = rb;
    __syncthreads();
    if (t0 + CH < n) fetch(t0 + CH);                   // in flight while this chunk is computed
    __builtin_amdgcn_sched_barrier(0);                 // (issued here, not where the scheduler would sink them: at their use)
    // One token: with D = diag(g) S and u = beta (v - D^T k), the read-out of the updated state is
    // (D + k u^T)^T q = D^T q + u (k . q): one pass over the decayed column gives both dot products, and a token has
    // one reduction among the RG lanes on its way instead of two.  Two partial sums each: shorter chains of additions.
    auto token = [&](int tt) {
      const float vv = sv[tt][lane / RG];
      const float bt = sb[tt];
      float kv0 = 0.f, kv1 = 0.f, dq0 = 0.f, dq1 = 0.f, kq0 = 0.f, kq1 = 0.f;
#pragma unroll
      for (int i = 0; i < DKL; i += 2) {
        const float k0 = sk[tt][rg * DKL + i], q0 = sq[tt][rg * DKL + i];
        const float k1 = sk[tt][rg * DKL + i + 1], q1 = sq[tt][rg * DKL + i + 1];
        if (BONUS) {
          dq0 = fmaf(s[i], q0, dq0);
          dq1 = fmaf(s[i + 1], q1, dq1);
          kq0 = fmaf(ub[i] * k0, q0, kq0);
          kq1 = fmaf(ub[i + 1] * k1, q1, kq1);
          s[i] *= sg[tt][rg * DKL + i];
          s[i + 1] *= sg[tt][rg * DKL + i + 1];
          continue;
        }
        s[i] *= sg[tt][rg * DKL + i];
        s[i + 1] *= sg[tt][rg * DKL + i + 1];
        kv0 = fmaf(s[i], k0, kv0);
        kv1 = fmaf(s[i + 1], k1, kv1);
        dq0 = fmaf(s[i], q0, dq0);
        dq1 = fmaf(s[i + 1], q1, dq1);
        kq0 = fmaf(k0, q0, kq0);
        kq1 = fmaf(k1, q1, kq1);
      }
      const float kv = BONUS ? 0.f : lanes_sum<RG>(kv0 + kv1);
      const float dq = lanes_sum<RG>(dq0 + dq1);
      const float kq = lanes_sum<RG>(kq0 + kq1);
      const float u = (!BONUS && beta) ? bt * (vv - kv) : vv;       // without beta: the plain rule, S <- diag(g) S + k v^T
#pragma unroll
      for (int i = 0; i < DKL; ++i) s[i] = fmaf(sk[tt][rg * DKL + i], u, s[i]);
      if (rg == 0) so[tt][lane / RG] = fmaf(u, kq, dq);
    };
    if (nt == CH) {
      // a whole chunk as straight code, so that a token's reads from LDS are issued while the one before is computed
#pragma unroll
      for (int tt = 0; tt < CH; ++tt) token(tt);
    } else {
      for (int tt = 0; tt < nt; ++tt) token(tt);
    }
    __syncthreads();
    for (int e = lane; e < nt * COLS; e += RB_WAVE) {
      const int tt = e / COLS, c = e - tt * COLS;
      if (col0 + c < vdim) out[((size_t)(row0 + t0 + tt) * n_heads + h) * vdim + col0 + c] = so[tt][c];
    }
  }
  if (quads) {
#pragma unroll
    for (int i = 0; i < DKL; i += 4) {
      const int r = rg * DKL + i;
      if (on && r < dim) *reinterpret_cast<float4*>(S + r) = make_float4(s[i], s[i + 1], s[i + 2], s[i + 3]);
    }
  } else {
#pragma unroll
    for (int i = 0; i < DKL; ++i) {
      const int r = rg * DKL + i;
      if (on && r < dim) S[r] = s[i];
    }
  }
}

template <int DKL, int RG, int CH, bool BONUS>
static void launch_delta_rule(const float* q, const float* k, size_t qk_stride, const float* v, size_t v_stride,
                              const float* g, size_t g_stride, const float* beta, float* state, const int32_t* cu_seqlens,
                              const int32_t* slots, float* out, int n_seqs, int n_heads, int n_kv, int dim, int vdim,
                              int g_per_head, const float* bonus, hipStream_t s) {
  constexpr int COLS = RB_WAVE / RG;
  static_assert((DKL * RG * CH) % RB_WAVE == 0 && CH <= RB_WAVE && DKL % 4 == 0, "a chunk's values are dealt evenly to the lanes");
  dim3 grid(n_seqs, n_heads, (vdim + COLS - 1) / COLS);
  delta_rule_kernel<DKL, RG, CH, BONUS><<<grid, RB_WAVE, 0, s>>>(q, k, qk_stride, v, v_stride, g, g_stride, beta, state, cu_seqlens,
                                                                 slots, out, n_heads, n_kv, dim, vdim, g_per_head, bonus);
}

extern "C" int rb_delta_rule(const float* q, const float* k, long long qk_stride, const float* v, long long v_stride,
                             const float* g, long long g_stride, const float* beta, float* state, const int32_t* cu_seqlens,
                             const int32_t* slots, float* out, int n_seqs, int n_tokens, int n_heads, int n_kv_heads, int dim,
                             int vdim, void* stream) {
  RB_RECORDED(rb_delta_rule(q, k, qk_stride, v, v_stride, g, g_stride, beta, state, cu_seqlens, slots, out, n_seqs, n_tokens,
                            n_heads, n_kv_heads, dim, vdim, stream));
  RB_REQUIRE(beta != nullptr, "rb_delta_rule: the delta rule needs beta");
  return rb_linear_recurrence(q, k, qk_stride, v, v_stride, g, g_stride, 0, beta, state, cu_seqlens, slots, out, n_seqs, n_tokens,
                              n_heads, n_kv_heads, dim, vdim, stream);
}

extern "C" int rb_linear_recurrence(const float* q, const float* k, long long qk_stride, const float* v, long long v_stride,
                                    const float* g, long long g_stride, int g_per_head, const float* beta, float* state,
                                    const int32_t* cu_seqlens, const int32_t* slots, float* out, int n_seqs, int n_tokens,
                                    int n_heads, int n_kv_heads, int dim, int vdim, void* stream) {
  RB_RECORDED(rb_linear_recurrence(q, k, qk_stride, v, v_stride, g, g_stride, g_per_head, beta, state, cu_seqlens, slots, out, n_seqs,
                                   n_tokens, n_heads, n_kv_heads, dim, vdim, stream));
  return rb_linear_recurrence_bonus(q, k, qk_stride, v, v_stride, g, g_stride, g_per_head, beta, nullptr, state, cu_seqlens, slots,
                                    out, n_seqs, n_tokens, n_heads, n_kv_heads, dim, vdim, stream);
}

// bonus (float32 [H, dim], null: rb_linear_recurrence): the plain rule read BEFORE the token's write, with the token's own
// k v^T weighted per key channel:  out = (S + diag(bonus) k v^T)^T q;  S <- diag(g) S + k v^T.  Goes without beta.
extern "C" int rb_linear_recurrence_bonus(const float* q, const float* k, long long qk_stride, const float* v, long long v_stride,
                                          const float* g, long long g_stride, int g_per_head, const float* beta,
                                          const float* bonus, float* state, const int32_t* cu_seqlens, const int32_t* slots,
                                          float* out, int n_seqs, int n_tokens, int n_heads, int n_kv_heads, int dim, int vdim,
                                          void* stream) {
  RB_RECORDED(rb_linear_recurrence_bonus(q, k, qk_stride, v, v_stride, g, g_stride, g_per_head, beta, bonus, state, cu_seqlens, slots,
                                         out, n_seqs, n_tokens, n_heads, n_kv_heads, dim, vdim, stream));
  RB_REQUIRE(bonus == nullptr || beta == nullptr, "rb_linear_recurrence: a bonus goes with the plain rule (no beta)");
  RB_REQUIRE(n_seqs >= 0 && n_heads > 0 && n_kv_heads > 0 && n_heads % n_kv_heads == 0 && dim > 0 && vdim > 0,
             "rb_linear_recurrence: bad sizes H=%d Hk=%d dim=%d vdim=%d", n_heads, n_kv_heads, dim, vdim);
  RB_REQUIRE(g_stride >= (long long)n_heads * (g_per_head ? 1 : dim), "rb_linear_recurrence: the decays' row stride is too short");
  RB_REQUIRE(dim <= 512, "rb_linear_recurrence: key size %d not supported (at most 512)", dim);
  RB_REQUIRE(n_heads <= 65535 && vdim <= 65535 * 4, "rb_linear_recurrence: too many heads or value channels");
  if (n_seqs == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  const size_t qs = (size_t)qk_stride, vs = (size_t)v_stride;
  // a step of one token per sequence (n_tokens == n_seqs) stages chunks of as few tokens as deal evenly to the lanes:
  // the machinery of a chunk of 16 would cost it several times its arithmetic
  const bool single = n_tokens <= n_seqs;
#define DR_GO(DKL, RG, CH)                                                                                                  \
  do {                                                                                                                      \
    constexpr int CH1 = (DKL * RG >= RB_WAVE) ? 1 : RB_WAVE / (DKL * RG);                                                   \
    if (single && bonus)                                                                                                    \
      launch_delta_rule<DKL, RG, CH1, true>(q, k, qs, v, vs, g, (size_t)g_stride, beta, state, cu_seqlens, slots, out,     \
                                            n_seqs, n_heads, n_kv_heads, dim, vdim, g_per_head, bonus, s);                  \
    else if (single)                                                                                                        \
      launch_delta_rule<DKL, RG, CH1, false>(q, k, qs, v, vs, g, (size_t)g_stride, beta, state, cu_seqlens, slots, out,    \
                                             n_seqs, n_heads, n_kv_heads, dim, vdim, g_per_head, bonus, s);                 \
    else if (bonus)                                                                                                         \
      launch_delta_rule<DKL, RG, CH, true>(q, k, qs, v, vs, g, (size_t)g_stride, beta, state, cu_seqlens, slots, out,      \
                                           n_seqs, n_heads, n_kv_heads, dim, vdim, g_per_head, bonus, s);                   \
    else                                                                                                                    \
      launch_delta_rule<DKL, RG, CH, false>(q, k, qs, v, vs, g, (size_t)g_stride, beta, state, cu_seqlens, slots, out,     \
                                            n_seqs, n_heads, n_kv_heads, dim, vdim, g_per_head, bonus, s);                  \
  } while (0)
  // Rows of a column over RG lanes, chunks as long as the registers that hold the next one allow.  A token's time is
  // its lane's share of the column, so while the waves do not fill the GPU's SIMDs a column goes to more lanes
  // (more and shorter waves); once they do, fewer lanes per column save the moves between them.
  const long long simds = 4LL * rb_compute_units();
  auto waves = [&](int rg) { return (long long)n_seqs * n_heads * ((vdim + RB_WAVE / rg - 1) / (RB_WAVE / rg)); };
  if (dim <= 16)
    DR_GO(4, 4, 16);
  else if (dim <= 32) {
    if (waves(4) >= simds) DR_GO(8, 4, 16);
    else DR_GO(4, 8, 16);
  } else if (dim <= 64) {
    if (waves(8) >= simds) DR_GO(8, 8, 16);
    else DR_GO(4, 16, 16);
  } else if (dim <= 128) {
    if (waves(8) >= simds) DR_GO(16, 8, 16);
    else DR_GO(8, 16, 16);
  } else if (dim <= 256)
    DR_GO(16, 16, 8);
  else
    DR_GO(32, 16, 4);
#undef DR_GO
  RB_LAUNCH_CHECK();
  return 0;
}

// ---------------------------------------------------------------- read-out norm with gate
// out[t, h, :] = o[t, h, :] / sqrt(mean(o^2) + eps) * weight * sigmoid(gate[t, h, :]); a wave per (token, head).
template <typename TO>
__global__ void gated_rmsnorm_kernel(const float* __restrict__ o, const float* __restrict__ weight,
                                     const float* __restrict__ gate, size_t gate_stride, float eps, TO* __restrict__ out,
                                     int n_heads, int vdim, long long n_pairs, int act, size_t weight_head_stride) {
  const long long pair = (long long)blockIdx.x * (blockDim.x / RB_WAVE) + threadIdx.x / RB_WAVE;
  if (pair >= n_pairs) return;
  const int lane = threadIdx.x & (RB_WAVE - 1);
  const size_t t = (size_t)(pair / n_heads);
  const int h = (int)(pair % n_heads);
  const float* p = o + (size_t)pair * vdim;
  const float* gp = gate + t * gate_stride + (size_t)h * vdim;
  const float* wp = weight + (size_t)h * weight_head_stride;
  float ss = 0.f;
  for (int i = lane; i < vdim; i += RB_WAVE) ss = fmaf(p[i], p[i], ss);
  ss = wave_sum(ss);
  const float f = 1.0f / sqrtf(ss / (float)vdim + eps);
  for (int i = lane; i < vdim; i += RB_WAVE)
    Num<TO>::store(out + (size_t)pair * vdim + i, p[i] * f * wp[i] * (act == 1 ? gp[i] * rb_sigmoid(gp[i]) : rb_sigmoid(gp[i])));
}

extern "C" int rb_gated_rmsnorm(const float* o, const float* weight, const float* gate, long long gate_stride, float eps,
                                void* out, int out_dtype, int n_tokens, int n_heads, int vdim, void* stream) {
  RB_RECORDED(rb_gated_rmsnorm(o, weight, gate, gate_stride, eps, out, out_dtype, n_tokens, n_heads, vdim, stream));
  return rb_gated_rmsnorm_act(o, weight, gate, gate_stride, 0, eps, out, out_dtype, n_tokens, n_heads, vdim, stream);
}

// act 0: the gate is sigmoid(gate); 1: silu(gate) = gate * sigmoid(gate)
extern "C" int rb_gated_rmsnorm_act(const float* o, const float* weight, const float* gate, long long gate_stride, int act, float eps,
                                    void* out, int out_dtype, int n_tokens, int n_heads, int vdim, void* stream) {
  RB_RECORDED(rb_gated_rmsnorm_act(o, weight, gate, gate_stride, act, eps, out, out_dtype, n_tokens, n_heads, vdim, stream));
  return rb_gated_rmsnorm_heads(o, weight, 0, gate, gate_stride, act, eps, out, out_dtype, n_tokens, n_heads, vdim, stream);
}

// The same with head h's weight at weight + h * weight_head_stride (0: one weight of vdim numbers for all heads; vdim: a
// weight over the concatenated heads).
extern "C" int rb_gated_rmsnorm_heads(const float* o, const float* weight, long long weight_head_stride, const float* gate,
                                      long long gate_stride, int act, float eps, void* out, int out_dtype, int n_tokens, int n_heads,
                                      int vdim, void* stream) {
  RB_RECORDED(rb_gated_rmsnorm_heads(o, weight, weight_head_stride, gate, gate_stride, act, eps, out, out_dtype, n_tokens, n_heads,
                                     vdim, stream));
  RB_REQUIRE(weight_head_stride >= 0, "rb_gated_rmsnorm: bad weight stride");
  RB_REQUIRE(n_tokens >= 0 && n_heads > 0 && vdim > 0 && (act == 0 || act == 1), "rb_gated_rmsnorm: bad sizes");
  RB_REQUIRE(gate_stride >= (long long)n_heads * vdim, "rb_gated_rmsnorm: the gate's row stride is too short");
  if (n_tokens == 0) return 0;
  const long long n_pairs = (long long)n_tokens * n_heads;
  const int grid = (int)((n_pairs + 3) / 4);
  hipStream_t s = (hipStream_t)stream;
  if (out_dtype == RB_F32)
    gated_rmsnorm_kernel<float><<<grid, 256, 0, s>>>(o, weight, gate, (size_t)gate_stride, eps, (float*)out, n_heads, vdim, n_pairs, act,
                                                     (size_t)weight_head_stride);
  else if (out_dtype == RB_BF16)
    gated_rmsnorm_kernel<bf16_t><<<grid, 256, 0, s>>>(o, weight, gate, (size_t)gate_stride, eps, (bf16_t*)out, n_heads, vdim, n_pairs, act,
                                                      (size_t)weight_head_stride);
  else
    RB_REQUIRE(false, "rb_gated_rmsnorm: unknown dtype %d", out_dtype);
  RB_LAUNCH_CHECK();
  return 0;
}
