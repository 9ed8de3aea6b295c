// A feed-forward of many small experts of which every token uses a few.
//
//   route:  scores s = sigmoid(z) of a token's router logits z [n_experts]; the `top` largest are chosen (among equals
//           the lowest index); pair p = t * top + k holds the k-th choice of token t: sel[p] its expert, weight[p] its score.
//   sort:   the pairs in the order of their experts, every expert's run padded to a multiple of 16 rows, so that a
//           tile of 16 rows belongs to one expert: row_pair[row] (-1: padding), tile_expert[row / 16] (-1: past the end),
//           and behind the experts of all tiles their positions in their experts' runs (0, 1, 2, ...).
//   up:     for every row, x = weight * h[token] (the weight multiplies the expert's INPUT), g = min(Wg x, limit),
//           u = clamp(Wu x, -limit, limit), y[row] = g * sigmoid(alpha * g) * (u + 1)
//   down:   out[pair] = Wd y[row]; a token's result is the sum of its pairs, in the order of k.
//
// Nothing goes through the host: the grid is made for the most rows there can be (pairs rounded up to 16, plus 16 for
// every expert), and tiles past the end leave at once.  A row's sums do not depend on which rows share its tile, so
// the result of a token is the same bits whatever else the step holds.
// bfloat16 with sizes that are multiples of 32 runs on the matrix cores (the experts' rows as the row operand, 16
// rows of the step as the columns, gate and up of the same 16 channels in one wave so that a lane holds both);
// float32, and other sizes, on the vector units with a wave per output.
#include <math.h>

#include "api.h"
#include "common.h"
#include "mfma.h"

#define RT_TILE 16
#define RT_MAX_EXPERTS 1024

// ---------------------------------------------------------------- route
// score 0: sigmoid(z) of the chosen logit.  score 1: the softmax of z over all outputs; the choice then goes by the
// softmax plus `correction` (null: nothing added), the weight is the softmax itself.
__global__ void route_kernel(const float* __restrict__ z, size_t z_stride, int n_experts, int top, int score,
                             const float* __restrict__ correction, int32_t* __restrict__ sel, float* __restrict__ weight,
                             int n_tokens) {
  const int t = blockIdx.x * (blockDim.x / RB_WAVE) + threadIdx.x / RB_WAVE;
  if (t >= n_tokens) return;
  const int lane = threadIdx.x & (RB_WAVE - 1);
  constexpr int PER = RT_MAX_EXPERTS / RB_WAVE;
  float v[PER];
#pragma unroll
  for (int j = 0; j < PER; ++j) {
    const int e = lane + RB_WAVE * j;
    v[j] = e < n_experts ? z[(size_t)t * z_stride + e] : -INFINITY;
    if (v[j] != v[j]) v[j] = -INFINITY;
  }
  float own[PER];                    // score 1: the softmax, kept beside what the choice goes by
  if (score == 1) {
    float m = -INFINITY;
#pragma unroll
    for (int j = 0; j < PER; ++j) m = fmaxf(m, v[j]);
    m = wave_max(m);
    float sum = 0.f;
#pragma unroll
    for (int j = 0; j < PER; ++j) {
      own[j] = v[j] == -INFINITY ? 0.f : expf(v[j] - m);
      sum += own[j];
    }
    sum = wave_sum(sum);
#pragma unroll
    for (int j = 0; j < PER; ++j) {
      const int e = lane + RB_WAVE * j;
      own[j] = own[j] / sum;
      if (e < n_experts) v[j] = own[j] + (correction ? correction[e] : 0.f);
      if (v[j] != v[j]) v[j] = -INFINITY;
    }
  }
  for (int k = 0; k < top; ++k) {
    float best = -INFINITY;
    int at = 0x7fffffff;
#pragma unroll
    for (int j = 0; j < PER; ++j) {
      const int e = lane + RB_WAVE * j;
      if (e < n_experts && (v[j] > best || (v[j] == best && e < at))) {
        best = v[j];
        at = e;
      }
    }
#pragma unroll
    for (int o = RB_WAVE / 2; o > 0; o >>= 1) {
      const float ob = __shfl_xor(best, o, RB_WAVE);
      const int oa = __shfl_xor(at, o, RB_WAVE);
      if (ob > best || (ob == best && oa < at)) {
        best = ob;
        at = oa;
      }
    }
    if (at == 0x7fffffff) at = k < n_experts ? k : 0;        // every logit was NaN or -inf: any expert, never out of range
    if (score == 1) {                   // the chosen output's softmax: from the lane that holds it
      float w = 0.f;
#pragma unroll
      for (int j = 0; j < PER; ++j)
        if (lane + RB_WAVE * j == at) w = own[j];
      best = wave_sum(w);
    } else {
      best = 1.0f / (1.0f + expf(-best));
    }
    if (lane == 0) {
      sel[(size_t)t * top + k] = at;
      weight[(size_t)t * top + k] = best;
    }
#pragma unroll
    for (int j = 0; j < PER; ++j)
      if (lane + RB_WAVE * j == at) v[j] = -INFINITY;
  }
}

// ---------------------------------------------------------------- sort (one workgroup)
__global__ __launch_bounds__(1024) void route_sort_kernel(const int32_t* __restrict__ sel, int n_pairs, int n_experts,
                                                          int32_t* __restrict__ row_pair, int32_t* __restrict__ tile_expert,
                                                          int32_t* __restrict__ tile_pos, int max_rows) {
  __shared__ int counts[RT_MAX_EXPERTS], offs[RT_MAX_EXPERTS], cursor[RT_MAX_EXPERTS];
  for (int e = threadIdx.x; e < n_experts; e += blockDim.x) counts[e] = cursor[e] = 0;
  __syncthreads();
  for (int p = threadIdx.x; p < n_pairs; p += blockDim.x)
    if (sel[p] < n_experts) atomicAdd(&counts[sel[p]], 1);      // an output behind the experts has no matrices and no run
  for (int r = threadIdx.x; r < max_rows; r += blockDim.x) row_pair[r] = -1;
  for (int i = threadIdx.x; i < max_rows / RT_TILE; i += blockDim.x) tile_expert[i] = -1;
  __syncthreads();
  if (threadIdx.x == 0) {
    int at = 0;
    for (int e = 0; e < n_experts; ++e) {
      offs[e] = at;
      at += (counts[e] + RT_TILE - 1) / RT_TILE * RT_TILE;
    }
  }
  __syncthreads();
  for (int e = threadIdx.x; e < n_experts; e += blockDim.x)
    for (int i = 0; i < (counts[e] + RT_TILE - 1) / RT_TILE; ++i) {
      tile_expert[offs[e] / RT_TILE + i] = e;
      tile_pos[offs[e] / RT_TILE + i] = i;                 // which tile of its expert's run
    }
  for (int p = threadIdx.x; p < n_pairs; p += blockDim.x) {
    const int e = sel[p];
    if (e < n_experts) row_pair[offs[e] + atomicAdd(&cursor[e], 1)] = p;
  }
}

extern "C" int rb_route_choose(const float* z, long long z_stride, int n_outputs, int n_experts, int top, int score,
                               const float* correction, int32_t* sel, float* weight, int32_t* row_pair, int32_t* tile_expert,
                               int max_rows, int n_tokens, void* stream) {
  RB_RECORDED(rb_route_choose(z, z_stride, n_outputs, n_experts, top, score, correction, sel, weight, row_pair, tile_expert, max_rows,
                              n_tokens, stream));
  RB_REQUIRE(n_tokens >= 0 && n_experts >= 0 && n_outputs >= n_experts && n_outputs > 0 && n_outputs <= RT_MAX_EXPERTS && top > 0 &&
                 top <= n_outputs && z_stride >= n_outputs,
             "rb_route_choose: bad sizes T=%d outputs=%d (at most %d) experts=%d top=%d", n_tokens, n_outputs, RT_MAX_EXPERTS, n_experts, top);
  RB_REQUIRE(score == 0 || score == 1, "rb_route_choose: score %d is neither the sigmoid (0) nor the softmax (1)", score);
  RB_REQUIRE(correction == nullptr || score == 1, "rb_route_choose: a correction goes with the softmax");
  const long long pairs = (long long)n_tokens * top;
  RB_REQUIRE(max_rows % RT_TILE == 0 && max_rows >= (pairs + RT_TILE - 1) / RT_TILE * RT_TILE + (long long)RT_TILE * n_experts,
             "rb_route_choose: room for %d rows, %lld pairs of %d experts may need more", max_rows, pairs, n_experts);
  if (n_tokens == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  route_kernel<<<(n_tokens + 3) / 4, 256, 0, s>>>(z, (size_t)z_stride, n_outputs, top, score, correction, sel, weight, n_tokens);
  route_sort_kernel<<<1, 1024, 0, s>>>(sel, (int)pairs, n_experts, row_pair, tile_expert, tile_expert + max_rows / RT_TILE, max_rows);
  RB_LAUNCH_CHECK();
  return 0;
}

extern "C" int rb_route_top(const float* z, long long z_stride, int n_experts, int top, int32_t* sel, float* weight,
                            int32_t* row_pair, int32_t* tile_expert, int max_rows, int n_tokens, void* stream) {
  return rb_route_choose(z, z_stride, n_experts, n_experts, top, 0, nullptr, sel, weight, row_pair, tile_expert, max_rows, n_tokens, stream);
}

// limit > 0: g = min(g, limit), u = clamp(u, +-limit), g sigmoid(alpha g) (u + 1).  limit <= 0: the plain gate silu(g) u.
__device__ __forceinline__ float gated_unit(float g, float u, float limit, float alpha) {
  if (!(limit > 0.f)) return g / (1.0f + expf(-g)) * u;
  g = fminf(g, limit);
  u = fminf(fmaxf(u, -limit), limit);
  return g / (1.0f + expf(-alpha * g)) * (u + 1.0f);
}

// ---------------------------------------------------------------- vector units: a wave per output
template <typename T>
__global__ void routed_up_generic_kernel(const T* __restrict__ h, const float* __restrict__ weight, int top,
                                         const int32_t* __restrict__ row_pair, const int32_t* __restrict__ tile_expert,
                                         const T* __restrict__ w_gate, const T* __restrict__ w_up, T* __restrict__ y, int width,
                                         int ff, float limit, float alpha) {
  const int e = tile_expert[blockIdx.x];
  if (e < 0) return;
  const int lane = threadIdx.x & (RB_WAVE - 1), wave = threadIdx.x / RB_WAVE, n_waves = blockDim.x / RB_WAVE;
  for (int i = 0; i < RT_TILE; ++i) {
    const int row = blockIdx.x * RT_TILE + i;
    const int p = row_pair[row];
    if (p < 0) continue;
    const T* x = h + (size_t)(p / top) * width;
    const float wt = weight ? weight[p] : 1.0f;
    for (int j = blockIdx.y * n_waves + wave; j < ff; j += gridDim.y * n_waves) {
      const T* gr = w_gate + ((size_t)e * ff + j) * width;
      const T* ur = w_up + ((size_t)e * ff + j) * width;
      float g = 0.f, u = 0.f;
      for (int k = lane; k < width; k += RB_WAVE) {
        const float xv = Num<T>::load(x + k) * wt;
        g = fmaf(Num<T>::load(gr + k), xv, g);
        u = fmaf(Num<T>::load(ur + k), xv, u);
      }
      g = wave_sum(g);
      u = wave_sum(u);
      if (lane == 0) Num<T>::store(y + (size_t)row * ff + j, gated_unit(g, u, limit, alpha));
    }
  }
}

template <typename T>
__global__ void routed_down_generic_kernel(const T* __restrict__ y, const int32_t* __restrict__ row_pair,
                                           const int32_t* __restrict__ tile_expert, const T* __restrict__ w_down,
                                           float* __restrict__ out, int width, int ff) {
  const int e = tile_expert[blockIdx.x];
  if (e < 0) return;
  const int lane = threadIdx.x & (RB_WAVE - 1), wave = threadIdx.x / RB_WAVE, n_waves = blockDim.x / RB_WAVE;
  for (int i = 0; i < RT_TILE; ++i) {
    const int row = blockIdx.x * RT_TILE + i;
    const int p = row_pair[row];
    if (p < 0) continue;
    const T* yr = y + (size_t)row * ff;
    for (int j = blockIdx.y * n_waves + wave; j < width; j += gridDim.y * n_waves) {
      const T* dr = w_down + ((size_t)e * width + j) * ff;
      float acc = 0.f;
      for (int k = lane; k < ff; k += RB_WAVE) acc = fmaf(Num<T>::load(dr + k), Num<T>::load(yr + k), acc);
      acc = wave_sum(acc);
      if (lane == 0) out[(size_t)p * width + j] = acc;
    }
  }
}

// ---------------------------------------------------------------- matrix cores (bfloat16, sizes that are multiples of 32)
// The matrix-core kernels read every operand fragment-major: blocks of 16 rows x 32 depth values (1 KB) in the order
// [rows / 16][depth / 32], inside a block the value of row r and depth d at 8 * (16 * (d / 8) + r) + d % 8, which is
// the 16 bytes of lane r + 16 (d / 8) of the matrix cores' operand.  A wave's load is then 1 KB in a row; with plain
// rows it touched 16 lines a fixed 2 * K bytes apart, and the kernels ran at a tenth of this speed.  The experts'
// matrices are stored so at load time; the step's rows are written so here, and the gated units by the kernel below.
// The rows of the step, scaled by their weights and rounded to bfloat16, in sorted order: xs[row] = bf16(weight h[token]).
__global__ void routed_gather_kernel(const bf16_t* __restrict__ h, const float* __restrict__ weight, int top,
                                     const int32_t* __restrict__ row_pair, bf16_t* __restrict__ xs, int width) {
  const int row = blockIdx.x;
  const int p = row_pair[row];
  if (p < 0) return;
  const float wt = weight ? weight[p] : 1.0f;
  const bf16_t* x = h + (size_t)(p / top) * width;
  bf16_t* dst = xs + (size_t)(row / RT_TILE) * RT_TILE * width + 8 * (row % RT_TILE);
  for (int k = 8 * threadIdx.x; k < width; k += 8 * blockDim.x) {
    const uint4 raw = load16(x + k);
    *reinterpret_cast<uint4*>(dst + (size_t)(k / 32) * 512 + 128 * ((k % 32) / 8)) =
        make_uint4(pack_bf16x2(bf16_bits_to_f32(raw.x & 0xffffu) * wt, bf16_bits_to_f32(raw.x >> 16) * wt),
                   pack_bf16x2(bf16_bits_to_f32(raw.y & 0xffffu) * wt, bf16_bits_to_f32(raw.y >> 16) * wt),
                   pack_bf16x2(bf16_bits_to_f32(raw.z & 0xffffu) * wt, bf16_bits_to_f32(raw.z >> 16) * wt),
                   pack_bf16x2(bf16_bits_to_f32(raw.w & 0xffffu) * wt, bf16_bits_to_f32(raw.w >> 16) * wt));
  }
}

// A workgroup of 8 waves takes up to RT_SPAN tiles of 16 rows that follow one another in an expert's run (the
// workgroup of the run's tiles 0, 16, 32, ... does the work, the others leave) and 64 channels.  Its waves are 4 x 2:
// a wave takes RT_GROUP of the tiles and 32 channels: the gate rows and the up rows of two blocks of 16 channels are
// its row operands, the tiles' rows the column operands, so that lane l holds gate and up of channels 4 (l / 16) + i
// of row l % 16.  A fragment of W serves four tiles in a wave, and the four waves that share it ask for it together, so
// that an expert's matrices come from memory once for every 256 rows.
#define RT_GROUP 4
#define RT_SPAN 16
#define RT_THREADS 512
__global__ __launch_bounds__(RT_THREADS) void routed_up_mfma_kernel(const bf16_t* __restrict__ xs, const int32_t* __restrict__ row_pair,
                                                             const int32_t* __restrict__ tile_expert,
                                                             const int32_t* __restrict__ tile_pos,
                                                             const bf16_t* __restrict__ w_gate, const bf16_t* __restrict__ w_up,
                                                             bf16_t* __restrict__ y, int width, int ff, float limit, float alpha,
                                                             int n_tiles) {
  // blockIdx.x counts the channels, so that workgroups that follow one another share their rows of the step (which
  // then come from memory once) and walk through an expert's matrices together
  const int e = tile_expert[blockIdx.y];
  if (e < 0 || (tile_pos[blockIdx.y] % RT_SPAN) != 0) return;
  const int lane = threadIdx.x & (RB_WAVE - 1), wave = threadIdx.x / RB_WAVE;
  const int t0 = blockIdx.y + (wave & 3) * RT_GROUP;          // this wave's first tile
  if (t0 >= n_tiles || tile_expert[t0] != e) return;
  int nt = 1;
  while (nt < RT_GROUP && t0 + nt < n_tiles && tile_expert[t0 + nt] == e) ++nt;
  const int c0 = (blockIdx.x * 2 + (wave >> 2)) * 32;
  if (c0 >= ff) return;
  const int r = lane & 15, grp = lane >> 4;
  const bf16_t* xr = xs + (size_t)t0 * RT_TILE * width + 8 * lane;
  const bf16_t* gr = w_gate + ((size_t)e * ff + c0) * width + 8 * lane;
  const bf16_t* ur = w_up + ((size_t)e * ff + c0) * width + 8 * lane;
  const size_t blk = (size_t)16 * width;               // 16 rows further: the next block of channels, the next tile
  f32x4_t ag[RT_GROUP][2], au[RT_GROUP][2];
#pragma unroll
  for (int j = 0; j < RT_GROUP; ++j)
#pragma unroll
    for (int cb = 0; cb < 2; ++cb) ag[j][cb] = au[j][cb] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  for (int k = 0; k < 16 * width; k += 512) {            // a block of 16 rows x 32 depth values further
    Frag8 fg[2], fu[2], fx[RT_GROUP];
#pragma unroll
    for (int cb = 0; cb < 2; ++cb) {
      fg[cb].u = load16(gr + cb * blk + k);
      fu[cb].u = load16(ur + cb * blk + k);
    }
#pragma unroll
    for (int j = 0; j < RT_GROUP; ++j) fx[j].u = j < nt ? load16(xr + j * blk + k) : zero16();
#pragma unroll
    for (int j = 0; j < RT_GROUP; ++j) {
      if (j < nt) {
#pragma unroll
        for (int cb = 0; cb < 2; ++cb) {
          ag[j][cb] = mfma16(fg[cb], fx[j], ag[j][cb]);
          au[j][cb] = mfma16(fu[cb], fx[j], au[j][cb]);
        }
      }
    }
  }
#pragma unroll
  for (int j = 0; j < RT_GROUP; ++j) {
    if (j >= nt) break;
    const int row = (t0 + j) * RT_TILE + r;
    if (row_pair[row] < 0) continue;
#pragma unroll
    for (int cb = 0; cb < 2; ++cb) {
      // channel c of this row lies, fragment-major, in block c / 32 of the tile at 8 * (16 * (c % 32 / 8) + r) + c % 8
      const int c = c0 + 16 * cb + 4 * grp;
      bf16_t* dst = y + (size_t)(t0 + j) * RT_TILE * ff + (size_t)(c / 32) * 512 + 8 * (16 * ((c % 32) / 8) + r) + c % 8;
      const f32x4_t g = ag[j][cb], u = au[j][cb];
      *reinterpret_cast<uint2*>(dst) = make_uint2(pack_bf16x2(gated_unit(g[0], u[0], limit, alpha), gated_unit(g[1], u[1], limit, alpha)),
                                                  pack_bf16x2(gated_unit(g[2], u[2], limit, alpha), gated_unit(g[3], u[3], limit, alpha)));
    }
  }
}

// The same for the way down: a wave takes 64 of the model's channels (four blocks of 16 rows of Wd), a workgroup 128.
__global__ __launch_bounds__(RT_THREADS) void routed_down_mfma_kernel(const bf16_t* __restrict__ y, const int32_t* __restrict__ row_pair,
                                                               const int32_t* __restrict__ tile_expert,
                                                               const int32_t* __restrict__ tile_pos,
                                                               const bf16_t* __restrict__ w_down, float* __restrict__ out, int width,
                                                               int ff, int n_tiles) {
  const int e = tile_expert[blockIdx.y];
  if (e < 0 || (tile_pos[blockIdx.y] % RT_SPAN) != 0) return;
  const int lane = threadIdx.x & (RB_WAVE - 1), wave = threadIdx.x / RB_WAVE;
  const int t0 = blockIdx.y + (wave & 3) * RT_GROUP;
  if (t0 >= n_tiles || tile_expert[t0] != e) return;
  int nt = 1;
  while (nt < RT_GROUP && t0 + nt < n_tiles && tile_expert[t0 + nt] == e) ++nt;
  const int c0 = (blockIdx.x * 2 + (wave >> 2)) * 64;
  if (c0 >= width) return;
  const int r = lane & 15, grp = lane >> 4;
  const int n_cb = (width - c0) / 16 < 4 ? (width - c0) / 16 : 4;      // width is a multiple of 32, not always of 64
  const bf16_t* yr = y + (size_t)t0 * RT_TILE * ff + 8 * lane;
  const bf16_t* dr = w_down + ((size_t)e * width + c0) * ff + 8 * lane;
  const size_t blk = (size_t)16 * ff;
  f32x4_t acc[RT_GROUP][4];
  int pair[RT_GROUP];                                    // this lane's row of every tile: its pair, -1 for none
#pragma unroll
  for (int j = 0; j < RT_GROUP; ++j) {
    pair[j] = j < nt ? row_pair[(t0 + j) * RT_TILE + r] : -1;
#pragma unroll
    for (int cb = 0; cb < 4; ++cb) acc[j][cb] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  }
  for (int k = 0; k < 16 * ff; k += 512) {
    Frag8 fd[4], fy[RT_GROUP];
#pragma unroll
    for (int cb = 0; cb < 4; ++cb) fd[cb].u = cb < n_cb ? load16(dr + cb * blk + k) : zero16();
#pragma unroll
    for (int j = 0; j < RT_GROUP; ++j) fy[j].u = pair[j] >= 0 ? load16(yr + j * blk + k) : zero16();
#pragma unroll
    for (int j = 0; j < RT_GROUP; ++j) {
      if (j < nt) {
#pragma unroll
        for (int cb = 0; cb < 4; ++cb) acc[j][cb] = mfma16(fd[cb], fy[j], acc[j][cb]);
      }
    }
  }
#pragma unroll
  for (int j = 0; j < RT_GROUP; ++j) {
    const int p = pair[j];
    if (p < 0) continue;
#pragma unroll
    for (int cb = 0; cb < 4; ++cb)
      if (cb < n_cb)
        *reinterpret_cast<float4*>(out + (size_t)p * width + c0 + 16 * cb + 4 * grp) =
            make_float4(acc[j][cb][0], acc[j][cb][1], acc[j][cb][2], acc[j][cb][3]);
  }
}

// h [T, width], weight [T * top], w_gate and w_up [experts, ff, width], w_down [experts, width, ff], all of dtype;
// y [max_rows, ff + width] of dtype is scratch; out [T * top, width] float32: the pairs' results.  tile_expert holds
// max_rows / 16 experts and then as many positions of the tiles in their experts' runs, as rb_route_top leaves them.
extern "C" int rb_routed_experts(const void* h, int dtype, const float* weight, int top, const int32_t* row_pair,
                                 const int32_t* tile_expert, int max_rows, const void* w_gate, const void* w_up, const void* w_down,
                                 int w_layout, void* y, float* out, int n_experts, int width, int ff, float limit, float alpha,
                                 void* stream) {
  RB_RECORDED(rb_routed_experts(h, dtype, weight, top, row_pair, tile_expert, max_rows, w_gate, w_up, w_down, w_layout, y, out,
                                n_experts, width, ff, limit, alpha, stream));
  RB_REQUIRE(w_layout == 0 || (w_layout == 1 && dtype == RB_BF16 && width % 32 == 0 && ff % 32 == 0),
             "rb_routed_experts: fragment-major experts are bfloat16 with sizes that are multiples of 32");
  RB_REQUIRE(max_rows >= 0 && max_rows % RT_TILE == 0 && n_experts > 0 && width > 0 && ff > 0 && top > 0,
             "rb_routed_experts: bad sizes rows=%d experts=%d width=%d ff=%d", max_rows, n_experts, width, ff);
  RB_REQUIRE(dtype == RB_F32 || dtype == RB_BF16, "rb_routed_experts: unknown dtype %d", dtype);
  RB_REQUIRE(max_rows / RT_TILE <= 65535, "rb_routed_experts: %d rows are more than one launch takes (at most %d)", max_rows, 65535 * RT_TILE);
  if (max_rows == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  const int tiles = max_rows / RT_TILE;
  auto aligned = [](const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; };
  if (w_layout == 1) {
    RB_REQUIRE(aligned(h) && aligned(w_gate) && aligned(w_up) && aligned(w_down) && aligned(y) && aligned(out),
               "rb_routed_experts: the matrix-core kernels need 16-byte aligned operands");
    bf16_t* xs = (bf16_t*)y + (size_t)max_rows * ff;
    const int threads = width / 8 >= 256 ? 256 : 64;
    routed_gather_kernel<<<max_rows, threads, 0, s>>>((const bf16_t*)h, weight, top, row_pair, xs, width);
    routed_up_mfma_kernel<<<dim3((ff + 63) / 64, tiles), RT_THREADS, 0, s>>>(xs, row_pair, tile_expert, tile_expert + tiles,
                                                                        (const bf16_t*)w_gate, (const bf16_t*)w_up, (bf16_t*)y, width,
                                                                        ff, limit, alpha, tiles);
    routed_down_mfma_kernel<<<dim3((width + 127) / 128, tiles), RT_THREADS, 0, s>>>((const bf16_t*)y, row_pair, tile_expert,
                                                                             tile_expert + tiles, (const bf16_t*)w_down, out, width,
                                                                             ff, tiles);
  } else if (dtype == RB_BF16) {
    routed_up_generic_kernel<bf16_t><<<dim3(tiles, (ff + 3) / 4 < 64 ? (ff + 3) / 4 : 64), 256, 0, s>>>(
        (const bf16_t*)h, weight, top, row_pair, tile_expert, (const bf16_t*)w_gate, (const bf16_t*)w_up, (bf16_t*)y, width, ff, limit,
        alpha);
    routed_down_generic_kernel<bf16_t><<<dim3(tiles, (width + 3) / 4 < 64 ? (width + 3) / 4 : 64), 256, 0, s>>>(
        (const bf16_t*)y, row_pair, tile_expert, (const bf16_t*)w_down, out, width, ff);
  } else {
    routed_up_generic_kernel<float><<<dim3(tiles, (ff + 3) / 4 < 64 ? (ff + 3) / 4 : 64), 256, 0, s>>>(
        (const float*)h, weight, top, row_pair, tile_expert, (const float*)w_gate, (const float*)w_up, (float*)y, width, ff, limit, alpha);
    routed_down_generic_kernel<float><<<dim3(tiles, (width + 3) / 4 < 64 ? (width + 3) / 4 : 64), 256, 0, s>>>(
        (const float*)y, row_pair, tile_expert, (const float*)w_down, out, width, ff);
  }
  RB_LAUNCH_CHECK();
  return 0;
}

// out[t, :] = sum_k pairs[t * top + k, :], in the order of k.
__global__ void pairs_sum_kernel(const float* __restrict__ pairs, int top, float* __restrict__ out, int width, size_t n) {
  for (size_t e = (size_t)blockIdx.x * blockDim.x + threadIdx.x; e < n; e += (size_t)gridDim.x * blockDim.x) {
    const size_t t = e / width, j = e - t * width;
    float v = pairs[(t * top) * width + j];
    for (int k = 1; k < top; ++k) v += pairs[(t * top + k) * width + j];
    out[e] = v;
  }
}

extern "C" int rb_pairs_sum(const float* pairs, int top, float* out, int n_tokens, int width, void* stream) {
  RB_RECORDED(rb_pairs_sum(pairs, top, out, n_tokens, width, stream));
  RB_REQUIRE(n_tokens >= 0 && width > 0 && top > 0, "rb_pairs_sum: bad sizes");
  if (n_tokens == 0) return 0;
  const size_t n = (size_t)n_tokens * width;
  const size_t blocks = (n + 255) / 256;
  pairs_sum_kernel<<<(int)(blocks < 65535 ? blocks : 65535), 256, 0, (hipStream_t)stream>>>(pairs, top, out, width, n);
  RB_LAUNCH_CHECK();
  return 0;
}

// out[t] = sum over k of weight[p] * (sel[p] < n_experts ? pairs[p] : h[t]), p = t * top + k, in the order of k: the score
// multiplies the expert's OUTPUT, and an output of the router behind the experts stands for the token's own input.
// With `shared` (float32 [T, width], what an expert that every token uses gave): + sigmoid(gate[t * gate_stride]) * shared[t].
template <typename T>
__global__ void experts_combine_kernel(const float* __restrict__ pairs, const int32_t* __restrict__ sel, const float* __restrict__ weight,
                                       int top, int n_experts, const T* __restrict__ h, const float* __restrict__ shared,
                                       const float* __restrict__ gate, size_t gate_stride, float* __restrict__ out, int width) {
  const int t = blockIdx.x;
  const float sg = shared ? 1.0f / (1.0f + expf(-gate[(size_t)t * gate_stride])) : 0.f;
  for (int j = threadIdx.x; j < width; j += blockDim.x) {
    float v = 0.f;
    for (int k = 0; k < top; ++k) {
      const size_t p = (size_t)t * top + k;
      const float term = sel[p] < n_experts ? pairs[p * width + j] : Num<T>::load(h + (size_t)t * width + j);
      v = fmaf(weight[p], term, v);
    }
    if (shared) v = fmaf(sg, shared[(size_t)t * width + j], v);
    out[(size_t)t * width + j] = v;
  }
}

extern "C" int rb_experts_combine(const float* pairs, const int32_t* sel, const float* weight, int top, int n_experts, const void* h,
                                  int h_dtype, const float* shared, const float* gate, long long gate_stride, float* out, int n_tokens,
                                  int width, void* stream) {
  RB_RECORDED(rb_experts_combine(pairs, sel, weight, top, n_experts, h, h_dtype, shared, gate, gate_stride, out, n_tokens, width, stream));
  RB_REQUIRE(n_tokens >= 0 && width > 0 && top > 0 && n_experts >= 0, "rb_experts_combine: bad sizes");
  RB_REQUIRE(shared == nullptr || gate != nullptr, "rb_experts_combine: a shared expert comes with its gate");
  if (n_tokens == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  const int threads = width >= 256 ? 256 : 64;
  if (h_dtype == RB_F32)
    experts_combine_kernel<float><<<n_tokens, threads, 0, s>>>(pairs, sel, weight, top, n_experts, (const float*)h, shared, gate,
                                                               (size_t)gate_stride, out, width);
  else if (h_dtype == RB_BF16)
    experts_combine_kernel<bf16_t><<<n_tokens, threads, 0, s>>>(pairs, sel, weight, top, n_experts, (const bf16_t*)h, shared, gate,
                                                                (size_t)gate_stride, out, width);
  else
    RB_REQUIRE(false, "rb_experts_combine: unknown dtype %d", h_dtype);
  RB_LAUNCH_CHECK();
  return 0;
}
