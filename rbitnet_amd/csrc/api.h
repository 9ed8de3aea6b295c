// C entry points of librbitnet_hip.so.  All pointers are device pointers unless a
// name starts with h_.  Every function returns 0 on success; otherwise
// rb_last_error() holds the reason.  `stream` is a hipStream_t.
//
// dtype codes: 0 = float32, 1 = bfloat16 (storage; arithmetic is float32 inside).
#pragma once
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

const char* rb_last_error(void);
int rb_version(void);
int rb_page_size(void);

// x[t, :] = table[ids[t], :] widened to float32.  ids are checked by the caller.
int rb_embed_gather(const void* table, int table_dtype, const int32_t* ids, float* x, int n_tokens, int width,
                    void* stream);

// Residual add and RMS norm in one pass.
//   src = rows ? rows[r] : r
//   v = x[src] + (delta ? delta[src] : 0);  if (delta && !rows) x[src] = v
//   out[r] = v * gain * rsqrt(mean(v^2) + eps)
// delta may be n_terms terms, each laid out like x and term_stride floats after the one before:
// they are added up first, in their order (rb_gemm_bf16_terms leaves such terms).
int rb_add_rmsnorm(float* x, const float* delta, int n_terms, long long term_stride, const float* gain, float eps,
                   const int32_t* rows, int n_rows, int width, void* out, int out_dtype, void* stream);

// Rotate q and k by the angle table, write q to q_out and k, v into the cache pages.
//   qkv      float32 [T, (Hq + 2 Hk) D]: q heads, then k heads, then v heads; as qkv_terms terms
//            to be added up in their order, qkv_term_stride floats apart (1 term: qkv itself)
//   cos, sin float32 [max_pos, D/2], or null for no rotation
//   style    0: pairs (2i, 2i+1); 1: pairs (i, i + D/2)
//   k_pages, v_pages [n_pages, Hk, 64, D] of cache_dtype; null when the layer keeps no cache
//   tok_pos, tok_seq int32 [T]; block_table int32 [B, bt_stride]
int rb_rope_kv_write(const float* qkv, int qkv_terms, long long qkv_term_stride, const float* cos, const float* sin,
                     int style, void* q_out, void* k_pages, void* v_pages, int cache_dtype, const int32_t* tok_pos, const int32_t* tok_seq,
                     const int32_t* block_table, int bt_stride, int n_tokens, int n_heads, int n_kv_heads,
                     int head_dim, void* stream);

// t[r, j] = silu(gu[r, j]) * gu[r, F + j]
int rb_swiglu(const float* gu, void* out, int out_dtype, int n_rows, int ff, void* stream);

// C[M, N] = A[M, K] * W[N, K]^T with float32 accumulation; any sizes.
// w_layout 0: W is N rows of K values.  1 (float32 with N % 16 == 0 and K % 128 == 0 only): fragment-major, blocks
// of 16 rows x 16 depth values, 1 KB each, in the order [N / 16][K / 16]; inside a block the value of row r and
// depth d lies at 4 * (16 * (d / 4) + r) + d % 4.  rb_place_rows writes either layout.
int rb_gemm_generic(const void* a, const void* w, int w_layout, void* c, int dtype_in, int dtype_out, int m, int n,
                    int k, void* stream);

// C[M, N] = A[M, K] * W[N, K]^T, bfloat16 inputs on the matrix cores.
//   epilogue 0: store C (float32 or bfloat16)
//   epilogue 1: W holds gate and up rows interleaved in blocks of 16
//               (16 gate rows, then the 16 up rows of the same columns); the result is
//               silu(gate) * up, [M, N/2]
// K must be a multiple of 8 (rows 16-byte aligned).
// rb_gemm_bf16_act with epilogue 1 and act = two numbers (limit, alpha), limit > 0: the gated pair with limits,
// g = min(gate, limit), u = clamp(up, -limit, limit), result g * sigmoid(alpha g) * (u + 1).
// w_layout says how W is stored.  0: N rows of K values.  1: fragment-major (K % 64 == 0 and
// N % 16 == 0 only): blocks of 16 rows x 32 depth values, 1 KB each, in the order [N / 16][K / 32];
// inside a block, the value of row r and depth d lies at 8 * (16 * (d / 8) + r) + d % 8.  A wave
// then reads 1 KB in a row per load, and a product of few tokens streams W with non-temporal
// loads: 6.0-6.8 TB/s instead of 5.3-5.8.  rb_place_rows writes either layout.
// workspace: rb_gemm_workspace_floats(m, n, k, epilogue) floats (0: none, null allowed); contents do
// not matter before or after.
long long rb_gemm_workspace_floats(int m, int n, int k, int epilogue);
int rb_gemm_bf16(const void* a, const void* w, int w_layout, void* c, int dtype_out, int epilogue, int m, int n, int k,
                 float* workspace, void* stream);

// rb_gemm_bf16 with an activation on the way out (epilogue 0 only): act holds xIELU's two numbers (p, q), and
// C = xIELU(A W^T) with xIELU(z) = softplus(p) z^2 + z/2 for z > 0, (1/2 + softplus(q)) (exp(z) - 1 - z) + z/2 otherwise,
// applied to the float32 sums before they are stored.  act null: rb_gemm_bf16.  An act[0] that is no number (NaN) asks for
// the tanh form of GELU instead, z / 2 (1 + tanh(sqrt(2 / pi) (z + 0.044715 z^3))), which has no numbers of its own.
int rb_gemm_bf16_act(const void* a, const void* w, int w_layout, void* c, int dtype_out, int epilogue, const float* act,
                     int m, int n, int k, float* workspace, void* stream);

// The plain product (float32, epilogue 0) as the terms that the K slices of its kernel computed:
// terms [rb_gemm_bf16_terms_count(m, n, k), M, N], to be added up in their order.  One term is
// the product itself.  For a caller that adds them to something else anyway.
int rb_gemm_bf16_terms_count(int m, int n, int k);
int rb_gemm_bf16_terms(const void* a, const void* w, int w_layout, float* terms, int m, int n, int k, void* stream);

// The same product for 1..16 tokens with what stands before and after it in a decode step folded
// in, so that no kernel runs between the products.  rb_gemm_bf16_few_ok: whether it takes these
// sizes (few tokens, and no tiled kernel would).
//   a: bfloat16 rows of K values; row i of the product is row rows[i] (row i without rows).
//   squares_in (may be null): float32 [*, ceil(K / 16)], rows as in a.  Then a holds float32 rows
//     times a norm's gain and squares_in their sums of squares over every 16 columns, and the
//     product is multiplied by 1 / sqrt(sum of them / K + eps): the RMS norm's factor.
//   epilogue 0, 1: as above.  2: C (float32) += product.  3: as 2, and for the norm that follows
//     gained [M, N] = bf16(C * gain), squares_out [M, ceil(N / 16)] = sums of C^2 over 16 columns.
int rb_gemm_bf16_few_ok(int m, int n, int k);
int rb_gemm_bf16_few(const void* a, const float* squares_in, float eps, const int32_t* rows, const void* w,
                     int w_layout, void* c, int dtype_out, int epilogue, const float* gain, void* gained,
                     float* squares_out, int m, int n, int k, void* stream);

// Causal attention of every token over its sequence's cache (keys 0..pos, or the last
// `window` of them), any head_dim up to 512 (a rotation in front of it needs an even one).
//   q [T, Hq, D], out [T, Hq * D], both of dtype; pages as in rb_rope_kv_write.
int rb_attention_generic(const void* q, const void* k_pages, const void* v_pages, void* out, int dtype,
                         const int32_t* tok_pos, const int32_t* tok_seq, const int32_t* block_table,
                         int bt_stride, int n_tokens, int n_heads, int n_kv_heads, int head_dim, float scale,
                         int window, void* stream);

// The same for bfloat16 and head_dim 64 or 128 on the matrix cores.
//   prefill: sequences b = 0..B-1 hold tokens cu_seqlens[b]..cu_seqlens[b+1] at positions past_len[b]...
int rb_attention_prefill_bf16(const void* q, const void* k_pages, const void* v_pages, void* out,
                              const int32_t* cu_seqlens, const int32_t* past_len, const int32_t* block_table,
                              int bt_stride, int n_seqs, int max_q_len, int n_heads, int n_kv_heads, int head_dim,
                              float scale, int window, void* stream);
//   decode: one token per sequence at position tok_pos[b]; the keys are split into
//   n_splits ranges whose partial results are combined in a second kernel.
//   workspace: float32 [B, Hq, n_splits, D + 2]
int rb_attention_decode_bf16(const void* q, const void* k_pages, const void* v_pages, void* out,
                             const int32_t* tok_pos, const int32_t* block_table, int bt_stride, int n_seqs,
                             int n_heads, int n_kv_heads, int head_dim, float scale, int window, int n_splits,
                             float* workspace, void* stream);

//   decode, fused: rotation of q and the new k, cache write and attention in one kernel (plus the
//   combination of the splits when there are several).  qkv float32 [B, (Hq + 2 Hk) D] as for
//   rb_rope_kv_write.
int rb_attention_decode_fused_bf16(const float* qkv, int qkv_terms, long long qkv_term_stride, const float* cos,
                                   const float* sin, int style, void* k_pages, void* v_pages, void* out,
                                   const int32_t* tok_pos, const int32_t* block_table,
                                   int bt_stride, int n_seqs, int n_heads, int n_kv_heads, int head_dim, float scale,
                                   int window, int n_splits, float* workspace, void* stream);

// rb_attention_generic with a sink per query head (sinks float32 [Hq], null: none): the softmax's denominator also
// holds exp(sink), a score that is not scaled and has no key and no value.  v_pages may be k_pages (attention over
// cached latents, which are keys and values at once).
int rb_attention_generic_sinks(const void* q, const void* k_pages, const void* v_pages, void* out, int dtype,
                               const int32_t* tok_pos, const int32_t* tok_seq, const int32_t* block_table,
                               int bt_stride, int n_tokens, int n_heads, int n_kv_heads, int head_dim, float scale,
                               int window, const float* sinks, void* stream);

// The matrix-core kernels with sinks as above (float32 [Hq] or null); v_pages may be k_pages.
int rb_attention_prefill_bf16_sinks(const void* q, const void* k_pages, const void* v_pages, void* out,
                                    const int32_t* cu_seqlens, const int32_t* past_len, const int32_t* block_table,
                                    int bt_stride, int n_seqs, int max_q_len, int n_heads, int n_kv_heads, int head_dim,
                                    float scale, int window, const float* sinks, void* stream);
int rb_attention_decode_bf16_sinks(const void* q, const void* k_pages, const void* v_pages, void* out,
                                   const int32_t* tok_pos, const int32_t* block_table, int bt_stride, int n_seqs,
                                   int n_heads, int n_kv_heads, int head_dim, float scale, int window, int n_splits,
                                   float* workspace, const float* sinks, void* stream);
int rb_attention_decode_fused_bf16_sinks(const float* qkv, int qkv_terms, long long qkv_term_stride, const float* cos,
                                         const float* sin, int style, void* k_pages, void* v_pages, void* out,
                                         const int32_t* tok_pos, const int32_t* block_table, int bt_stride, int n_seqs,
                                         int n_heads, int n_kv_heads, int head_dim, float scale, int window, int n_splits,
                                         float* workspace, const float* sinks, void* stream);

// ---- a residual stream in several copies, layer norm, xIELU, the cap of logits (streams.hip)
// x [S, T, E] float32, stream_stride floats from one copy to the next.
//   rb_embed_streams:     x[s][t, :] = table[ids[t], :] for every copy
//   rb_streams_layernorm: u = sum_s coef[s] x[s][src] (+ delta[src]), src = rows ? rows[r] : r;
//                         out[r] = (u - mean) / sqrt(var + eps) * weight + bias (variance: mean of squared deviations).
//                         coef null: all 1; bias null: none; one stream with a delta and no rows: x = u as well.
//   rb_streams_update:    x'[j] = sum_s mix[s * S + j] x[s] + out_coef[j] * (scale ? scale[e] : 1) * y, all copies at once
int rb_embed_streams(const void* table, int table_dtype, const int32_t* ids, float* x, int n_streams, long long stream_stride,
                     int n_tokens, int width, void* stream);
int rb_streams_layernorm(float* x, int n_streams, long long stream_stride, const float* coef, const float* delta,
                         const float* weight, const float* bias, float eps, const int32_t* rows, int n_rows, int width,
                         void* out, int out_dtype, void* stream);
int rb_streams_update_layernorm(float* x, int n_streams, long long stream_stride, const float* mix, const float* out_coef,
                                const float* y, const float* scale, const float* coef, const float* delta, const float* weight,
                                const float* bias, float eps, const int32_t* rows, int n_rows, int width, void* out,
                                int out_dtype, void* stream);      // rb_streams_update (mix null: none), then the norm, in one pass
int rb_streams_update(float* x, int n_streams, long long stream_stride, const float* mix, const float* out_coef, const float* y,
                      const float* scale, int n_tokens, int width, void* stream);
// out = z > 0 ? softplus(act[0]) z^2 + z/2 : (1/2 + softplus(act[1])) (exp(z) - 1 - z) + z/2; act[0] NaN: the tanh form of GELU
int rb_xielu(const float* z, const float* act, void* out, int out_dtype, long long n, void* stream);
// x <- cap * tanh(x / cap)
int rb_tanh_cap(float* x, float cap, long long n, void* stream);

// ---- layers with a fixed-size state per sequence (recurrent.hip)
// Causal convolution over time per channel: y[t, c] = (residual ? x[t, c] : 0) + sum_d w[c, taps-1-d] x[t-d, c], act 1: silu.
// x float32 rows x_stride apart; rows before the step come from state [slots, taps-1, C] (the sequence's last taps-1
// inputs, oldest first; zero for a fresh slot), which the same launch then moves on by the step's rows.
int rb_short_conv(const float* x, long long x_stride, const float* w, int taps, float* state, const int32_t* tok_pos,
                  const int32_t* tok_seq, const int32_t* cu_seqlens, const int32_t* slots, void* out, long long out_stride,
                  int out_dtype, int residual, int act, int n_tokens, int n_seqs, int channels, void* stream);
// What enters the gated delta rule, in place: qk [T, qk_stride] holds Hk q heads, then Hk k heads, of `dim` numbers;
// each becomes x / sqrt(sum x^2 + unit_eps), q times q_scale.  a [T, H, dim] (rows a_stride apart) becomes the decay
// exp(-exp(a_log[h]) softplus(a + dt_bias)); beta [T, H] = sigmoid(b_in[t * b_stride + h]).
int rb_delta_prep(float* qk, long long qk_stride, int n_kv_heads, int dim, float* a, long long a_stride, const float* dt_bias, const float* a_log,
                  int n_heads, const float* b_in, long long b_stride, float* beta, float q_scale, float unit_eps, int n_tokens,
                  void* stream);
// Per sequence b (rows cu_seqlens[b]..) and head h, token after token on the state S, kept column by column as
// [slots, H, vdim, dim]:
//   S <- diag(g) S;  u = beta (v - S^T k);  S <- S + k u^T;  out[t, h, :] = S^T q      (head h reads q/k head h / (H / Hk))
int rb_delta_rule(const float* q, const float* k, long long qk_stride, const float* v, long long v_stride, const float* g,
                  long long g_stride, const float* beta, float* state, const int32_t* cu_seqlens, const int32_t* slots, float* out, int n_seqs,
                  int n_tokens, int n_heads, int n_kv_heads, int dim, int vdim, void* stream);
// out[t, h, :] = o / sqrt(mean(o^2) + eps) * weight[vdim] * sigmoid(gate[t * gate_stride + h * vdim + :])
int rb_gated_rmsnorm(const float* o, const float* weight, const float* gate, long long gate_stride, float eps, void* out,
                     int out_dtype, int n_tokens, int n_heads, int vdim, void* stream);

// rb_delta_prep with its choices spelled out.  unit 1: q and k heads become unit vectors (q times q_scale); 0: q is
// only multiplied by q_scale.  The a_cols numbers of a row of `a` (a_cols = H: one decay per head; H * dim: one per head
// and key channel) become decays in place: decay 0: exp(-exp(a_log[head]) softplus(a + bias[i])); decay 1:
// sigmoid(a + bias[i]) ^ (1 / tau).  bias may be null.  b_in null: no beta.
int rb_recurrence_prep(float* qk, long long qk_stride, int n_kv_heads, int dim, int unit, float q_scale, float unit_eps, float* a,
                       long long a_stride, int a_cols, int decay, const float* bias, const float* a_log, float tau, int n_heads,
                       const float* b_in, long long b_stride, float* beta, int n_tokens, void* stream);
// rb_delta_rule with one decay per head (g_per_head 1: g[t * g_stride + h]) or per key channel (0), and, with beta null,
// the plain rule without the correction:  S <- diag(g) S + k v^T;  out = S^T q.
int rb_linear_recurrence(const float* q, const float* k, long long qk_stride, const float* v, long long v_stride, const float* g,
                         long long g_stride, int g_per_head, const float* beta, float* state, const int32_t* cu_seqlens,
                         const int32_t* slots, float* out, int n_seqs, int n_tokens, int n_heads, int n_kv_heads, int dim, int vdim,
                         void* stream);
// rb_gated_rmsnorm with the gate's activation: act 0 sigmoid(gate), 1 silu(gate).
int rb_gated_rmsnorm_act(const float* o, const float* weight, const float* gate, long long gate_stride, int act, float eps, void* out,
                         int out_dtype, int n_tokens, int n_heads, int vdim, void* stream);

// ---- a plain stream with layer norm (streams.hip)
// v = x[src] + dscale * (delta[src] + (delta2 ? delta2[src] : 0)), src = rows ? rows[r] : r; without rows x[src] = v too;
// out[r] = (v - mean) / sqrt(var + eps) * weight + bias.  delta null: the norm alone.
int rb_layernorm_residual(float* x, const float* delta, const float* delta2, float dscale, const float* weight, const float* bias,
                          float eps, const int32_t* rows, int n_rows, int width, void* out, int out_dtype, void* stream);

// ---- around the mixers (mixers.hip)
// rb_rope_kv_write for heads whose keys and values differ in size and of which only the first `rot` numbers are rotated
// (i paired with i + rot / 2; cos, sin [positions, rot / 2]).  A row of qkv (row_width floats apart) holds Hq and Hk
// heads of `dim` and Hk heads of `vdim`; q_out [T, Hq, pad] and the pages [*, Hk, 64, pad] get them padded with zeros.
int rb_rope_store(const float* qkv, long long row_width, const float* cos, const float* sin, int rot, void* q_out, void* k_pages,
                  void* v_pages, int cache_dtype, const int32_t* tok_pos, const int32_t* tok_seq, const int32_t* block_table,
                  int bt_stride, int n_tokens, int n_heads, int n_kv_heads, int dim, int vdim, int pad, void* stream);
// x[t, h, :] *= sigmoid(gate[t * gate_stride + h]); x [T, H, D] of dtype, in place.
int rb_head_gate(void* x, int dtype, const float* gate, long long gate_stride, int n_tokens, int n_heads, int head_dim, void* stream);
// out = (rmsnorm(a) * wa + rmsnorm(b) * wb) / 2 over rows of `width` float32 numbers.
int rb_pair_norm_mean(const float* a, const float* wa, const float* b, const float* wb, float eps, float* out, int n_tokens,
                      int width, void* stream);

// ---- a feed-forward of routed experts (routed.hip)
// Router logits z [T, z_stride >= experts] -> the `top` experts with the largest sigmoid(z) per token (lowest index among
// equals): sel, weight [T * top] (pair p = t * top + k), and the pairs sorted by expert in runs padded to 16 rows:
// row_pair [max_rows] (-1: padding), tile_expert [2 * max_rows / 16]: the tiles' experts (-1: past the end), then the
// tiles' positions in their experts' runs.  max_rows: a multiple of 16, at least T * top rounded up to 16, plus 16
// for every expert.
int rb_route_top(const float* z, long long z_stride, int n_experts, int top, int32_t* sel, float* weight, int32_t* row_pair,
                 int32_t* tile_expert, int max_rows, int n_tokens, void* stream);
// For every pair p of token t: x = weight[p] h[t]; g = min(Wg x, limit), u = clamp(Wu x, -limit, limit);
// out[p] = Wd (g sigmoid(alpha g) (u + 1)), the expert being the pair's.  w_gate, w_up [experts, ff, width] and w_down
// [experts, width, ff] of dtype; y [max_rows, ff + width] of dtype is scratch; out [T * top, width] float32.
// w_layout 0: every expert's matrices as rows.  1 (bfloat16, width and ff multiples of 32): every expert's matrices
// fragment-major, as rb_place_rows writes them; then the matrix cores run.
int rb_routed_experts(const void* h, int dtype, const float* weight, int top, const int32_t* row_pair, const int32_t* tile_expert,
                      int max_rows, const void* w_gate, const void* w_up, const void* w_down, int w_layout, void* y, float* out,
                      int n_experts, int width, int ff, float limit, float alpha, void* stream);
// rb_route_top with its choices spelled out.  The router has n_outputs outputs, of which the first n_experts are experts
// with matrices; a pair whose output lies behind them belongs to no run (rb_experts_combine gives it the token's input).
// score 0: weight = sigmoid(z) of the chosen, chosen by z.  score 1: weight = softmax(z) over all outputs, chosen by
// softmax + correction (float32 [n_outputs], null: nothing added).
int rb_route_choose(const float* z, long long z_stride, int n_outputs, int n_experts, int top, int score, const float* correction,
                    int32_t* sel, float* weight, int32_t* row_pair, int32_t* tile_expert, int max_rows, int n_tokens, void* stream);
// rb_routed_experts takes weight null (the input is not scaled) and limit <= 0 (no clamps, the plain gate:
// out[p] = Wd (silu(Wg x) * (Wu x))).
// out[t] = sum over k of weight[p] * (sel[p] < n_experts ? pairs[p] : h[t]), p = t * top + k, in the order of k; with
// shared (float32 [T, width]) also + sigmoid(gate[t * gate_stride]) * shared[t].  h of h_dtype [T, width].
int rb_experts_combine(const float* pairs, const int32_t* sel, const float* weight, int top, int n_experts, const void* h,
                       int h_dtype, const float* shared, const float* gate, long long gate_stride, float* out, int n_tokens,
                       int width, void* stream);
// out[t] = sum over k of pairs[t * top + k], in the order of k.
int rb_pairs_sum(const float* pairs, int top, float* out, int n_tokens, int width, void* stream);

// ---- attention whose heads' scores are mixed before the softmax, and what stands around it (talking.hip)
// x[t, :] = table[ids[t], :] * scale + positions[tok_pos[t], :] (positions of the table's dtype, null: none), float32.
int rb_embed_scaled_pos(const void* table, int table_dtype, const int32_t* ids, float scale, const void* positions,
                        const int32_t* tok_pos, float* x, int n_tokens, int width, void* stream);
// x <- s x
int rb_scale(float* x, float s, long long n, void* stream);
// rb_rope_store without a rotation, with a bias (float32, laid out like a row of qkv; null: none) added first and, norm != 0,
// every query and key head divided by sqrt(mean(head^2) + eps).  k_pages null: the row holds query heads only.
int rb_bias_norm_store(const float* qkv, long long row_width, const float* bias, int norm, float eps, void* q_out, void* k_pages,
                       void* v_pages, int cache_dtype, const int32_t* tok_pos, const int32_t* tok_seq, const int32_t* block_table,
                       int bt_stride, int n_tokens, int n_heads, int n_kv_heads, int dim, int vdim, int pad, void* stream);
// Causal attention with all heads of a token in one workgroup: score[g, j] = q_g . k_j * scale, mixed[h, j] = sum_g
// talk[h * Hq + g] score[g, j] (talk float32 [Hq, Hq], null: no mixing), softmax over the keys j <= pos that lie in the
// token's chunk (chunk > 0: pos / chunk == j / chunk) and among the last `window` (window > 0).  Layouts as
// rb_attention_generic; Hq <= 64, Hq * head_dim <= 8192.
int rb_attention_mixed(const void* q, const void* k_pages, const void* v_pages, void* out, int dtype, const int32_t* tok_pos,
                       const int32_t* tok_seq, const int32_t* block_table, int bt_stride, int n_tokens, int n_heads,
                       int n_kv_heads, int head_dim, float scale, const float* talk, int chunk, int window, void* stream);
// The same on the matrix cores: bfloat16, head_dim 64 or 128, Hq <= 32, talk not null.  The step's sequences as
// rb_attention_prefill_bf16 takes them (cu_seqlens [B + 1], past_len [B]); steps of single tokens and of prompts alike.
// n_splits > 1 deals every sequence's pages out to that many workgroups (for steps of few tokens with long contexts) and
// needs a workspace of n_splits * T * Hq * (head_dim + 2) floats.
int rb_attention_mixed_bf16(const void* q, const void* k_pages, const void* v_pages, void* out, const int32_t* cu_seqlens,
                            const int32_t* past_len, const int32_t* block_table, int bt_stride, int n_seqs, int n_tokens,
                            int n_heads, int n_kv_heads, int head_dim, float scale, const float* talk, int chunk, int window,
                            int n_splits, float* workspace, void* stream);

// ---- attention through a latent (latent.hip)
// Per token: cq = rmsnorm(proj[t, 0:q_rank]) * q_gain -> cq [T, q_rank]; rmsnorm(proj[t, kv_col:+kv_rank]) * kv_gain ->
// the token's place in pages [n_pages, 1, 64, kv_rank].  A rank of 0 leaves that half out.
int rb_latent_norm_store(const float* proj, long long stride, int q_rank, const float* q_gain, void* cq, int kv_col,
                         int kv_rank, const float* kv_gain, void* pages, int dtype, const int32_t* tok_pos,
                         const int32_t* tok_seq, const int32_t* block_table, int bt_stride, float eps, int n_tokens,
                         void* stream);
// y[t, h, n] = sum_k w[h, k, n] x[t, h, k]
int rb_heads_linear(const void* x, int x_dtype, const void* w, int w_dtype, void* y, int y_dtype, int n_tokens, int n_heads,
                    int n, int k, void* stream);

// ---- a norm on the sublayer's output, limits in the gated unit, and what the mixers of such layers need
// x <- (assign ? 0 : x) + y / sqrt(mean(y^2) + eps) * gain with y = sa * a + sb * b (b null: sa * a), rows of `width` float32
// numbers; h_out (null: none) gets the new rows of x in h_dtype.
int rb_outnorm_residual(float* x, const float* a, const float* b, float sa, float sb, const float* gain, float eps, int assign,
                        void* h_out, int h_dtype, int n_tokens, int width, void* stream);
// g = min(gu[r, j], limit), u = clamp(gu[r, F + j], -limit, limit); out[r, j] = g sigmoid(alpha g) (u + 1).  limit <= 0: none.
int rb_clamped_glu(const float* gu, void* out, int out_dtype, int n_rows, int ff, float limit, float alpha, void* stream);
// out = tanh(z), n numbers.
int rb_tanh_cast(const float* z, void* out, int out_dtype, long long n, void* stream);
// rb_attention_generic_sinks with kept first keys behind the window (j < keep_first stays visible) and capped scores
// (softcap > 0: s <- softcap tanh(s / softcap) after the scale).
int rb_attention_generic_opts(const void* q, const void* k_pages, const void* v_pages, void* out, int dtype,
                              const int32_t* tok_pos, const int32_t* tok_seq, const int32_t* block_table, int bt_stride,
                              int n_tokens, int n_heads, int n_kv_heads, int head_dim, float scale, int window, int keep_first,
                              float softcap, const float* sinks, void* stream);
// The matrix-core kernels with the same two choices (see rb_attention_prefill_bf16_sinks, rb_attention_decode_bf16_sinks).
// The decode entry point also takes more than 16 query heads on a key/value head: they run as the fewest groups of equal
// size that hold at most 16 each, every group reading that head's pages.
int rb_attention_prefill_bf16_opts(const void* q, const void* k_pages, const void* v_pages, void* out,
                                   const int32_t* cu_seqlens, const int32_t* past_len, const int32_t* block_table,
                                   int bt_stride, int n_seqs, int max_q_len, int n_heads, int n_kv_heads, int head_dim,
                                   float scale, int window, int keep_first, float softcap, const float* sinks, void* stream);
int rb_attention_decode_bf16_opts(const void* q, const void* k_pages, const void* v_pages, void* out,
                                  const int32_t* tok_pos, const int32_t* block_table, int bt_stride, int n_seqs,
                                  int n_heads, int n_kv_heads, int head_dim, float scale, int window, int keep_first,
                                  float softcap, int n_splits, float* workspace, const float* sinks, void* stream);
// rb_rope_store with every query and key head RMS-normed first over its dim numbers, x / sqrt(mean(x^2) + eps) * w, with a
// weight of dim numbers that the heads share (q_norm, k_norm float32 [dim]).
int rb_norm_rope_store(const float* qkv, long long row_width, const float* cos, const float* sin, int rot, const float* q_norm,
                       const float* k_norm, float eps, void* q_out, void* k_pages, void* v_pages, int cache_dtype,
                       const int32_t* tok_pos, const int32_t* tok_seq, const int32_t* block_table, int bt_stride, int n_tokens,
                       int n_heads, int n_kv_heads, int dim, int vdim, int pad, void* stream);
// x[e] *= sigmoid(gate[e]) for n numbers, x of dtype, gate float32, laid out alike.
int rb_sigmoid_gate(void* x, int dtype, const float* gate, long long n, void* stream);
// out[m, t, :] = h[t] + (h[t - 1] - h[t]) * mu[m] for m < n_mix (mu float32 [n_mix, E]); the row before a step's first
// comes from state [slots, E] (float32), which then holds the step's last row.  h and out [n_mix, T, E] of dtype.
int rb_shift_mix(const void* h, int dtype, float* state, const float* mu, int n_mix, void* out, const int32_t* cu_seqlens,
                 const int32_t* tok_seq, const int32_t* slots, int n_tokens, int n_seqs, int width, void* stream);
// rb_short_conv on x + bias (float32 [C], null: none); the state holds the inputs with their bias.
int rb_short_conv_bias(const float* x, long long x_stride, const float* bias, const float* w, int taps, float* state,
                       const int32_t* tok_pos, const int32_t* tok_seq, const int32_t* cu_seqlens, const int32_t* slots, void* out,
                       long long out_stride, int out_dtype, int residual, int act, int n_tokens, int n_seqs, int channels,
                       void* stream);
// rb_recurrence_prep takes decay 2 as well: exp(-exp(a + bias[i])).
// rb_linear_recurrence read before the token's write, with a weight per head and key channel on the token's own k v^T
// (bonus float32 [H, dim]; null: rb_linear_recurrence):  out = (S + diag(bonus) k v^T)^T q;  S <- diag(g) S + k v^T.
int rb_linear_recurrence_bonus(const float* q, const float* k, long long qk_stride, const float* v, long long v_stride,
                               const float* g, long long g_stride, int g_per_head, const float* beta, const float* bonus,
                               float* state, const int32_t* cu_seqlens, const int32_t* slots, float* out, int n_seqs, int n_tokens,
                               int n_heads, int n_kv_heads, int dim, int vdim, void* stream);
// rb_gated_rmsnorm_act with head h's weight at weight + h * weight_head_stride (0: one weight for all heads).
int rb_gated_rmsnorm_heads(const float* o, const float* weight, long long weight_head_stride, const float* gate,
                           long long gate_stride, int act, float eps, void* out, int out_dtype, int n_tokens, int n_heads, int vdim,
                           void* stream);
// rb_heads_linear on a part of every head: a head of x takes x_head_stride numbers (the first k are read), a head of y
// y_head_stride (the first n are written).
int rb_heads_linear_strided(const void* x, int x_dtype, long long x_head_stride, const void* w, int w_dtype, void* y, int y_dtype,
                            long long y_head_stride, int n_tokens, int n_heads, int n, int k, void* stream);
// rb_heads_linear_strided with two things in the same launch: a gate per head on the outputs (gate float32, rows gate_stride
// apart, null: none: head h of token t times sigmoid(gate[t * gate_stride + h])), and (rot >= 0) the `rot` numbers at x_rot_col
// of every head of x rotated by the token's position into y at y_rot_col >= n, with zeros behind them up to y_head_stride.
int rb_heads_linear_more(const void* x, int x_dtype, long long x_head_stride, const void* w, int w_dtype, void* y, int y_dtype,
                         long long y_head_stride, int n_tokens, int n_heads, int n, int k, const float* gate, long long gate_stride,
                         int rot, int x_rot_col, int y_rot_col, const float* cos, const float* sin, int style,
                         const int32_t* tok_pos, void* stream);
// rb_latent_norm_store into pages [n_pages, 1, 64, page_width] with, behind the latent, the `rot` numbers at rot_col of the
// row rotated by the token's position (style 0: 2i with 2i + 1; 1: i with i + rot / 2) and zeros up to page_width.
int rb_latent_norm_rope_store(const float* proj, long long stride, int q_rank, const float* q_gain, void* cq, int kv_col,
                              int kv_rank, const float* kv_gain, void* pages, int page_width, int rot_col, int rot, const float* cos,
                              const float* sin, int style, int dtype, const int32_t* tok_pos, const int32_t* tok_seq,
                              const int32_t* block_table, int bt_stride, float eps, int n_tokens, void* stream);
// tokens[r] = argmax of logits[r, :] (NaN counts as -inf, lowest index among equals), or, where
// temperature[r] > 0, the first index whose running sum of exp(z/T - max) reaches u[r] times the total.
// workspace: rb_sample_workspace_bytes(n_rows, vocab) bytes, 8-byte aligned, contents do not matter.
int rb_sample_workspace_bytes(int n_rows, int vocab);
int rb_sample(const float* logits, int n_rows, int vocab, const float* temperature, const float* u,
              int32_t* tokens, void* workspace, void* stream);

// rb_sample for callers that cannot allocate device memory: code under HIP graph capture, tight
// serving loops, harnesses that forbid hipMalloc.  It has no counterpart in the reference.  The
// same kernels and the same result as rb_sample, but the chunk statistics go into device memory
// that the library holds itself (256 KiB on every GPU it runs on, until the process ends), so no
// workspace is passed and neither this call nor anything under it allocates or frees.
// Limit: n_rows * ceil(vocab / 4096) <= rb_sample_static_max_stats() (16384: 512 rows of a
// 128k vocabulary); more is refused with an error and nothing is launched.  The stream must belong
// to the current device.  All calls on one GPU share that memory: two calls whose kernels may
// overlap there (different streams, no dependency between them) race; calls on one stream do not.
// The first use on a device asks the runtime for the address of that device's copy; before the
// first call under stream capture, call rb_sample_static_max_stats() (or rb_sample_static once) on
// that device outside of any capture.
int rb_sample_static_max_stats(void);
int rb_sample_static(const float* logits, int n_rows, int vocab, const float* temperature, const float* u,
                     int32_t* tokens, void* stream);

// Load-time helpers (weights_init.hip).
// rb_fill_normal: out[i] = mean + std * z_i for i < n, z_i the standard normal number that (key, i)
// fixes; the same bits as weights/random_init.py draws on the host.
int rb_fill_normal(void* out, int dtype, long long n, unsigned long long key, double mean, double std, void* stream);
// rb_place_rows: row r of src [n_rows, width] goes, cast to dst's dtype, to row
// row0 + (r / block) * period + r % block of dst [dst_rows, width].  block = n_rows places the rows
// one after another from row0 (q, k, v in one matrix); block 16, period 32, row0 0 and 16 interleave
// gate and up rows in blocks of 16.
// dst_layout 1: dst is fragment-major for its type (bfloat16: see rb_gemm_bf16, dst_rows % 16 == 0, width % 32 == 0;
// float32: see rb_gemm_generic, dst_rows % 16 == 0, width % 16 == 0).
int rb_place_rows(const void* src, int src_dtype, void* dst, int dst_dtype, int dst_layout, long long n_rows,
                  long long width, long long dst_rows, long long row0, long long block, long long period, void* stream);

// What the GPU reaches, measured the simplest way: rb_probe_read reads `bytes` bytes (a multiple of
// 16) once with 16-byte loads from `blocks` workgroups of 256 lanes (mode 0: all workgroups stride
// through the buffer together, plain loads; mode 1: every workgroup walks pieces of 64 KB of its own
// with non-temporal loads, which is a quarter faster on this GPU); rb_probe_mfma runs 4 * iters bfloat16 32x32x16 MFMAs in each of `waves`
// waves (a multiple of 4).  `sink` is one float of device memory that is practically never written.
int rb_probe_read(const void* p, long long bytes, int blocks, int mode, float* sink, void* stream);
int rb_probe_mfma(int waves, int iters, float* sink, void* stream);

#ifdef __cplusplus
}
#endif
