/*
 * aphrodite_mi355x_mixers.h -- C ABI of libaphrodite_mi355x_mixers.so
 *
 * MI355X (gfx950 / CDNA4) kernels of the sequence mixers that are not plain rotary softmax attention: layer norm around
 * an fp32 residual stream, gated activations, softmax attention over a paged cache with a tabulated distance bias and a
 * position-dependent query temperature, gated outer-product memories (decay linear attention, mLSTM) with their state
 * in per-request slots, and -- further down -- an fp32 residual stream averaged over depth with scalar-gain RMS norms, a
 * polynomial-norm activation, short causal convolutions with per-request state, (differential) attention under a sliding
 * window that keeps the first tokens, and routed experts on unquantised weights.  Same conventions as aphrodite_mi355x.h: device pointers, sizes and a hipStream_t (void*); every
 * entry point is asynchronous on `stream`, allocates nothing, never synchronises and returns APHRO_OK or a negative code;
 * aphro_mixers_last_error() describes the failure (thread-local).
 *
 * `dtype` is the storage of activations and weights: APHRO_BF16 or APHRO_F32.  Whatever the dtype, statistics, softmax,
 * gates, decays and memory states are fp32.  Row strides are in ELEMENTS.
 *
 * A batch is a list of `num_seqs` segments of consecutive rows: segment s owns rows q_start[s] .. q_start[s]+q_len[s]-1,
 * its first row is position ctx_len[s] of its sequence (ctx_len tokens were processed by earlier steps).
 */
#ifndef APHRODITE_MI355X_MIXERS_H_
#define APHRODITE_MI355X_MIXERS_H_

#include <stddef.h>
#include <stdint.h>

#include "aphrodite_mi355x.h"

#ifdef __cplusplus
extern "C" {
#endif

const char* aphro_mixers_last_error(void);

/* residual[t, :] = table[ids[t], :] * scale   (fp32 residual [T, width]; table [vocab, width] of `dtype`) */
int aphro_embed_scale_f32(float* residual, const void* table, const int64_t* ids, int64_t num_tokens, int width,
                          int64_t vocab, float scale, int dtype, void* stream);

/* One launch around an fp32 residual stream r [T, width], every step optional (NULL pointers switch it off):
 *   1. r += layer_norm(y + y_bias; post_w, post_b)      y [T, width] of `dtype` (row stride y_stride), y_bias fp32 [width]
 *   2. r += add_vec                                      add_vec [width] of `dtype`
 *   3. out = layer_norm(r; pre_w, pre_b)                 out [T, width] of `dtype`, contiguous
 * layer_norm(x; w, b) = (x - mean) / sqrt(mean((x - mean)^2) + eps) * w + b.  r is written back when 1 or 2 ran. */
int aphro_residual_layer_norm(float* residual, const void* y, int64_t y_stride, const float* y_bias, const void* post_w,
                              const void* post_b, const void* add_vec, const void* pre_w, const void* pre_b, void* out,
                              int64_t num_tokens, int width, float eps, int dtype, void* stream);

/* out[t, j] = act(in[t, j]) * in[t, d + j], j < d.  act: 0 silu, 1 gelu (tanh form).  in [T, 2 d] (row stride in_stride),
 * out [T, d] contiguous; math in fp32, one rounding. */
int aphro_act_and_mul(void* out, const void* in, int64_t in_stride, int64_t num_tokens, int d, int act, int dtype,
                      void* stream);

/* out[t, n] = out_scale * x[t, n] / rms(group of n) * weight[n] * sigmoid(gate[t, n]);  x fp32 [T, N] contiguous, groups of
 * `group` consecutive columns (N % group == 0), rms = sqrt(mean(x^2) + eps); weight [N] (NULL: ones) and gate [T, N]
 * (row stride gate_stride, NULL: no gate) of `dtype`; out of `dtype`, row stride out_stride. */
int aphro_gated_group_rms_norm(void* out, int64_t out_stride, const float* x, const void* weight, const void* gate,
                               int64_t gate_stride, int64_t num_tokens, int n, int group, float eps, float out_scale,
                               int dtype, void* stream);

/* Token-major paged cache write: k_cache [blocks, block_size, kv_heads, dim], v_cache [.., vdim] of `dtype`;
 * k [T, kv_heads * dim], v [T, kv_heads * vdim] (row strides); slots int64 [T] (block * block_size + offset, < 0: skip). */
int aphro_paged_kv_write(void* k_cache, void* v_cache, const void* k, int64_t k_stride, const void* v, int64_t v_stride,
                         const int64_t* slots, int64_t num_tokens, int kv_heads, int dim, int vdim, int64_t num_slots,
                         int dtype, void* stream);

/* Causal softmax attention of a batch of segments over the paged cache (which already holds the segments' own keys):
 *   score(i, j) = temp(i) * scale * q_i . k_j + bias_lut[h, min(i - j, lut_len - 1)]
 *   temp(i) = 1 + temp_coef * ln(floor((i + 1) / temp_every) + 1)         (temp_coef == 0: none)
 *   out[t, h, :] = out_scale * sigmoid(gate[t, h]) * sum_j softmax_j(score) v_j     (gate NULL: no gate)
 * q [T, heads * dim] (row stride), gate [T, heads] (row stride) and out [T, heads * vdim] (row stride) of `dtype`;
 * bias_lut fp32 [heads, lut_len] (NULL: no bias); block_tables int32 [num_seqs, max_blocks]; seq_of_token int32 [T].
 * Query head h reads key/value head h / (heads / kv_heads).  q_len int32 [num_seqs] with its host-side minimum and
 * maximum choose the kernels: bf16 segments of 8 rows or more run on the matrix cores (dim, vdim in {32, 64, 96, 128}),
 * shorter ones on a kernel that reads each key once for all query heads of its kv head (dim, vdim multiples of 8, at most
 * 256, 1 / 2 / 4 / 8 query heads per kv head); every other case -- and fp32 -- runs the scalar fp32 kernel.
 * max_kv_len (host-side longest ctx_len + q_len) and an optional fp32 workspace let the shared-key kernel split long key
 * ranges over up to 8 workgroups per row (num_tokens * heads * splits * (2 + vdim) floats; NULL: no split). */
int aphro_distance_bias_attention(void* out, int64_t out_stride, const void* q, int64_t q_stride, const void* gate,
                                  int64_t gate_stride, const void* k_cache, const void* v_cache, const int32_t* block_tables,
                                  int max_blocks, int64_t num_blocks, int block_size, const int32_t* q_start,
                                  const int32_t* q_len, const int32_t* ctx_len, const int32_t* seq_of_token,
                                  int64_t num_tokens, int num_seqs, int min_q_len, int max_q_len, int heads, int kv_heads,
                                  int dim, int vdim, float scale, const float* bias_lut, int lut_len, float temp_coef,
                                  int temp_every, float out_scale, int max_kv_len, float* workspace,
                                  int64_t workspace_floats, int dtype, void* stream);

/* Gated outer-product memory, one state per (slot, head):  S <- a_t S + b_t k_t v_t^T,  o_t = S^T q_t  [/ normaliser].
 *   mode 0 (decay linear attention): q, k, v = silu(raw); a_t = decay[h], b_t = 1.
 *   mode 1 (mLSTM): q = raw * q_scale; log gates i = cap tanh(raw_i / cap), f = logsigmoid(cap tanh(raw_f / cap));
 *     m_t = max(f + m_(t-1), i), a_t = exp(f + m_(t-1) - m_t), b_t = exp(i - m_t); n <- a_t n + b_t k_t;
 *     o_t = S^T q_t / (max(|n . q_t|, exp(-m_t)) + 1e-6).  m, n and S start at zero.
 * q, k [T, heads * dim], v [T, heads * vdim], gates [T, heads] (row strides) of `dtype`; out fp32 [T, heads * vdim].
 * state_s fp32 [slots, heads, dim, vdim]; mode 1 only: state_n fp32 [slots, heads, tiles, dim] and state_m fp32
 * [slots, heads, tiles], tiles = ceil(vdim / 16) (every 16 value columns keep their own copy of n and m, so no workgroup
 * reads what another one writes, whichever of the two work splits -- chosen by max_q_len, the host-side longest segment --
 * a launch uses).  slot_of_seq int32 [num_seqs]; a segment with ctx_len == 0 starts from zero
 * without reading its slot. */
int aphro_outer_memory_scan(float* out, const void* q, int64_t q_stride, const void* k, int64_t k_stride, const void* v,
                            int64_t v_stride, const void* gate_i, const void* gate_f, int64_t gate_stride, float* state_s,
                            float* state_n, float* state_m, const int32_t* slot_of_seq, int num_slots,
                            const int32_t* q_start, const int32_t* q_len, const int32_t* ctx_len, int num_seqs,
                            int64_t num_tokens, int heads, int dim, int vdim, int mode, const float* decay, float q_scale,
                            float gate_cap, int max_q_len, int dtype, void* stream);

/* ---- an fp32 residual stream joined over depth, scalar-gain RMS norm ---------------------------------------------------
 * One launch, every step optional:
 *   1. r = x_in + y                                       y [T, width] of `dtype` (row stride y_stride), NULL: r = x_in
 *   2. history[n_hist] = r;  r = sum_{j <= n_hist} depth_w[j] * history[j]        (depth_w NULL: skipped)
 *      history fp32 [.., T, width] with hist_stride elements between entries, depth_w fp32 [n_hist + 1]
 *   3. x_out = r                                          fp32 [T, width], may be x_in; NULL: not written
 *   4. out = r / sqrt(mean(r^2) + eps) * gain * weight    out [T, width] of `dtype`; weight [width] of `dtype` or NULL (ones) */
int aphro_depth_residual_rms_norm(const float* x_in, float* x_out, const void* y, int64_t y_stride, float* history,
                                  int64_t hist_stride, int n_hist, const float* depth_w, float gain, const void* weight,
                                  void* out, int64_t num_tokens, int width, float eps, int dtype, void* stream);

/* out[t, :] = a N(z) + b N(z^2) + c N(z^3) + e, powers element by element, N(v) = v / sqrt(mean(v^2) + eps) over the row.
 * z [T, n] (row stride z_stride), out [T, n] contiguous, both of `dtype`; fp32 math, one rounding. */
int aphro_poly_norm(void* out, const void* z, int64_t z_stride, int64_t num_tokens, int n, float a, float b, float c, float e,
                    float eps, int dtype, void* stream);

/* Joins the maps of a head: a fp32 [T, heads * maps * vdim] (head by head, map after map; maps 1 or 2),
 *   o = a_1 - lambda * a_2  (maps == 1: o = a_1);  out = out_scale * o / sqrt(mean(o^2) + eps) * sigmoid(gate)
 * with the mean over the head's vdim values; gate [T, heads * vdim] of `dtype` (NULL: none); out of `dtype`. */
int aphro_differential_norm_gate(void* out, int64_t out_stride, const float* a, int64_t a_stride, const void* gate,
                                 int64_t gate_stride, int64_t num_tokens, int heads, int maps, int vdim, float lambda,
                                 float out_scale, float eps, int dtype, void* stream);

/* Short causal convolution over time on each channel of u [T, cq + ck + cv] (row stride u_stride):
 *   y_t[c] = sum_j w[c, j] * u_(t - taps + 1 + j)[c],  zeros before the sequence's start;  w [channels, taps] of `dtype`.
 * Channels [0, cq) go to q_out [T, cq] (row stride); [cq, cq + ck) and the last cv go into the token-major paged caches
 * k_cache [cache slots, ck] / v_cache [cache slots, cv] at row cache_slots[t] (int64; outside 0 .. num_cache_slots - 1: skipped).
 * ck == cv == 0: no cache.  state [state slots, taps - 1, channels] of `dtype` holds each request's last taps - 1 inputs:
 * read for the rows before a segment (never for positions before the sequence's start), rewritten afterwards.
 * 1 <= taps <= 16.  act: 0 none, 1 silu on the convolution's result. */
int aphro_short_conv(void* q_out, int64_t q_out_stride, void* k_cache, void* v_cache, const int64_t* cache_slots,
                     int64_t num_cache_slots, const void* u, int64_t u_stride, const void* w, void* state,
                     const int32_t* state_slots, const int32_t* q_start, const int32_t* q_len, const int32_t* ctx_len,
                     const int32_t* seq_of_token, int64_t num_tokens, int num_seqs, int cq, int ck, int cv, int taps, int act,
                     int dtype, void* stream);

/* Softmax attention under a sliding window that keeps the first tokens: row i sees key j if j <= i and
 * (i - j < window or j < keep_first); window <= 0: every earlier key.  No rotation, no bias.  A head carries `maps`
 * attentions of their own over the same values: q [T, heads * maps * dim], k_cache [blocks, block_size, kv_heads * maps, dim],
 * v_cache [blocks, block_size, kv_heads, vdim] of `dtype`; out fp32 [T, heads * maps * vdim], every map's normalised output.
 * Segments as for aphro_distance_bias_attention.  bf16 with dim, vdim in {32, 64, 96, 128}: segments of 8 rows or more run on
 * the matrix cores, shorter ones on the shared-key kernel (workspace as there); everything else on the fp32-math kernel. */
int aphro_windowed_attention(float* out, int64_t out_stride, const void* q, int64_t q_stride, const void* k_cache,
                             const void* v_cache, const int32_t* block_tables, int max_blocks, int64_t num_blocks,
                             int block_size, const int32_t* q_start, const int32_t* q_len, const int32_t* ctx_len,
                             const int32_t* seq_of_token, int64_t num_tokens, int num_seqs, int min_q_len, int max_q_len,
                             int heads, int kv_heads, int maps, int dim, int vdim, float scale, int window, int keep_first,
                             int max_kv_len, float* workspace, int64_t workspace_floats, int dtype, void* stream);

/* Differential attention under the same window in one launch (bf16; dim, vdim in {32, 64, 96, 128}): the two maps of every head
 * (q [T, heads * 2 * dim], k_cache [.., kv_heads * 2, dim], head by head as [map 1, map 2]) over the shared values,
 *   o = a_1 - lambda * a_2;  out = out_scale * o / sqrt(mean(o^2) + eps) * sigmoid(gate)      (mean over the head's vdim values)
 * out and gate [T, heads * vdim] of `dtype` (gate NULL: none); at most 16 query heads per kv head.  Segments of 8 rows or more
 * run on the prompt kernel, shorter ones on the decode kernel (a kv head's query heads side by side), which splits long key ranges over up to 8 workgroups per row when max_kv_len (host-side longest
 * ctx_len + q_len) and an fp32 workspace of num_tokens * heads * 2 * splits * (2 + vdim) floats are given (NULL: no split).
 * aphro_differential_window_attention_supported says whether the sizes are served; what is not goes
 * through aphro_windowed_attention and aphro_differential_norm_gate. */
int aphro_differential_window_attention_supported(int heads, int kv_heads, int dim, int vdim, int dtype);
int aphro_differential_window_attention(void* out, int64_t out_stride, const void* q, int64_t q_stride, const void* gate,
                                        int64_t gate_stride, const void* k_cache, const void* v_cache, const int32_t* block_tables,
                                        int max_blocks, int64_t num_blocks, int block_size, const int32_t* q_start,
                                        const int32_t* q_len, const int32_t* ctx_len, const int32_t* seq_of_token,
                                        int64_t num_tokens, int num_seqs, int min_q_len, int max_q_len, int heads, int kv_heads,
                                        int dim, int vdim, float scale, int window, int keep_first, float lambda, float out_scale,
                                        float eps, int max_kv_len, float* workspace, int64_t workspace_floats, int dtype,
                                        void* stream);

/* ---- mixture of experts on unquantised weights ---------------------------------------------------------------------------
 * A SLOT is one (token, choice): slot = token * top + choice.
 * moe_route: router_out fp32 [T, outputs] -> ids int32 [T, top], weights fp32 [T, top]: s = softmax(router_out); the top
 *   values of s + correction (fp32 [outputs], NULL: none; ties to the lower index) are chosen, weights are their s. */
int aphro_experts_route(int32_t* ids, float* weights, const float* router_out, const float* correction, int64_t num_tokens,
                    int outputs, int top, void* stream);
/* rows per block of a step of num_slots slots over `experts` experts: 16, or 64 / 128 where an expert has hundreds of rows */
int aphro_experts_block_rows(int64_t num_slots, int experts);
/* rows of sorted_slots that such a step can need (a multiple of the block) */
int64_t aphro_experts_align_capacity(int64_t num_slots, int experts);
/* Sorts the slots whose id is below `experts` by expert into blocks (one expert per block, -1 pads a block):
 * sorted_slots int32 [capacity], block_expert int32 [capacity / block rows], num_blocks int32 [1].  Other ids are left out. */
int aphro_experts_align(int32_t* sorted_slots, int64_t capacity, int32_t* block_expert, int32_t* num_blocks, const int32_t* ids,
                    int64_t num_slots, int experts, void* stream);
/* y[row, :] of `dtype` [capacity, ff], row = place in sorted_slots: g = min(W_gate h, limit), u = clamp(W_up h, +-limit),
 * y = g * sigmoid(alpha * g) * (u + 1) with the block's expert; w_gate_up [experts, 2 * ff, width] (gate rows, then up rows);
 * h [T, width] (row stride), the slot's token is slot / top.  Rows of padding are zero. */
int aphro_experts_glu_gemm(void* y, const void* h, int64_t h_stride, const void* w_gate_up, const int32_t* sorted_slots,
                       const int32_t* block_expert, const int32_t* num_blocks, int64_t capacity, int64_t num_slots, int experts,
                       int top, int ff, int width, float limit, float alpha, int dtype, void* stream);
/* expert_out fp32 [slots, width]: row slot = W_down(expert) y[its sorted row]; w_down [experts, width, ff]. */
int aphro_experts_down_gemm(float* expert_out, const void* y, const void* w_down, const int32_t* sorted_slots,
                        const int32_t* block_expert, const int32_t* num_blocks, int64_t capacity, int64_t num_slots, int experts,
                        int top, int width, int ff, int dtype, void* stream);
/* out[t] = sum_k weights[t, k] * (ids[t, k] < experts ? expert_out[t * top + k] : h[t])
 *          + sigmoid(shared_gate[t]) * shared[t]        (shared NULL: none; shared_gate NULL: ungated; one number per row) */
int aphro_experts_combine(void* out, const float* expert_out, const int32_t* ids, const float* weights, const void* h,
                      int64_t h_stride, const void* shared, int64_t shared_stride, const void* shared_gate,
                      int64_t shared_gate_stride, int64_t num_tokens, int width, int top, int experts, int dtype, void* stream);
/* out[t, j] = g * sigmoid(alpha * g) * (u + 1), g = min(in[t, j], limit), u = clamp(in[t, d + j], +-limit), j < d;
 * limit <= 0 (here and in aphro_experts_glu_gemm): the plain gated form in[t, j] * sigmoid(alpha * in[t, j]) * in[t, d + j] */
int aphro_clamped_glu(void* out, const void* in, int64_t in_stride, int64_t num_tokens, int d, float limit, float alpha,
                      int dtype, void* stream);

/* ---- sublayers side by side, hashed token-pair embedding, attention through a low-rank latent ------------------------------ */

/* x[t] = table[ids[t]] + pair_table[row], row = (previous * mul_prev + ids[t] * mul_cur) mod buckets, or row `buckets` for a
 * sequence's first token (pair_table has buckets + 1 rows).  The previous token of a segment's first row is
 * token_state[state_slots[s]] (read only if ctx_len[s] > 0).  x fp32 [T, width]. */
int aphro_hashed_pair_embed(float* x, const void* table, const void* pair_table, const int64_t* ids, const int32_t* token_state,
                            const int32_t* state_slots, const int32_t* q_start, const int32_t* ctx_len,
                            const int32_t* seq_of_token, int64_t num_tokens, int width, int64_t vocab, int64_t buckets,
                            int64_t mul_prev, int64_t mul_cur, int dtype, void* stream);
/* token_state[state_slots[s]] = the last token of segment s (after hashed_pair_embed of the same step, on the same stream) */
int aphro_token_state_write(int32_t* token_state, const int64_t* ids, const int32_t* state_slots, const int32_t* q_start,
                            const int32_t* q_len, int num_seqs, void* stream);
/* x += ya + yb + bias (each optional), then out = x / rms(x) * weight (out NULL: the add alone).  x fp32 [T, width] in place;
 * ya, yb [T, width] of `dtype` with their row strides; bias, weight [width] of `dtype`; out [T, width] contiguous. */
int aphro_residual_add2_rms_norm(float* x, const void* ya, int64_t ya_stride, const void* yb, int64_t yb_stride, const void* bias,
                                 const void* weight, void* out, int64_t num_tokens, int width, float eps, int dtype, void* stream);

/* Per token, from the rows of one input product (proj, row stride proj_stride): cq[t] = rms_norm(proj[t, q_at : q_at + q_rank]) *
 * wq (q_rank 0: none); cache[slot_mapping[t]] = [rms_norm(proj[t, kv_at : kv_at + kv_rank]) * wkv | rotate(next rot_dim numbers)].
 * cache [num_cache_rows, kv_rank + rot_dim].  The rotation turns pair (i, i + rot_dims / 2) of the first rot_dims numbers by
 * position * inv_freq[i] and scales it by mscale; inv_freq fp32 [rot_dims / 2]. */
int aphro_latent_prep(void* cq, void* cache, int64_t num_cache_rows, const void* proj, int64_t proj_stride, int q_at, int kv_at,
                      const void* wq, const void* wkv, const int64_t* slot_mapping, const int32_t* q_start, const int32_t* ctx_len,
                      const int32_t* seq_of_token, const float* inv_freq, float mscale, int64_t num_tokens, int q_rank, int kv_rank,
                      int rot_dim, int rot_dims, float eps, int dtype, void* stream);
/* Causal softmax attention of every head over the shared latent rows cache [blocks, block, kv_rank + rot_dim]:
 * score = ([q_lat | rotate(q_rot)] . row) * scale, out = sum p * row[:kv_rank].  q_lat / q_rot / out are addressed as
 * base + t * stride + head * head_stride (elements); any sizes (kv_rank <= 1024), fp32 math.
 * window > 0: row i sees key j only if i - j < window.  sink fp32 [heads] (NULL: none): exp(sink[head]) -- not scaled -- is
 * one more term of the softmax denominator, without a value. */
int aphro_latent_attention_plain(void* out, int64_t out_stride, int64_t out_head_stride, const void* q_lat, int64_t ql_stride,
                                 int64_t ql_head_stride, const void* q_rot, int64_t qr_stride, int64_t qr_head_stride,
                                 const void* cache, const int32_t* block_tables, int max_blocks, int64_t num_blocks, int block_size,
                                 const int32_t* q_start, const int32_t* ctx_len, const int32_t* seq_of_token, const float* inv_freq,
                                 float mscale, int64_t num_tokens, int heads, int kv_rank, int rot_dim, int rot_dims, float scale,
                                 int window, const float* sink, int dtype, void* stream);
/* The same attention with the kernel chosen by size: bf16 with (kv_rank, rot_dim) in {(128, 16), (128, 32), (256, 32), (256, 64),
 * (512, 64)}, rot_dims == rot_dim and 16-byte aligned rows run on the matrix cores (aphro_latent_attention_fast_supported), the
 * query rows of a segment flattened to (token, head) pairs, 64 per workgroup; everything else runs the kernel above.  min/max
 * segment lengths and the longest ctx_len + q_len come from the host.  Decode-sized launches split long key ranges over
 * aphro_latent_attention_splits(...) workgroups when `workspace` holds num_tokens * heads * splits * (2 + kv_rank) floats. */
int aphro_latent_attention_fast_supported(int kv_rank, int rot_dim, int rot_dims, int dtype);
int aphro_latent_attention_splits(int64_t num_tokens, int num_seqs, int max_q_len, int heads, int max_kv_len);
int aphro_latent_attention(void* out, int64_t out_stride, int64_t out_head_stride, const void* q_lat, int64_t ql_stride,
                           int64_t ql_head_stride, const void* q_rot, int64_t qr_stride, int64_t qr_head_stride, const void* cache,
                           const int32_t* block_tables, int max_blocks, int64_t num_blocks, int block_size, const int32_t* q_start,
                           const int32_t* q_len, const int32_t* ctx_len, const int32_t* seq_of_token, const float* inv_freq,
                           float mscale, int64_t num_tokens, int num_seqs, int max_q_len, int max_kv_len, int heads, int kv_rank,
                           int rot_dim, int rot_dims, float scale, int window, const float* sink, float* workspace,
                           int64_t workspace_floats, int dtype, void* stream);
/* out[t, i] = x[t, i] * sigmoid(gate[t, i]), i < n (out may be x) */
int aphro_sigmoid_gate_mul(void* out, int64_t out_stride, const void* x, int64_t x_stride, const void* gate, int64_t gate_stride,
                           int64_t num_tokens, int n, int dtype, void* stream);
/* Sigmoid router limited to groups: s = sigmoid(router_out) fp32 [T, experts]; the experts form `groups` equal groups of
 * neighbours, a group's score is the sum of its group_top largest s, only the `keep` best groups' experts can be chosen; ids
 * int32 [T, top] are the `top` largest s among them, weights fp32 [T, top] = s * scale. */
int aphro_experts_route_grouped(int32_t* ids, float* weights, const float* router_out, int64_t num_tokens, int experts, int top,
                                int groups, int keep, int group_top, float scale, void* stream);

/* Router whose weights are the softmax over the chosen logits only: the `top` largest of router_out + bias (fp32 [outputs],
 * NULL: none; ties to the lower index) are chosen, weights = softmax over those `top` logits. */
int aphro_experts_route_topk(int32_t* ids, float* weights, const float* router_out, const float* bias, int64_t num_tokens,
                             int outputs, int top, void* stream);

/* ---- a residual in several streams, the gated delta rule, rotary attention's preparation ------------------------------------ */

/* Hyper-connections around x fp32 [T, streams, width], both halves optional:
 *   write (y != NULL):  x_t <- sum_s mix[s, t] x_s + mult * out_coef[t] * (scale (.) y)   all streams from the old ones
 *   read (out != NULL): u = sum_s in_coef[s] x_s;  out = u / sqrt(mean(u^2) + eps) * weight;  sum_out (fp32 [T, width], NULL: not
 *                       written) = u
 * y [T, width] (row stride), scale and weight [width] of `dtype` (NULL: ones); mix [streams, streams] indexed [from, to] (NULL:
 * identity), out_coef and in_coef [streams] (NULL: ones) are HOST arrays of floats, copied into the launch.  streams <= 16. */
int aphro_hyper_residual_rms_norm(float* x, const void* y, int64_t y_stride, const void* scale, const float* mix,
                                  const float* out_coef, float mult, const float* in_coef, const void* weight, void* out,
                                  float* sum_out, int64_t num_tokens, int streams, int width, float eps, int dtype, void* stream);
/* out[i] = cap * tanh(in[i] * scale / cap)  (cap <= 0: in[i] * scale); in of `dtype`, out fp32, n numbers */
int aphro_logit_softcap(float* out, const void* in, int64_t n, float scale, float cap, int dtype, void* stream);

/* Gated delta rule, one state S fp32 [dim, vdim] per (slot, head):
 *   S <- g S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q      (the read-out sees the current token's write)
 * q, k [T, kv_heads * dim] are made unit vectors per head here (x / sqrt(sum x^2 + norm_eps); q times q_scale); value head h
 * uses query / key head h / (heads / kv_heads); v [T, heads * vdim]; beta = sigmoid(b), g = exp(-exp(a_log[h]) *
 * softplus(a + dt_bias[h])) from b, a [T, heads] (row strides, `dtype`); a_log, dt_bias fp32 [heads].  out fp32 [T, heads * vdim].
 * state fp32 [slots, heads, dim, vdim]; a segment with ctx_len == 0 starts from zero without reading its slot.  dim <= 256.
 * max_q_len (host: longest segment) picks the work split. */
int aphro_gated_delta_scan(float* out, const void* q, int64_t q_stride, const void* k, int64_t k_stride, const void* v,
                           int64_t v_stride, const void* b, int64_t b_stride, const void* a, int64_t a_stride, const float* a_log,
                           const float* dt_bias, float* state, const int32_t* slot_of_seq, int num_slots, const int32_t* q_start,
                           const int32_t* q_len, const int32_t* ctx_len, int num_seqs, int64_t num_tokens, int heads, int kv_heads,
                           int dim, int vdim, float q_scale, float norm_eps, int max_q_len, int dtype, void* stream);
/* out[t, h, i] = x[t, h, i] / sqrt(mean_i x^2 + eps) * weight[i] * act(gate[t, h, i]); x fp32 [T, heads * vdim] contiguous;
 * weight [vdim] (shared by the heads; NULL: ones), gate (row stride; NULL: none) and out (row stride) of `dtype`;
 * act 0: sigmoid, 1: silu. */
int aphro_gated_head_rms_norm(void* out, int64_t out_stride, const float* x, const void* weight, const void* gate,
                              int64_t gate_stride, int64_t num_tokens, int heads, int vdim, float eps, int act, int dtype,
                              void* stream);

/* From the rows of a rotary attention's input product: the first rot_dims numbers of every query and key head turned by
 * position * inv_freq[i] (layout 0: number i pairs with i + rot_dims / 2; 1: number 2 i with 2 i + 1), then -- qk_norm != 0 --
 * every query and key head divided by sqrt(mean(x^2) + eps); values blended v <- (1 - lambda) v + lambda v_other (v_other NULL:
 * none).  Queries go to q_out [T, heads * dim], keys and values into k_cache [rows, kv_heads, dim] / v_cache [rows, kv_heads,
 * vdim] at slot_mapping[t] (outside 0 .. num_cache_rows - 1: skipped).  dim <= 512. */
int aphro_rotary_qk_norm_kv_write(void* q_out, int64_t q_out_stride, void* k_cache, void* v_cache, const int64_t* slot_mapping,
                                  int64_t num_cache_rows, const void* q, int64_t q_stride, const void* k, int64_t k_stride,
                                  const void* v, int64_t v_stride, const void* v_other, int64_t v_other_stride, float lambda,
                                  const int32_t* q_start, const int32_t* ctx_len, const int32_t* seq_of_token, const float* inv_freq,
                                  int64_t num_tokens, int heads, int kv_heads, int dim, int vdim, int rot_dims, int layout,
                                  int qk_norm, float eps, int dtype, void* stream);

#ifdef __cplusplus
}
#endif
#endif
