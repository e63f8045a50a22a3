/*
 * nanovllm_hip_mixers.h -- C ABI of the second gfx950 library (libnanovllm_hip_mixers.so).
 *
 * Same conventions as nanovllm_hip.h (raw device pointers, a HIP stream as void*, NV_OK or a negative NV_ERR_* code,
 * nv_strerror / nv_last_error / nv_abi_version exported by this library too).
 */
#ifndef NANOVLLM_HIP_MIXERS_H
#define NANOVLLM_HIP_MIXERS_H

#include "nanovllm_hip.h"

#ifdef __cplusplus
extern "C" {
#endif

/* -------------------------------------------------------------------------------------------------
 * Entry points for designs outside the reference's model family (no counterpart in the reference):
 * an fp32 residual stream with LayerNorms, attention with score modifiers and free head sizes, and a
 * recurrent mixer with per-sequence state slots.  They take the element type of activations and
 * caches as an argument; norm weights, biases, sinks, distance biases and decay constants are fp32.
 * ------------------------------------------------------------------------------------------------- */
#define NV_DTYPE_BF16 0
#define NV_DTYPE_F32 1

/*
 * One sublayer boundary of an fp32 residual stream, per row:
 *   r <- r + LN(h; w1, b1) + extra        (h and/or extra may be NULL: that part is absent; r is written
 *                                          only if it changed)
 *   y <- LN(r; w2, b2)                    (y may be NULL)
 * LN(x; w, b) = (x - mean) / sqrt(mean((x - mean)^2) + eps) * w + b, all in fp32.
 * resid, extra: [rows, cols] fp32 contiguous; h: [rows, cols] of h_dtype with row stride h_stride;
 * y: [rows, cols] of y_dtype contiguous.  cols <= 16384.
 */
NV_API int nv_add_layernorm(void* resid, const void* h, int h_dtype, int64_t h_stride, const void* w1,
                            const void* b1, const void* extra, const void* w2, const void* b2, void* y,
                            int y_dtype, int64_t rows, int cols, float eps, void* stream);

/* y[r, j] = gelu_tanh(x[r, j]) * x[r, inter + j]; gelu_tanh(z) = z/2 (1 + tanh(sqrt(2/pi) (z + 0.044715 z^3))). */
NV_API int nv_gelu_tanh_and_mul(const void* x, void* y, int dtype, int64_t rows, int inter, int64_t x_stride,
                                void* stream);

/*
 * Query/key preparation and KV scatter in front of nv_attn_scoremod_paged.
 *   rotary: pairs (2i, 2i+1), i < rot_dims/2, of every q and k head are rotated by positions[t] * inv_freq[i]
 *           (rot_dims = 0: none);
 *   query temperature: q *= 1 + temp_coef * ln(floor((p + 1) / temp_every) + 1)   (temp_every = 0: none);
 *   scatter: k (rotated) and v rows go to k_cache / v_cache at slot_mapping[t] (slot < 0 or NULL mapping: skipped).
 * q: [T, H, D], k: [T, G, D], v: [T, G, Dv] with token strides; q_out: [T, H, D] contiguous;
 * k_cache: [num_slots, G, D], v_cache: [num_slots, G, Dv].
 */
NV_API int nv_qk_prep_store(const void* q, const void* k, const void* v, void* q_out, void* k_cache,
                            void* v_cache, const int64_t* positions, const int32_t* slot_mapping,
                            const float* inv_freq, int rot_dims, float temp_coef, int temp_every, int dtype,
                            int64_t T, int H, int G, int D, int Dv, int64_t q_stride, int64_t k_stride,
                            int64_t v_stride, void* stream);

/*
 * Causal paged attention with score modifiers (fp32 scores and softmax):
 *   s = scale * q.k;  s = softcap * tanh(s / softcap) if softcap > 0;  s += dist_bias[h][min(i - j, n_dist - 1)] if
 *   dist_bias;  the softmax denominator also holds exp(sink[h]) if sink.
 * q: [T, H, D] (token stride q_stride), out: [T, H, Dv] (token stride out_stride);
 * k_cache: [num_blocks, block_size, G, D], v_cache: [num_blocks, block_size, G, Dv]; query i of sequence b sits at
 * position len_k(b) - len_q(b) + i.  Dv <= 512 (above 256 on the row-per-wave kernel only).
 * max_seqlen_q / max_seqlen_k: the most rows / keys any sequence has in this step (0 = unknown).  Three kernels
 * share the work: sequences with several rows run on a bf16 MFMA tile kernel (head sizes: multiples of 16 up to 128, of 32 up to 320 / 256) sized from
 * max_seqlen_q; sequences with one row on a decode kernel that reads K/V once per group of query heads and cuts long
 * contexts into key slices (planned from max_seqlen_k, joined through `workspace`); whatever shape neither takes
 * runs one row per wave.  single_rows = 0 promises that no sequence has exactly one row; max_seqlen_q = 1 that all do.
 */
NV_API int nv_attn_scoremod_paged(const void* q, const void* k_cache, const void* v_cache, void* out,
                                  const int32_t* cu_seqlens_q, const int32_t* cu_seqlens_k,
                                  const int32_t* block_tables, int num_seqs, int max_blocks_per_seq, int64_t T,
                                  int H, int G, int D, int Dv, int64_t num_blocks, int block_size, float scale,
                                  float softcap, const float* sink, const float* dist_bias, int n_dist,
                                  int max_seqlen_q, int max_seqlen_k, int single_rows, int dtype, int64_t q_stride,
                                  int64_t out_stride, void* workspace, int64_t workspace_bytes, void* stream);
/* The same with the value rows `v_row_stride` elements apart (>= Dv; Dv: a dense cache).  A value cache that is a
 * column range of the key cache (value row = the first Dv columns of the key row, v_row_stride = G * D with G = 1, or
 * any layout with one stride between consecutive (slot, kv head) rows) is read in place. */
NV_API int nv_attn_scoremod_paged_vld(const void* q, const void* k_cache, const void* v_cache, int64_t v_row_stride,
                                      void* out, const int32_t* cu_seqlens_q, const int32_t* cu_seqlens_k,
                                      const int32_t* block_tables, int num_seqs, int max_blocks_per_seq, int64_t T,
                                      int H, int G, int D, int Dv, int64_t num_blocks, int block_size, float scale,
                                      float softcap, const float* sink, const float* dist_bias, int n_dist,
                                      int max_seqlen_q, int max_seqlen_k, int single_rows, int dtype, int64_t q_stride,
                                      int64_t out_stride, void* workspace, int64_t workspace_bytes, void* stream);
/* Scratch bytes the launches above need for these sizes (key slices of single rows; 0 when it needs none). */
NV_API int64_t nv_attn_scoremod_workspace_bytes(int num_seqs, int64_t T, int H, int G, int Dv, int max_seqlen_k);

/*
 * Short causal convolution over time per channel, then SiLU, with the last taps-1 inputs of every sequence carried
 * in conv_state[slot] ([num_slots, taps-1, C] of dtype).  x, y: [T, C] with row strides; w: [C, taps] fp32, the
 * last column multiplies the current token.  A sequence at position 0 ignores what its slot holds.  taps <= 64
 * (up to 8 the window is kept in registers).
 */
NV_API int nv_causal_conv_silu(const void* x, int64_t x_stride, const float* w, void* conv_state, void* y,
                               int64_t y_stride, const int32_t* cu_seqlens_q, const int32_t* cu_seqlens_k,
                               const int32_t* state_slots, int num_seqs, int64_t T, int C, int taps, int dtype,
                               void* stream);

/*
 * Gated delta rule with one decay per head and key channel, state [num_slots, H, D, Dv] fp32 carried per slot:
 *   S <- diag(g) S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q      (token by token)
 *   q, k: unit vectors per head (x / sqrt(sum x^2 + 1e-6)), q also times D^-1/2; value head h reads q/k head
 *   h / (H / G);  beta = sigmoid(b_raw[t, h]);  g = exp(-exp(A_log[h]) * softplus(a_raw[t, h, d] + dt_bias[h, d]));
 *   out[t, h, :] = o / sqrt(mean(o^2) + eps) * norm_w * sigmoid(gate_raw[t, h, :]).
 * q, k: [T, G, D]; v, gate_raw, out: [T, H, Dv]; a_raw: [T, H, D]; b_raw: [T, H]; all of dtype with token strides.
 * D, Dv <= 256.
 */
NV_API int nv_gated_delta_rule(const void* q, const void* k, const void* v, int64_t q_stride, int64_t k_stride,
                               int64_t v_stride, const void* a_raw, int64_t a_stride, const void* b_raw,
                               int64_t b_stride, const void* gate_raw, int64_t gate_stride, const float* A_log,
                               const float* dt_bias, const float* norm_w, float* state, void* out,
                               int64_t out_stride, const int32_t* cu_seqlens_q, const int32_t* cu_seqlens_k,
                               const int32_t* state_slots, int num_seqs, int H, int G, int D, int Dv, float eps,
                               int dtype, void* stream);

/* -------------------------------------------------------------------------------------------------
 * An fp32 stream with one grouped RMS norm per layer, parallel sublayers and a normalised side input.
 * ------------------------------------------------------------------------------------------------- */
/*
 * One boundary of an fp32 residual stream, per row and in place (every part optional):
 *   r <- r + mult * (add + sum_j parts[:, j])       add: [rows, cols] of dtype (row stride add_stride);
 *                                                   parts: [rows, n_parts, cols] fp32 contiguous
 *   r <- r + mult * n / sqrt(mean(n^2) + eps) * normed_w         normed: [rows, cols] of dtype
 *   copy <- r (dtype, contiguous)
 *   y32 / y <- grouped RMS norm of r times norm_w: the row is cut into `groups` equal consecutive parts and each is
 *   divided by its own sqrt(mean(part^2) + eps); y32 fp32, y of dtype, either or both.
 * cols <= 16384, groups <= 1024 and a divisor of cols.
 */
NV_API int nv_stream_boundary(void* resid, const void* add, int64_t add_stride, const void* parts, int n_parts,
                              const void* normed, int64_t normed_stride, const float* normed_w, float mult,
                              const float* norm_w, int groups, float eps, void* y32, void* y, void* copy, int dtype,
                              int64_t rows, int cols, void* stream);

/* y = x / sqrt(mean(x^2) + eps) * w per row; x (row stride x_stride) and y (contiguous) of dtype, w fp32. */
NV_API int nv_rms_norm_rows(const void* x, int64_t x_stride, const float* w, void* y, int dtype, int64_t rows,
                            int cols, float eps, void* stream);

/*
 * y[t, c] = x[t, c] + sum_j w[c, j] * x[t - taps + 1 + j, c]: a causal convolution over time per channel, added to its
 * input.  x: [T, C] fp32 contiguous; w: [C, taps] fp32 (the last column multiplies the current token); y: [T, C] of
 * y_dtype; conv_state: [num_slots, taps - 1, C] fp32, the last inputs of every sequence, updated.  A sequence at
 * position 0 ignores what its slot holds.
 */
NV_API int nv_causal_conv_add(const float* x, const float* w, float* conv_state, void* y, int y_dtype,
                              const int32_t* cu_seqlens_q, const int32_t* cu_seqlens_k, const int32_t* state_slots,
                              int num_seqs, int64_t T, int C, int taps, void* stream);

/* y[t, j] = gelu_tanh(z[t, j]) * table[ids[t], offset + j], j < dim; z, table, y of dtype, y contiguous. */
NV_API int nv_token_gate(const void* z, int64_t z_stride, const void* table, int64_t table_stride,
                         const int64_t* ids, int offset, int dim, void* y, int dtype, int64_t T, void* stream);

/*
 * Generalized delta rule, state [num_slots, H, D, D] fp32 carried per slot (key channel x value channel):
 *   u = k / sqrt(sum k^2 + key_eps);  w = exp(-decay_rate * sigmoid(w_raw + w_bias));  a = sigmoid(a_raw + a_bias)
 *   S <- diag(w) S - (a * u)(u^T S) + k v^T        (both terms read the old state; token by token)
 *   out[t, h] = (S^T r) / sqrt(mean((S^T r)^2) + eps) * norm_w[h] * sigmoid(gate_raw[t, h])
 * r, k, v, w_raw, a_raw, gate_raw, out: [T, H, D] of dtype with token strides; w_bias, a_bias, norm_w: [H, D] fp32.
 * D <= 256.
 */
NV_API int nv_general_delta_rule(const void* r, const void* k, const void* v, int64_t r_stride, int64_t k_stride,
                                 int64_t v_stride, const void* w_raw, int64_t w_stride, const void* a_raw,
                                 int64_t a_stride, const void* gate_raw, int64_t gate_stride, const float* w_bias,
                                 const float* a_bias, const float* norm_w, float* state, void* out, int64_t out_stride,
                                 const int32_t* cu_seqlens_q, const int32_t* cu_seqlens_k, const int32_t* state_slots,
                                 int num_seqs, int H, int D, float eps, float decay_rate, float key_eps, int dtype,
                                 void* stream);

/*
 * In front of nv_attn_scoremod_paged when keys / values are cached as one normalised latent per token plus one rotated
 * key part shared by all heads (attention in the latent space, G = 1, key size rank + R, value size rank):
 *   c = ckv[t, :rank] / sqrt(mean(.^2) + eps) * latent_w;   k_r = rot(ckv[t, rank:])
 *   q_full[t, h] = [q_lat[t, h] | rot(q[t, h, Dq - R:])];   k_cache[slot] = [c | k_r];   v_cache[slot] = c
 *   (v_cache NULL: the values are read out of the key rows, nothing else is stored)
 * rot turns pair i by positions[t] * freq[i], cos and sin times mag; pairs (2i, 2i+1) if interleaved else (i, i + R/2).
 * q: [T, H, Dq] (token stride q_stride); q_lat: [T, H, rank] with token / head strides; ckv: [T, rank + R];
 * q_full: [T, H, rank + R] contiguous; k_cache: [num_slots, rank + R]; v_cache: [num_slots, rank].
 */
NV_API int nv_latent_prep_store(const void* q, int64_t q_stride, int Dq, const void* q_lat, int64_t ql_stride_t,
                                int64_t ql_stride_h, const void* ckv, int64_t ckv_stride, const float* latent_w,
                                const float* freq, float mag, int interleaved, const int64_t* positions,
                                const int32_t* slot_mapping, void* q_full, void* k_cache, void* v_cache, int dtype,
                                int64_t T, int H, int rank, int R, float eps, void* stream);

/*
 * Routed experts.  nv_moe_route: the `top` largest of every row of logits [T, E] (fp32), weights = softmax over the
 * chosen; ids / weights: [T, top].  nv_moe_align: sorted_pairs [pairs] = the (token, choice) pairs ordered by expert,
 * meta = [number of row tiles, then (expert, first position, rows) per tile], tiles of at most tile_rows (16 or 64,
 * nv_moe_tile_rows suggests one) rows of one expert; meta holds 1 + 3 * nv_moe_max_tiles ints.  nv_moe_gate_up:
 * y[position] = g * sigmoid(alpha g) * (u + 1), g = min(G_e h, limit), u = clamp(U_e h, -limit, limit), with
 * gate_up: [E, 2 ff, width] (gate rows, then up rows), y: [pairs, ff] of dtype.  nv_moe_down: out[pair] =
 * pair_weights[pair] * (D_e y[position]), down: [E, width, ff], out: [pairs, width] fp32.
 */
NV_API int nv_moe_route(const float* logits, int32_t* ids, float* weights, int64_t T, int E, int top, void* stream);
NV_API int nv_moe_tile_rows(int64_t pairs, int E);
NV_API int64_t nv_moe_max_tiles(int64_t pairs, int E, int tile_rows);
NV_API int nv_moe_align(const int32_t* ids, int32_t* sorted_pairs, int32_t* meta, int64_t pairs, int E,
                        int tile_rows, void* stream);
NV_API int nv_moe_gate_up(const void* h, int64_t h_stride, const void* gate_up, const int32_t* sorted_pairs,
                          const int32_t* meta, void* y, int dtype, int64_t pairs, int E, int top, int width, int ff,
                          float limit, float alpha, int tile_rows, void* stream);
NV_API int nv_moe_down(const void* y, const void* down, const int32_t* sorted_pairs, const int32_t* meta,
                       const float* pair_weights, float* out, int dtype, int64_t pairs, int E, int width, int ff,
                       int tile_rows, void* stream);

/* nv_causal_conv_silu with a bias [C] (fp32, may be NULL) added to the convolution before the SiLU. */
NV_API int nv_causal_conv_bias_silu(const void* x, int64_t x_stride, const float* w, const float* bias, void* conv_state,
                                    void* y, int64_t y_stride, const int32_t* cu_seqlens_q, const int32_t* cu_seqlens_k,
                                    const int32_t* state_slots, int num_seqs, int64_t T, int C, int taps, int dtype,
                                    void* stream);

/* The same convolution with the activation as an argument: NV_CONV_ACT_NONE leaves the sum as it is. */
#define NV_CONV_ACT_NONE 0
#define NV_CONV_ACT_SILU 1
NV_API int nv_causal_conv_act(const void* x, int64_t x_stride, const float* w, const float* bias, void* conv_state,
                              void* y, int64_t y_stride, const int32_t* cu_seqlens_q, const int32_t* cu_seqlens_k,
                              const int32_t* state_slots, int num_seqs, int64_t T, int C, int taps, int act, int dtype,
                              void* stream);

/* nv_moe_gate_up with a free shift of the up branch: act = g * sigmoid(alpha g) * (u + up_shift); limit = +inf, alpha = 1,
 * up_shift = 0 is the plain SiLU-gated unit. */
NV_API int nv_moe_gate_up_act(const void* h, int64_t h_stride, const void* gate_up, const int32_t* sorted_pairs,
                              const int32_t* meta, void* y, int dtype, int64_t pairs, int E, int top, int width, int ff,
                              float limit, float alpha, float up_shift, int tile_rows, void* stream);

/*
 * Embedding with a hashed bigram table, RMS-normed into an fp32 stream x [T, cols]:
 *   x[t] = rmsnorm(embed[id_t] + bigram[row_t]) * norm_w,  row_t = (id_{t-1} * mul_prev + id_t * mul_cur) mod buckets,
 *   or row `buckets` at position 0.  prev_state [num_slots] int64 carries each sequence's last id between steps.
 *   bigram NULL: the embedding row alone.  norm_w NULL: the sum goes into the stream as it is.  embed: [vocab, cols], bigram: [buckets + 1, cols] of dtype.
 */
NV_API int nv_hashed_bigram_embed(const int64_t* ids, const int64_t* positions, const void* embed, const void* bigram,
                                  int64_t buckets, int64_t mul_prev, int64_t mul_cur, const float* norm_w, float eps,
                                  int64_t* prev_state, float* x, const int32_t* cu_seqlens_q, const int32_t* state_slots,
                                  int num_seqs, int64_t T, int cols, int dtype, void* stream);

/*
 * One layer boundary of an fp32 stream that is read through two RMS norms, per row and in place:
 *   r += add1 + add2 + parts_scale * sum_j parts[:, j]                          (each may be NULL / absent)
 *   r += normed_mult * (rmsnorm(normed1) * normed1_w + rmsnorm(normed2) * normed2_w)      (each may be NULL)
 *   y32[:, :cols] = rmsnorm(r) * norm_a;  y32[:, cols:] = rmsnorm(r) * norm_b    (norm_b NULL: y32 is [rows, cols])
 *   y = rmsnorm(r) * norm_a in dtype                                             (y32 and / or y)
 * add*, normed*: [rows, cols] of dtype with row strides; parts: [rows, n_parts, cols] fp32.
 */
NV_API int nv_stream_boundary_pair(void* resid, const void* add1, int64_t add1_stride, const void* add2,
                                   int64_t add2_stride, const float* parts, int n_parts, float parts_scale,
                                   const void* normed1, int64_t normed1_stride, const float* normed1_w,
                                   const void* normed2, int64_t normed2_stride, const float* normed2_w, float normed_mult,
                                   const float* norm_a, const float* norm_b, float eps, float* y32, void* y, int dtype,
                                   int64_t rows, int cols, void* stream);

/* y = max(x, 0)^2; x: [rows, cols] with a row stride, y contiguous. */
NV_API int nv_relu_squared(const void* x, int64_t x_stride, void* y, int dtype, int64_t rows, int cols, void* stream);

/*
 * Decayed outer-product memory read BEFORE it is written, with a bonus for the current token; state
 * [num_slots, H, Dk, Dv] fp32 carried per slot:
 *   w = exp(-exp(w_raw + w_bias));  o = (S + diag(bonus) k v^T)^T r;  S <- diag(w) S + k v^T      (token by token)
 *   out[t, h] = o / sqrt(mean(o^2) + eps) * norm_w[h] * silu(gate_raw[t, h])
 * r, k, w_raw: [T, H, Dk]; v, gate_raw, out: [T, H, Dv] of dtype with token strides; w_bias, bonus: [H, Dk] fp32;
 * norm_w: [H, Dv] fp32.  Dk, Dv <= 256.
 */
NV_API int nv_decay_memory(const void* r, const void* k, const void* v, int64_t r_stride, int64_t k_stride,
                           int64_t v_stride, const void* w_raw, int64_t w_stride, const void* gate_raw,
                           int64_t gate_stride, const float* w_bias, const float* bonus, const float* norm_w, float* state,
                           void* out, int64_t out_stride, const int32_t* cu_seqlens_q, const int32_t* cu_seqlens_k,
                           const int32_t* state_slots, int num_seqs, int H, int Dk, int Dv, float eps, int dtype,
                           void* stream);

/*
 * State-space scan with one scalar decay per head and step; state [num_slots, H, N, P] fp32 carried per slot:
 *   dt = softplus(dt_raw + dt_bias);  S <- exp(-exp(A_log) dt) S + dt B x^T;  y = S^T C + D x;  out = y * silu(z)
 * x, z: [T, H, P]; B, C: [T, G, N] (head h reads group h / (H / G)); dt_raw: [T, H] of dtype with token strides;
 * dt_bias, A_log, D: [H] fp32; out: [T, H * P] fp32 (a grouped norm follows).  N, P <= 256.
 */
NV_API int nv_state_space_scan(const void* x, const void* B, const void* C, int64_t x_stride, int64_t b_stride,
                               int64_t c_stride, const void* dt_raw, int64_t dt_stride, const void* z, int64_t z_stride,
                               const float* dt_bias, const float* A_log, const float* D_skip, float* state, float* out,
                               int64_t out_stride, const int32_t* cu_seqlens_q, const int32_t* cu_seqlens_k,
                               const int32_t* state_slots, int num_seqs, int H, int G, int N, int P, int dtype,
                               void* stream);

/*
 * out[s, t] = h[t] + (h[t-1] - h[t]) * mu[s] for n_mix blends at once; the row before a sequence's first row of the
 * step comes from state[slot] (zeros at position 0), which then takes the step's last row.  h: [T, C] of dtype with a
 * row stride; mu: [n_mix, C] fp32; state: [num_slots, C] of dtype; out: [n_mix, T, C] of dtype.
 */
NV_API int nv_token_shift_mix(const void* h, int64_t h_stride, const float* mu, int n_mix, void* state, void* out,
                              const int32_t* cu_seqlens_q, const int32_t* cu_seqlens_k, const int32_t* state_slots,
                              int num_seqs, int64_t T, int C, int dtype, void* stream);

/* y = x / sqrt(mean(part^2) + eps) * w over `groups` equal consecutive parts of every fp32 row; y of y_dtype. */
NV_API int nv_group_rms_norm(const float* x, int64_t x_stride, const float* w, void* y, int64_t y_stride, int y_dtype,
                             int64_t rows, int cols, int groups, float eps, void* stream);

/*
 * In front of nv_attn_chunk_sigmoid_paged: RMS norm over the whole q row [H * D] and the whole k row [G * D] (weights
 * q_norm, k_norm of those sizes), rotate-half rotary on the first rot_dims dimensions of every head (pair (i, i +
 * rot_dims / 2) by positions[t] * freq[i]), every value head turned the same way over all Dv dimensions by positions[t] *
 * value_freq[m], and the scatter of the rotated k / v rows into the paged caches.  q_out: [T, H, D] contiguous.
 */
NV_API int nv_chunk_attn_prep_store(const void* q, const void* k, const void* v, int64_t q_stride, int64_t k_stride,
                                    int64_t v_stride, const float* q_norm, const float* k_norm, float eps,
                                    const float* freq, int rot_dims, const float* value_freq, const int64_t* positions,
                                    const int32_t* slot_mapping, void* q_out, void* k_cache, void* v_cache, int dtype,
                                    int64_t T, int H, int G, int D, int Dv, void* stream);

/*
 * Sigmoid attention inside chunks of `chunk` positions (0: plain causal) over a paged cache of ROTATED values:
 *   out[i] = R(-i) sum_{j <= i, same chunk} sigmoid(scale q_i . k_j + head_bias[h]) v_cache[j]
 * R(p) turns the pair (m, m + Dv / 2) by p * value_freq[m].  q: [T, H, D]; caches [num_blocks, block_size, G, D | Dv];
 * out: [T, H * Dv].  tile_seq / tile_q0 [num_tiles] (may be 0 tiles): blocks of 64 query rows of sequences with several
 * rows, for the bf16 MFMA kernel (nv_attn_chunk_sigmoid_tile_ok says whether it is built for the sizes); with tiles,
 * single_rows != 0 says that the step also has sequences with one row.  Without tiles every row takes the
 * one-wave-per-row kernel.
 */
NV_API int nv_attn_chunk_sigmoid_tile_ok(int D, int Dv, int dtype);
NV_API int nv_attn_chunk_sigmoid_paged(const void* q, const void* k_cache, const void* v_cache, void* out,
                                       const int32_t* cu_seqlens_q, const int32_t* cu_seqlens_k,
                                       const int32_t* block_tables, int num_seqs, int max_blocks, int64_t T, int H, int G,
                                       int D, int Dv, int64_t num_blocks, int block_size, float scale,
                                       const float* head_bias, int chunk, const float* value_freq,
                                       const int32_t* tile_seq, const int32_t* tile_q0, int num_tiles, int single_rows,
                                       int dtype, int64_t q_stride, int64_t out_stride, void* stream);

/* -------------------------------------------------------------------------------------------------
 * An fp32 stream whose sublayers run one after the other, each output scaled per column; memories that are written
 * before they are read; attention whose values are its un-normed keys; sigmoid routing over groups of experts.
 * ------------------------------------------------------------------------------------------------- */
/*
 * One sublayer boundary of a pre-norm fp32 stream, per row and in place (every part optional):
 *   r += col_scale * (add1 + sigmoid(gate2[row]) * add2 + sum_j parts[:, j])
 *   y32 / y = r / sqrt(mean(r^2) + eps) * norm_w                       (fp32 and / or dtype; norm_w NULL: no norm)
 * add1, add2: [rows, cols] of dtype with row strides; gate2: one raw gate per row of dtype, gate2_stride elements apart
 * (NULL: add2 counts fully); parts: [rows, n_parts, cols] fp32; col_scale, norm_w: [cols] fp32.  cols <= 16384.
 */
NV_API int nv_stream_boundary_scaled(void* resid, const void* add1, int64_t add1_stride, const void* add2,
                                     int64_t add2_stride, const void* gate2, int64_t gate2_stride, const float* parts,
                                     int n_parts, const float* col_scale, const float* norm_w, float eps, float* y32,
                                     void* y, int dtype, int64_t rows, int cols, void* stream);

/* y = c0 z / rms(z) + c1 z^2 / rms(z^2) + c2 z^3 / rms(z^3) + c3 per row (powers element by element, rms(u) =
 * sqrt(mean(u^2) + eps) over the row, fp32); x: [rows, cols] of dtype with a row stride, coef: 4 fp32 on the device,
 * y contiguous. */
NV_API int nv_poly_norm(const void* x, int64_t x_stride, const float* coef, float eps, void* y, int dtype, int64_t rows,
                        int cols, void* stream);

/*
 * In front of nv_attn_scoremod_paged: per-head RMS norm of q and k (weights q_norm, k_norm [D], shared by the heads),
 * rotate-half rotary on the first rot_dims dimensions (pair (i, i + rot_dims / 2) by positions[t] * freq[i]); the
 * prepared k rows are scattered into k_cache and the k rows AS GIVEN into v_cache (slot < 0 or NULL mapping: skipped).
 * q: [T, H, D], k: [T, G, D] with token strides; q_out: [T, H, D] contiguous; caches [num_slots, G, D].
 */
NV_API int nv_head_norm_rope_store(const void* q, const void* k, int64_t q_stride, int64_t k_stride, const float* q_norm,
                                   const float* k_norm, float eps, const float* freq, int rot_dims,
                                   const int64_t* positions, const int32_t* slot_mapping, void* q_out, void* k_cache,
                                   void* v_cache, int dtype, int64_t T, int H, int G, int D, void* stream);

/*
 * Matrix memory with exponential gates, written before it is read; per slot the state [H, Dk, Dv], the normaliser
 * [H, Dk] and the running maximum [H], all fp32 (a sequence at position 0 starts from zeros, the maximum from 0):
 *   i = cap tanh((i_pre + i_bias) / cap);  f = logsigmoid(cap tanh((f_pre + f_bias) / cap));  m' = max(f + m, i)
 *   S <- exp(f + m - m') S + exp(i - m') k v^T;  n likewise with k alone;  o = S^T (q q_scale) / (max(|n . q q_scale|,
 *   exp(-m')) + 1e-6);  out[t, h] = o / sqrt(mean(o^2) + eps) * norm_w[h] * sigmoid(gate_raw[t, h])
 * q, k: [T, H * Dk]; v, gate_raw, out: [T, H * Dv] of dtype with token strides; i_pre, f_pre: [T, H] fp32,
 * gate_pre_stride floats apart per token; i_bias, f_bias: [H]; norm_w: [H * Dv] fp32.  Dk, Dv <= 256.
 */
NV_API int nv_mlstm_memory(const void* q, const void* k, const void* v, int64_t q_stride, int64_t k_stride,
                           int64_t v_stride, const float* i_pre, const float* f_pre, int64_t gate_pre_stride,
                           const void* gate_raw, int64_t gate_stride, const float* i_bias, const float* f_bias,
                           const float* norm_w, float* state, float* norm_state, float* max_state, void* out,
                           int64_t out_stride, const int32_t* cu_seqlens_q, const int32_t* cu_seqlens_k,
                           const int32_t* state_slots, int num_seqs, int H, int Dk, int Dv, float eps, float gate_cap,
                           float q_scale, int dtype, void* stream);

/*
 * Keyless gated linear recurrence (what is written is one minus the forget gate); state [num_slots, H, Dk, Dv] fp32:
 *   f = lower + (1 - lower) sigmoid(f_raw + f_bias);  S <- diag(f) S + (1 - f) v^T;  o = S^T silu(q)
 *   out[t, h] = o / sqrt(mean(o^2) + eps) * norm_w            (norm_w: [Dv], the same for every head)
 * q, f_raw: [T, H * Dk]; v, out: [T, H * Dv] of dtype with token strides; f_bias, lower: [H * Dk] fp32.  Dk, Dv <= 256.
 */
NV_API int nv_gated_write_memory(const void* q, const void* f_raw, const void* v, int64_t q_stride, int64_t f_stride,
                                 int64_t v_stride, const float* f_bias, const float* lower, const float* norm_w,
                                 float* state, void* out, int64_t out_stride, const int32_t* cu_seqlens_q,
                                 const int32_t* cu_seqlens_k, const int32_t* state_slots, int num_seqs, int H, int Dk,
                                 int Dv, float eps, int dtype, void* stream);

/*
 * Routing by sigmoid scores: s = sigmoid(logits); the choice is made on s + correction (NULL: s) among the experts of
 * the keep_groups best of n_groups equal consecutive blocks of experts (a block's merit: the sum of its top two biased
 * scores, or its one score); weights = s of the chosen, as they are.  E <= 512.  ids, weights: [T, top].
 */
NV_API int nv_moe_route_grouped(const float* logits, const float* correction, int32_t* ids, float* weights, int64_t T,
                                int E, int top, int n_groups, int keep_groups, void* stream);

/* nv_moe_gate_up for experts without a gate: y[position] = max(U_e h, 0)^2, up: [E, ff, width]. */
NV_API int nv_moe_up_relu2(const void* h, int64_t h_stride, const void* up, const int32_t* sorted_pairs,
                           const int32_t* meta, void* y, int dtype, int64_t pairs, int E, int top, int width, int ff,
                           int tile_rows, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* NANOVLLM_HIP_MIXERS_H */
