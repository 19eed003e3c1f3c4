/* C-ABI of libvla_seq_gfx950.so: the layers of decoder stacks that keep their residual stream in
 * fp32 and mix tokens with a paged sliding-window attention and / or a gated linear recurrence.
 *
 * Conventions are those of vla_paged_attention.h: raw device pointers, element strides, VLA_F16 /
 * VLA_BF16 / VLA_F32 codes for the activation dtype, a hipStream_t, VLA_OK or a VLA_ERR_* code
 * back; nothing is allocated, every launch goes to the caller's stream and can be captured.
 *
 * A step is a packed batch of `num_tokens` rows that belong to `num_seqs` sequences: sequence b
 * owns rows query_start_loc[b] .. query_start_loc[b + 1] - 1, its tokens continue
 * context_lens[b] tokens that earlier steps left in the cache / state.  A decode step is the
 * case of one row per sequence; a prompt (or any portion of one) is the case of several.  The
 * same kernels serve both, so a position's result does not depend on how its sequence was cut.
 */
#ifndef VLA_SEQUENCE_OPS_H
#define VLA_SEQUENCE_OPS_H

#include <stdint.h>

#include "vla_paged_attention.h"

#ifdef __cplusplus
extern "C" {
#endif

int vla_seq_last_hip_error(void);

/* out[t, :] = table[ids[t], :] + pe(positions[t]) in fp32, pe[2i] = sin(p * inv_freq[i]),
 * pe[2i + 1] = cos(p * inv_freq[i]).  table is `dtype`, inv_freq fp32 [(width + 1) / 2]
 * (null: no position term). */
int vla_seq_embed_positions(float* out, const void* table, const int64_t* ids,
                            const int64_t* positions, const float* inv_freq, int num_tokens,
                            int width, int vocab, int dtype, void* stream);

/* RMS norm of an fp32 stream with a single gain: first x += add_rows + add_row (either may be
 * null; add_rows [T, width] fp32, add_row [width] fp32; x is written back when one is given),
 * then out = dtype(x / sqrt(mean(x^2) + eps) * gain[0]). */
int vla_seq_scalar_rms_norm(void* out, float* x, const float* add_rows, const float* add_row,
                            const float* gain, float eps, int num_tokens, int width, int dtype,
                            void* stream);

/* x[fp32] += y[dtype], elementwise over n values. */
int vla_seq_residual_add(float* x, const void* y, int64_t n, int dtype, void* stream);

/* PolyNorm: out = c0 N(z) + c1 N(z^2) + c2 N(z^3) + c3 per row of `features` values,
 * N(u) = u / sqrt(mean(u^2) + eps); coef fp32 [4] on the device; fp32 arithmetic. */
int vla_seq_poly_norm(void* out, int64_t out_stride, const void* z, int64_t z_stride,
                      const float* coef, float eps, int num_tokens, int features, int dtype,
                      void* stream);

/* Per (token, head): out = dtype(o / sqrt(mean_v(o^2) + eps) * weight[v] * silu(gate) * scale);
 * o fp32 [T, heads, vdim] contiguous, weight fp32 [vdim], gate / out `dtype` rows of
 * heads * vdim with their own strides. */
int vla_seq_gated_head_rms_norm(void* out, int64_t out_stride, const float* o,
                                const float* weight, const void* gate, int64_t gate_stride,
                                float eps, float scale, int num_tokens, int heads, int vdim,
                                int dtype, void* stream);

/* Keys of a step into the paged key cache [num_blocks, block_size, kv_heads, dim] (`dtype`);
 * slot = block * block_size + offset, negative = skip. */
int vla_seq_key_cache_write(void* cache, const void* k, int64_t k_stride,
                            const int64_t* slot_mapping, int num_tokens, int kv_heads, int dim,
                            int block_size, int num_blocks, int dtype, void* stream);

/* Sliding-window attention over the paged key cache whose values are its keys.
 * For the token at position p of sequence b and query head h (KV head h / (heads / kv_heads)):
 *   s_j = (q . k_j) * scale * (1 + temp_coef * ln(floor((p + 1) / temp_every) + 1))
 *         - slopes[h] * (p - j)            for max(0, p - window + 1) <= j <= p
 *   out = sum_j softmax(s)_j k_j, then * sigmoid(gate) (gate null: no gate) * out_scale.
 * All of it fp32; the step's own keys must be in the cache already.  slopes null = no bias,
 * temp_coef 0 = no temperature, window <= 0 = everything before p.  token_seq [T] names each
 * row's sequence; positions int64 [T]; block_tables int32 [num_seqs, max_blocks]. */
int vla_seq_window_attention(void* out, int64_t out_stride, const void* q, int64_t q_stride,
                             const void* gate, int64_t gate_stride, const void* cache,
                             const int* block_tables, int max_blocks, const int* token_seq,
                             const int64_t* positions, const float* slopes, int num_tokens,
                             int heads, int kv_heads, int dim, int block_size, int num_blocks,
                             int window, float scale, float temp_coef, float temp_every,
                             float out_scale, int dtype, void* stream);

/* Log-decays of a gated linear recurrence from a low-rank projection:
 * out[t, c] = -softplus(-(sum_r w2[c, r] y[t, r] + bias[c])) * inv_tau   (= ln sigmoid(z)^(1/tau)),
 * fp32; y `dtype` [T, rank] with stride, w2 `dtype` [channels, rank], bias fp32 [channels]. */
int vla_seq_gla_log_decay(float* out, const void* y, int64_t y_stride, const void* w2,
                          const float* bias, float inv_tau, int num_tokens, int channels,
                          int rank, int dtype, void* stream);

/* Gated linear attention with a per-key-channel decay, state carried in fp32 slots:
 *   S_t = diag(exp(g_t)) S_(t-1) + k_t v_t^T,   o_t = S_t^T (q_t * q_scale)
 * per head, S [dim, vdim].  Sequence b starts from zero when context_lens[b] == 0 and from
 * state[state_slots[b]] otherwise, and leaves its state there.  q, k [T, heads * dim] and
 * v [T, heads * vdim] `dtype` with strides, log_decay fp32 [T, heads * dim], o fp32
 * [T, heads, vdim], state fp32 [num_slots, heads, dim, vdim].  max_query_len: the longest run of
 * rows of one sequence in the step, or 0 if unknown (a hint that sizes the staging buffers). */
int vla_seq_gla_scan(float* o, const void* q, int64_t q_stride, const void* k, int64_t k_stride,
                     const void* v, int64_t v_stride, const float* log_decay, float* state,
                     const int* query_start_loc, const int* context_lens, const int* state_slots,
                     float q_scale, int num_seqs, int num_slots, int max_query_len, int heads,
                     int dim, int vdim, int dtype, void* stream);

/* A long run of rows cut into pieces that are walked at once (each from a zero state, through
 * vla_seq_gla_scan with one entry per piece): with c_t the sum of the log decays from a piece's
 * first row to row t, vla_seq_gla_piece_prefix writes q_decayed[t] = q[t] * q_scale * exp(c_t)
 * (fp32 [T, channels], channels = heads * dim) and totals[piece] = exp(c_last) for the pieces
 * piece_start_loc[i] .. piece_start_loc[i + 1] - 1; the caller adds q_decayed S_start to the
 * outputs of each piece (a matrix product).  vla_seq_gla_combine_states walks one sequence's
 * pieces: state[slots[i]] <- totals[pieces[i]] (per key channel) * state[slots[i - 1]] +
 * state[slots[i]] for i = 1 .. count - 1, then state[final_slot] <- state[slots[count - 1]]. */
int vla_seq_gla_piece_prefix(float* q_decayed, float* totals, const void* q, int64_t q_stride,
                             const float* log_decay, const int* piece_start_loc, float q_scale,
                             int num_pieces, int channels, int dtype, void* stream);
int vla_seq_gla_combine_states(float* state, const int* slots, const int* pieces,
                               const float* totals, int count, int final_slot, int num_slots,
                               int heads, int dim, int vdim, void* stream);

/* The same attention for 16-bit activations, tiled over runs of 32 query rows of a sequence on
 * the matrix cores: rows query_start_loc[b] .. query_start_loc[b + 1] - 1 of sequence b sit at
 * positions context_lens[b] ...  dim must be a multiple of 32, at most 128
 * (vla_seq_window_attention_tiles_supported); query rows and cache rows must be 8-byte aligned. */
int vla_seq_window_attention_tiles_supported(int dim, int dtype);
int vla_seq_window_attention_tiles(void* out, int64_t out_stride, const void* q, int64_t q_stride,
                                   const void* gate, int64_t gate_stride, const void* cache,
                                   const int* block_tables, int max_blocks,
                                   const int* query_start_loc, const int* context_lens,
                                   const float* slopes, int num_seqs, int max_query_len, int heads,
                                   int kv_heads, int dim, int block_size, int num_blocks,
                                   int window, float scale, float temp_coef, float temp_every,
                                   float out_scale, int dtype, void* stream);

/* Kernel choice for tests: window attention 0 = per shape, 1 = one wave per (row, head);
 * scan 0 = per shape, 1 = token by token. */
int vla_seq_set_window_kernel(int mode);
int vla_seq_set_scan_kernel(int mode);

#ifdef __cplusplus
}
#endif
#endif
