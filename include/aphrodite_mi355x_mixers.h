/*
 * aphrodite_mi355x_mixers.h -- C ABI of libaphrodite_mi355x_mixers.so
 *
 * MI355X (gfx950 / CDNA4) kernels of the sequence mixers that are not plain rotary softmax attention: layer norm around
 * an fp32 residual stream, gated activations, softmax attention over a paged cache with a tabulated distance bias and a
 * position-dependent query temperature, and gated outer-product memories (decay linear attention, mLSTM) with their state
 * in per-request slots.  Same conventions as aphrodite_mi355x.h: device pointers, sizes and a hipStream_t (void*); every
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

#ifdef __cplusplus
}
#endif
#endif
