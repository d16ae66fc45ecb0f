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
 * position len_k(b) - len_q(b) + i.  Dv <= 256.
 * max_seqlen_q / max_seqlen_k: the most rows / keys any sequence has in this step (0 = unknown).  Three kernels
 * share the work: sequences with several rows run on a bf16 MFMA tile kernel (head sizes in multiples of 16) sized from
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
/* Scratch bytes the launch above needs for these sizes (key slices of single rows; 0 when it needs none). */
NV_API int64_t nv_attn_scoremod_workspace_bytes(int num_seqs, int64_t T, int H, int G, int Dv, int max_seqlen_k);

/*
 * Short causal convolution over time per channel, then SiLU, with the last taps-1 inputs of every sequence carried
 * in conv_state[slot] ([num_slots, taps-1, C] of dtype).  x, y: [T, C] with row strides; w: [C, taps] fp32, the
 * last column multiplies the current token.  A sequence at position 0 ignores what its slot holds.  taps <= 8.
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

#ifdef __cplusplus
}
#endif
#endif /* NANOVLLM_HIP_MIXERS_H */
