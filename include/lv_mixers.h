/*
 * lv_mixers.h — C ABI of liblvmix.so: the MI355X (gfx950) kernels of the sequence mixers and the
 * residual machinery that are not plain softmax attention over a full causal context:
 *
 *   lv_hc_update_norm        hyper-connection stream update fused with the next sublayer's stream
 *                            read-out and grouped RMS norm
 *   lv_clamped_glu           clamped gated linear unit  min(g, L) * sigmoid(alpha g) * (clamp(u, -L, L) + 1)
 *   lv_delta_prep            short causal convolution + silu over the q/k/v channels of a ragged step,
 *                            unit-norm q and k, write strength and decay of the gated delta rule
 *   lv_conv_state_update     carries the last taps-1 convolution inputs of every sequence
 *   lv_gated_delta_rule      the recurrence itself, state in 32-bit, any number of new tokens per sequence
 *   lv_head_norm_gate        per-head RMS norm of the read-out times weight times silu(gate)
 *   lv_qk_fullnorm_store     RMS norm over the whole q and k projection, K/V scatter into the paged cache
 *   lv_pool_update           means of completed blocks of P cached keys and values
 *   lv_window_pool_attn      sliding-window attention over cached tokens plus pooled blocks that lie
 *                            before the window, softmax with a zero-score sink, sigmoid output gate
 *
 * A "ragged step" is a batch of B sequences; sequence b brings cu_q[b+1]-cu_q[b] new tokens that
 * follow ctx_lens[b] tokens already in the cache / state (a whole prompt, a portion of one, or one
 * decoded token: the kernels make no difference). tok_seq[t] is the sequence of packed token t.
 *
 * Conventions: device pointers; `dtype` LV_MIX_BF16 or LV_MIX_F32 is the element type of activations,
 * caches and convolution state ("act"); vectors named *_w, the stream tensor, recurrent state and
 * everything documented as f32 are 32-bit floats; index tensors int32; strides in elements; every
 * call only enqueues on `stream` (void* hipStream_t), allocates nothing and never synchronises.
 * Return 0 or a negative code; lv_mix_last_error() gives the message.
 */
#ifndef LV_MIXERS_H
#define LV_MIXERS_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define LV_MIX_ABI_VERSION 4
#define LV_MIX_BF16 0
#define LV_MIX_F32 1
#define LV_MIX_MAX_STREAMS 8

int lv_mix_abi_version(void);
const char* lv_mix_last_error(void);

/* x [T, S, W] f32, updated in place when y != NULL:  x'[t'] = sum_s mix[s, t'] x[s] + out_w[t'] * y.
 * When out != NULL:  u = sum_s in_w[s] x'[s];  out = grouped_rms_norm(u) * norm_w  (groups equal
 * consecutive parts, each divided by its own sqrt(mean(part^2) + eps)).  y, out: act [T, W]. */
int lv_hc_update_norm(void* x, const void* y, const void* mix, const void* out_w, const void* in_w,
                      const void* norm_w, void* out, int64_t T, int S, int W, int groups, float eps,
                      int dtype, void* stream);

/* in act [T, 2F] (row stride ld_in) = [gate | up];  out act [T, F]. */
int lv_clamped_glu(const void* in, int64_t ld_in, void* out, int64_t T, int F, float limit, float alpha,
                   int dtype, void* stream);

/* proj act [T, ld]: columns [0, G*D) q, [G*D, 2*G*D) k, [2*G*D, 2*G*D + H*Dv) v (the convolution
 * channels, C of them), b at column off_b (H wide), a at column off_a (H wide).
 * conv_w f32 [C, taps] (last column = current token); conv_state act [slots, taps-1, C].
 * Outputs f32: qn [T, G, D] (unit norm times D^-1/2), kn [T, G, D], v [T, H, Dv], beta [T, H], decay [T, H]. */
int lv_delta_prep(const void* proj, int64_t ld, const void* conv_w, const void* conv_state,
                  const void* A_log, const void* dt_bias, const int32_t* cu_q, const int32_t* ctx_lens,
                  const int32_t* slots, const int32_t* tok_seq, void* qn, void* kn, void* v, void* beta,
                  void* decay, int64_t T, int G, int H, int D, int Dv, int taps, int off_b, int off_a,
                  float unit_eps, int dtype, void* stream);

int lv_conv_state_update(const void* proj, int64_t ld, void* conv_state, const int32_t* cu_q,
                         const int32_t* ctx_lens, const int32_t* slots, int B, int C, int taps, int dtype,
                         void* stream);

/* state f32 [slots, H, D, Dv], read unless ctx_lens[b] == 0, written back.  o f32 [T, H, Dv]. */
int lv_gated_delta_rule(const void* qn, const void* kn, const void* v, const void* beta, const void* decay,
                        void* state, const int32_t* cu_q, const int32_t* ctx_lens, const int32_t* slots,
                        void* o, int B, int G, int H, int D, int Dv, void* stream);

/* out act [T, H*Dv] = o / sqrt(mean_dv(o^2) + eps) * norm_w[dv] * silu(gate);  gate act rows of stride ld_gate. */
int lv_head_norm_gate(const void* o, const void* gate, int64_t ld_gate, const void* norm_w, void* out,
                      int64_t T, int H, int Dv, float eps, int dtype, void* stream);

/* q act [T, H*D] (row stride ld), k [T, G*D], v [T, G*Dv] rows of the same stride.  q_out act [T, H*D]
 * contiguous = rms_norm(q over all H*D) * q_w; k likewise into k_cache [pages, page, G, D]; v copied into
 * v_cache [pages, page, G, Dv] at the slot of position ctx_lens[b] + index in the step. */
int lv_qk_fullnorm_store(const void* q, const void* k, const void* v, int64_t ld, const void* q_w,
                         const void* k_w, void* q_out, void* k_cache, void* v_cache, const int32_t* cu_q,
                         const int32_t* ctx_lens, const int32_t* tok_seq, const int32_t* block_tables,
                         int bt_stride, int64_t T, int H, int G, int D, int Dv, int page, float eps, int dtype,
                         void* stream);

/* Pooled entry of block b (positions bP .. bP+P-1) lives with the page of its last token:
 * kp [pages, ceil(page/P), G, D], vp [pages, ceil(page/P), G, Dv], local index b - floor(page*j/P) in page j.
 * Computes the blocks completed by this step; max_new_blocks bounds them per sequence. */
int lv_pool_update(const void* k_cache, const void* v_cache, void* kp, void* vp, const int32_t* cu_q,
                   const int32_t* ctx_lens, const int32_t* block_tables, int bt_stride, int B, int max_new_blocks,
                   int G, int D, int Dv, int page, int P, int dtype, void* stream);

/* Query at position i sees cached positions j with 0 <= i-j < window and every pooled block b with
 * b*P + P - 1 <= i - window (P == 0: no pooled blocks); weights exp(s) / (sink + sum exp(s)) with
 * sink = 1 for has_sink, else 0.  gate (optional) act rows of stride ld_gate: out *= sigmoid(gate).
 * q act [T, H*D] contiguous; out act [T, H*Dv]. */
int lv_window_pool_attn(const void* q, const void* k_cache, const void* v_cache, const void* kp, const void* vp,
                        const void* gate, int64_t ld_gate, void* out, const int32_t* cu_q, const int32_t* ctx_lens,
                        const int32_t* tok_seq, const int32_t* block_tables, int bt_stride, int64_t T, int H, int G,
                        int D, int Dv, int page, int window, int P, float scale, int has_sink, int dtype,
                        void* stream);

/* The same attention on the matrix cores: bf16 only, D and Dv multiples of 16 up to 256. Tiles of 16 new
 * tokens per sequence; max_new_tokens = the largest cu_q[b+1] - cu_q[b] of the step.
 * nsplit > 1 (only with max_new_tokens <= 16, i.e. decode-shaped steps): the key tiles of a sequence are cut over nsplit
 * workgroups whose partials a second kernel merges; workspace: f32 [T, H, nsplit, Dv + 4] (read-out, maximum, sum, padding), T = total new tokens. */
int lv_window_pool_attn_mfma(const void* q, const void* k_cache, const void* v_cache, const void* kp, const void* vp,
                             const void* gate, int64_t ld_gate, void* out, const int32_t* cu_q, const int32_t* ctx_lens,
                             const int32_t* block_tables, int bt_stride, int B, int max_new_tokens, int H, int G, int D,
                             int Dv, int page, int window, int P, float scale, int has_sink, int nsplit, void* workspace,
                             int64_t T, void* stream);

#ifdef __cplusplus
}
#endif
#endif
