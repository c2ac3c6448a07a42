/*
 * orin_layer -- C ABI of the decode layer around the attention path on MI355X (gfx950): the
 * operators the orin_llm engine's decode_layer calls between its attention calls (reference:
 * src/model_gpu.cu:251-293, captured as a graph by :295-316), and one call that runs a whole
 * layer in six launches.  Part of liborin_fa.so; conventions as in orin_fa.h (device pointers
 * owned by the caller, asynchronous launches on the stream of orin_fa_set_stream, process-global
 * state, 0 or a negative ORIN_FA_E_* code).  Nothing here allocates or synchronises: every entry
 * point may run under stream capture.
 *
 * Weight matrices are GGUF tensors as the reference maps them (reference: src/common.h:47-77,
 * src/quant.h:14-45): `type` is the ggml type number (0 F32, 1 F16, 8 Q8_0, 12 Q4_K, 13 Q5_K,
 * 14 Q6_K), a matrix is n_out rows of n_in elements, rows packed back to back.
 * Limits: n_in a multiple of 32 (256 for the K types), at most 32768; matrices of type F32, F16,
 * Q4_K, Q5_K 16-byte aligned (2 bytes for Q8_0 and Q6_K, whose blocks are 34 and 210 bytes);
 * activations and norm weights 16-byte aligned; outputs and biases plain float arrays (4-byte aligned).
 * ORIN_FA_E_INVALID otherwise.  orin_decode_layer checks all seven of its matrices against these limits
 * before its first launch.
 *
 * Arithmetic: the reference's GPU operators round the activation to int8 in blocks of 32 before a
 * product (quantize_activation + dp4a).  These keep it at fp32 precision (as fp32, or as three int8
 * digits of a 24-bit integer per sub-block on the matrix cores) and use the weights' exact values as the
 * reference's CPU backend decodes them (src/model_cpu.cpp:70-167), so results agree with that backend up to
 * the order of an fp32 sum.
 */
#ifndef ORIN_LAYER_H
#define ORIN_LAYER_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum { ORIN_F32 = 0, ORIN_F16 = 1, ORIN_Q8_0 = 8, ORIN_Q4_K = 12, ORIN_Q5_K = 13, ORIN_Q6_K = 14 };

/* Bytes of a row of n elements of the given type; 0 for an unknown type or a partial block
 * (reference: tensor_nbytes, src/common.h:72-77). */
size_t orin_row_bytes(int type, int n);

/* Replaces llm::cuda::rms_norm and rms_norm_rows (reference: src/kernels.h:43-44,
 * src/kernels.cu:1596-1617, 2029-2039): y = x / sqrt(mean(x^2) + eps) * w, per row of `cols` elements with
 * one weight vector for all rows.  y may be x. */
int orin_rms_norm(const float* x, const float* w, int n, float eps, float* y);
int orin_rms_norm_rows(const float* x, const float* w, int rows, int cols, float eps, float* y);

/* Replaces llm::cuda::quantize_activation (reference: src/kernels.h:15, src/kernels.cu:136-157, 1778-1784).
 * The reference stores an int8 copy of x for the *_q8 products that follow; this stores an fp32
 * copy (n_in <= 32768, the longest row the products take) in the library's own device
 * memory, so that those products see x as it was at this call, as they do in the reference. */
int orin_quantize_activation(const float* x, int n_in);

/* Replace llm::cuda::gemv_q8 / gemv_q8_bias / gemv_q8_add (reference: src/kernels.h:21-27,
 * src/kernels.cu:1786-1806, 1825-1836): y = W xs, y = W xs + bias, y += W xs, with xs the activation of the
 * last orin_quantize_activation call, of which a product over n_in elements reads the first n_in (as the
 * reference's do: its decode_layer stages n_embd elements of the attention output and multiplies by wo, whose
 * rows have n_head * head_dim, src/model_gpu.cu:284-285); a product longer than what was staged is refused.
 * The accumulating form may add a row's sum to y in several shares with atomic adds (long rows of a matrix with
 * few rows): y must be written by nothing else while the launch runs, and the order in which a row's shares are
 * added is not fixed, so the last bits of y may differ from run to run and between replays of one graph (the
 * reference's gemv_q8_add is a plain sum, src/kernels.cu:350-374).  orin_gemv_row_shares(1) switches the shares
 * off: y is then bit for bit the same on every run. */
int orin_gemv_q8(int type, const void* W, float* y, int n_in, int n_out);
int orin_gemv_q8_bias(int type, const void* W, const float* bias, float* y, int n_in, int n_out);
int orin_gemv_q8_add(int type, const void* W, float* y, int n_in, int n_out);

/* Replaces llm::cuda::gemv_fused_gate_up_swiglu (reference: src/kernels.h:33-34,
 * src/kernels.cu:1944-1954): out[i] = silu(Wg[i] . xs) * (Wu[i] . xs), both matrices of `type`. */
int orin_gemv_fused_gate_up_swiglu(int type, const void* Wg, const void* Wu, float* out, int n_in, int n_out);

/* Replaces llm::cuda::gemv (reference: src/kernels.h:18, src/kernels.cu:1808-1823): y = W x with x
 * given directly (the output matrix behind the last norm). */
int orin_gemv(int type, const void* W, const float* x, float* y, int n_in, int n_out);

/* Replaces llm::cuda::dequant_row (reference: src/kernels.h:38, src/kernels.cu:1572-1585, 2004-2014): one
 * weight row of n elements to fp32 (the token's embedding), bit for bit what the reference's CPU
 * backend decodes. */
int orin_dequant_row(int type, const void* src, float* y, int n);

/* Replaces llm::cuda::swiglu (reference: src/kernels.h:47, src/kernels.cu:1702-1707, 2041-2044):
 * act[i] = silu(gate[i]) * up[i]. */
int orin_swiglu(float* act, const float* gate, const float* up, int n);

/* Products over the block types (Q4_K, Q5_K, Q6_K, Q8_0) run on the matrix cores where the row length is a
 * multiple of 256 (the activation carried as three int8 digits per sub-block, integer matrix instructions, the
 * blocks' scales applied in fp32) and on the vector ALU otherwise, as F16 and F32 always do.  on = 0 keeps
 * everything on the vector ALU: for comparisons and tests; the results agree to the order of an fp32 sum. */
void orin_gemv_use_matrix_cores(int on);

/* How many shares an accumulating projection (y += W x: orin_gemv_q8_add, orin_gemv_multi with accumulate,
 * the output and down projections of orin_decode_layer) may cut a row into: 0 (default) = the launcher
 * chooses 1, 2 or 4 by shape, which is fastest and leaves the order of a row's adds open (see orin_gemv_q8_add);
 * 1 = never cut, every result bit for bit reproducible, at 1-2 us more per projection on small models; 2, 4 = forced
 * (tuning).  Takes effect with the next launch; graphs captured earlier keep the launches they recorded.
 * ORIN_GEMV_KSPLIT in the environment sets the initial value. */
void orin_gemv_row_shares(int shares);

/* ---- forms with no counterpart in the reference: fewer launches per layer ---- */

/* Up to three matrices of one type over the same activation in one launch (the q, k, v
 * projections), the RMS norm folded in: y_m = W_m norm(x) + bias_m, with
 * norm(x) = x / sqrt(mean(x^2) + eps) * norm_w computed by every workgroup for itself (norm_w NULL:
 * no norm), bias_m NULL: none.  accumulate != 0: y_m += instead. */
int orin_gemv_multi(int type, int n_mat, const void* const* W, const float* const* bias, float* const* y,
                    const int* n_out, const float* x, const float* norm_w, float eps, int n_in, int accumulate);

/* The same with a type per matrix (a file that keeps attn_v in Q6_K beside Q4_K projections): one launch
 * where every type is Q4_K or Q6_K, one launch per matrix otherwise. */
int orin_gemv_multi_types(const int* types, int n_mat, const void* const* W, const float* const* bias, float* const* y,
                          const int* n_out, const float* x, const float* norm_w, float eps, int n_in);

/* out[i] = silu(Wg[i] . norm(x)) * (Wu[i] . norm(x)): the layer's second norm and its gate/up pair in
 * one launch. */
int orin_gemv_norm_gate_up_swiglu(int type, const void* Wg, const void* Wu, const float* x, const float* norm_w,
                                  float eps, float* out, int n_in, int n_out);

/* One decode layer (reference: src/model_gpu.cu:251-293), six launches where the types allow:
 *   [attn_norm + q, k, v projections (+ bias)]  [per-head q/k norms, if the model has them]
 *   [rotary embedding + cache store + attention: orin_fa_decode_rope_store_ind, two launches]
 *   [output projection, added to x]  [ffn_norm + gate/up + SwiGLU]  [down projection, added to x]
 * Projections of different types take a launch each; a rotary layout the fused attention call does
 * not take (NeoX pairing with n_rot < head_dim) goes through the separate rope and store calls.
 * x is updated in place; q, k, v, attn, act (and up_tmp, needed only when ffn_gate and ffn_up
 * differ in type) are scratch the caller provides; k and v leave un-rotated / as projected.
 * The two projections that add into x may cut their rows into shares that meet by atomic adds, so x can differ
 * in its last bits between runs and between replays of a captured layer unless orin_gemv_row_shares(1) was
 * called before the launches (or the capture).
 * A descriptor with a missing pointer or a non-positive size returns ORIN_FA_E_INVALID before
 * anything is launched; shapes a kernel cannot take are refused by the launch that meets them. */
typedef struct orin_decode_layer_desc {
    int n_embd, n_head, n_kv, head_dim, n_ff, n_ctx, n_rot, neox;
    float rms_eps, rope_theta, scale;
    int wq_type, wk_type, wv_type, wo_type, gate_type, up_type, down_type;
    const void *wq, *wk, *wv, *wo, *ffn_gate, *ffn_up, *ffn_down;
    const float *attn_norm, *ffn_norm;
    const float *q_norm, *k_norm;   /* [head_dim] each, or NULL */
    const float *bq, *bk, *bv;      /* or NULL */
    const float* freq_factors;      /* [n_rot / 2], or NULL */
    const float* rope_angles;       /* table of orin_fa_rope_angles_ind for this token, or NULL */
    uint16_t *kc, *vc;              /* this layer's cache */
    float* x;                       /* [n_embd] */
    float *q, *k, *v;               /* [n_head * head_dim], [n_kv * head_dim] twice */
    float* attn;                    /* [n_head * head_dim] */
    float* act;                     /* [n_ff] */
    float* up_tmp;                  /* [n_ff], or NULL */
    const int* d_pos;
} orin_decode_layer_desc;
int orin_decode_layer(const orin_decode_layer_desc* layer);

#ifdef __cplusplus
}
#endif
#endif
