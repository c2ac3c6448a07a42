/*
 * CPU oracle for the GQA attention path -- TEST INFRASTRUCTURE, NOT PRODUCT CODE.
 *
 * Only tests, the smoke check and the benchmark's cpu_baseline leg may link or
 * load this library, and only as the checker / reported baseline.  The product
 * (liborin_fa.so) never calls into it.
 *
 * Each function restates, in plain C, what the reference engine's CPU backend
 * computes for attention (reference: src/model_cpu.cpp).  All arithmetic is
 * fp32 in the reference's operation order unless a function says otherwise.
 *
 * KV cache layout everywhere: element (kv_head, pos, i) at
 * (kv_head * n_ctx + pos) * head_dim + i   (reference: src/model_cpu.cpp:277,
 * src/kernels.cu:1675).
 */
#ifndef ORIN_ORACLE_ATTENTION_REF_H
#define ORIN_ORACLE_ATTENTION_REF_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* IEEE binary16 bit pattern -> fp32, exact (reference: src/model_cpu.cpp:49-68). */
float orc_fp16_to_fp32(uint16_t h);

/* fp32 -> binary16 bit pattern, round-to-nearest-even, the rounding the GPU
 * cache writer applies (reference: src/kernels.cu:1676-1677, __float2half). */
uint16_t orc_fp32_to_fp16(float f);

/* Array forms of the two conversions. */
void orc_fp16_to_fp32_n(const uint16_t* src, float* dst, size_t n);
void orc_fp32_to_fp16_n(const float* src, uint16_t* dst, size_t n);

/* Cache writers (reference: src/model_cpu.cpp:276-279 for the fp32 cache,
 * src/kernels.cu:1659-1678 for the fp16 cache).  k, v: [batch][n_kv][head_dim]. */
void orc_kv_store_f32(float* kc, float* vc, const float* k, const float* v,
                      int n_kv, int head_dim, int n_ctx, int pos_base, int batch);
void orc_kv_store_f16(uint16_t* kc, uint16_t* vc, const float* k, const float* v,
                      int n_kv, int head_dim, int n_ctx, int pos_base, int batch);

/* Rolling-window shift (reference: src/model_cpu.cpp:321-338, src/kernels.cu:1682-1700).
 * kc, vc: the whole cache, [n_layer][n_kv][n_ctx][head_dim] 16-bit elements each. */
void orc_kv_shift_u16(uint16_t* kc, uint16_t* vc, int n_layer, int n_kv, int head_dim, int n_ctx,
                      int n_keep, int shift);

/* Rotary position embedding, in place (reference: src/model_cpu.cpp:179-203, call site :264-275).
 * x: [rows][head_dim] with row = token * heads + head; position of a row = n_past + token. */
void orc_rope_neox_row(float* x, int n_rot, float theta, int pos, const float* freq_factors);
void orc_rope_normal_row(float* x, int n_rot, float theta, int pos, const float* freq_factors);
void orc_rope_batch(float* x, int rows, int head_dim, int n_rot, float theta, int n_past, int heads,
                    const float* freq_factors, int neox);

/* One query token against the first npos cache positions
 * (reference: src/model_cpu.cpp:281-295, softmax :20-30, dot :32-36).
 * q, out: [n_head][head_dim].  score: caller scratch of >= npos floats.
 * Loop order is the reference's (PV with the output element outermost). */
void orc_attention_token_f32(const float* q, const float* kc, const float* vc, float* out,
                             int n_head, int n_kv, int head_dim, int n_ctx, int npos,
                             float scale, float* score);
void orc_attention_token_f16(const float* q, const uint16_t* kc, const uint16_t* vc, float* out,
                             int n_head, int n_kv, int head_dim, int n_ctx, int npos,
                             float scale, float* score);

/* One (token, head) output row, same arithmetic and summation order as above
 * (bit-identical result) but with the PV loop position-outermost so it streams
 * the cache.  qh, outh: [head_dim]. */
void orc_attention_row_f16(const float* qh, const uint16_t* kc, const uint16_t* vc, float* outh,
                           int kv_head, int head_dim, int n_ctx, int npos,
                           float scale, float* score);

/* Same call shapes as the operator API (reference: src/kernels.h:77-81).
 * Prefill is the token-at-a-time loop of src/model_cpu.cpp:314-319: token b of
 * the chunk sees positions [0, n_past + b + 1).  The cache must already hold
 * the chunk's own K/V (call-site contract, src/model_gpu.cu:383-384). */
void orc_flash_attention(const float* q, const uint16_t* kc, const uint16_t* vc, float* out,
                         int n_head, int n_kv, int head_dim, int n_ctx, int n_past, int batch,
                         float scale);
void orc_flash_attention_decode_ind(const float* q, const uint16_t* kc, const uint16_t* vc, float* out,
                                    int n_head, int n_kv, int head_dim, int n_ctx, const int* pos,
                                    float scale);

/* Row-sampled prefill: computes only the listed (token, head) rows.
 * rows: n_rows pairs {token, head}; out_rows: [n_rows][head_dim].
 * threads <= 1 runs single-threaded; otherwise rows are spread over OpenMP threads. */
void orc_flash_attention_rows(const float* q, const uint16_t* kc, const uint16_t* vc, float* out_rows,
                              const int* rows, int n_rows,
                              int n_head, int n_kv, int head_dim, int n_ctx, int n_past,
                              float scale, int threads);

/* Number of OpenMP threads the library would use by default. */
int orc_max_threads(void);

#ifdef __cplusplus
}
#endif
#endif
