/*
 * CPU oracle for the decode layer around the attention path -- TEST INFRASTRUCTURE, NOT
 * PRODUCT CODE.  Only tests, the smoke check and the benchmark's cpu_baseline leg may link or
 * load this library, and only as the checker / reported baseline.
 *
 * Restates, in plain C, the pieces of the reference CPU backend's forward pass that surround
 * attention (reference: src/model_cpu.cpp:11-18 silu and rms_norm, :38-47 scale unpacking,
 * :70-167 block decoders, :169-177 gemv, :299-304 the feed-forward block).  All arithmetic is
 * fp32 in the reference's operation order; the norm's sum of squares is double, as there.
 * The forward pass itself is the sequence of these calls and of attention_ref.h's, written out
 * in oracle/ref.py (decode_forward) after src/model_cpu.cpp:241-312.
 *
 * Weight types carry the reference's numbers (src/common.h:47-54).
 */
#ifndef ORIN_ORACLE_LAYER_REF_H
#define ORIN_ORACLE_LAYER_REF_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum { ORC_F32 = 0, ORC_F16 = 1, ORC_Q8_0 = 8, ORC_Q4_K = 12, ORC_Q5_K = 13, ORC_Q6_K = 14 };

/* Bytes of a row of n elements (reference: src/common.h:61-77); 0 for an unknown type or an n that
 * is not a whole number of blocks. */
size_t orc_row_bytes(int type, int64_t n);

/* One row of k elements to fp32 (reference: src/model_cpu.cpp:70-167).  Returns 0, or -1 for an
 * unknown type. */
int orc_dequantize_row(int type, const void* src, float* y, int64_t k);

/* y[j] = dot(row j of W decoded to fp32, x), the sum taken element by element in fp32
 * (reference: src/model_cpu.cpp:32-36, 169-177).  row: caller scratch of n_in floats. */
int orc_gemv(int type, const void* w, const float* x, float* y, int n_in, int n_out, float* row);

/* y = x / sqrt(mean(x^2) + eps) * w, the mean in double (reference: src/model_cpu.cpp:13-18).
 * y may be x. */
void orc_rms_norm(const float* x, const float* w, int n, float eps, float* y);

/* act[i] = gate[i] / (1 + exp(-gate[i])) * up[i] (reference: src/model_cpu.cpp:11, 302). */
void orc_swiglu(float* act, const float* gate, const float* up, int n);

#ifdef __cplusplus
}
#endif
#endif
