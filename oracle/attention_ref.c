/*
 * CPU oracle for the GQA attention path -- TEST INFRASTRUCTURE, NOT PRODUCT CODE.
 * See attention_ref.h.  Build: make -C oracle   (gcc -O3 -ffp-contract=off, no
 * fast-math, matching the reference's CPU flags in src/Makefile:2 so that the
 * fp32 operation order below is what the machine executes).
 *
 * How each function is pinned (tests/test_oracle_*.py):
 *   orc_fp16_to_fp32 / orc_fp32_to_fp16   all 65,536 patterns / 2^24 sampled floats vs numpy float16
 *   orc_attention_token_f32               bit-exact logits of the unmodified reference CPU build
 *                                         (tests/golden/cfg1_*.npz) + float64 closed form
 *   orc_attention_token_f16, _row_f16     bit-equal to _f32 on fp16-representable caches + float64 closed form
 *   orc_flash_attention*, _rows           composition of the above, checked against the same fixtures
 *   orc_kv_store_*                        exact against numpy astype(float16) at the documented offset
 *   orc_kv_shift_u16                      exact against the slice statement new[keep:n-s] = old[keep+s:], tail 0
 *   orc_rope_*                            bit-exact logits of the unmodified reference CPU build run with its rotary
 *                                         embedding on (tests/golden/rope_reference.npz: NeoX and adjacent pairs,
 *                                         frequency factors, n_rot < head_dim, positions near 0 and near 32768);
 *                                         float64 rotation by the same fp32 angle; neox == permuted normal, bit for
 *                                         bit; position 0 is the identity; elements past n_rot untouched
 */
#include "attention_ref.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

/* ---- binary16 <-> binary32 ------------------------------------------------ */

float orc_fp16_to_fp32(uint16_t h) {
    const uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    const uint32_t exp = (h >> 10) & 0x1fu;
    const uint32_t man = h & 0x3ffu;
    uint32_t bits;
    if (exp == 0) {
        /* zero or subnormal: man * 2^-24, exactly representable in fp32 */
        float f = (float)man * 0x1.0p-24f;
        memcpy(&bits, &f, 4);
        bits |= sign;
    } else if (exp == 31) {
        bits = sign | 0x7f800000u | (man << 13);
    } else {
        bits = sign | ((exp + 112u) << 23) | (man << 13);
    }
    float out;
    memcpy(&out, &bits, 4);
    return out;
}

uint16_t orc_fp32_to_fp16(float f) {
    uint32_t x;
    memcpy(&x, &f, 4);
    const uint16_t sign = (uint16_t)((x >> 16) & 0x8000u);
    const uint32_t ax = x & 0x7fffffffu;
    if (ax >= 0x7f800000u) { /* inf / nan */
        if (ax == 0x7f800000u) return (uint16_t)(sign | 0x7c00u);
        return (uint16_t)(sign | 0x7e00u | ((ax >> 13) & 0x3ffu)); /* quiet nan, keep payload top bits */
    }
    if (ax >= 0x477ff000u) { /* >= 65520 rounds to inf */
        return (uint16_t)(sign | 0x7c00u);
    }
    if (ax < 0x38800000u) { /* below the smallest normal half (2^-14): subnormal or zero */
        if (ax < 0x33000000u) { /* < 2^-25: rounds to zero (2^-25 itself ties to even = 0) */
            return sign;
        }
        /* value = m * 2^(e-150) with implicit bit; target unit is 2^-24 */
        const uint32_t e = ax >> 23;
        const uint32_t m = (ax & 0x7fffffu) | 0x800000u;
        const uint32_t shift = 126u - e; /* 14..24: m >> shift is the count of 2^-24 units */
        uint32_t q = m >> shift;
        const uint32_t rem = m & ((1u << shift) - 1u);
        const uint32_t half = 1u << (shift - 1u);
        if (rem > half || (rem == half && (q & 1u))) q++;
        return (uint16_t)(sign | q);
    }
    /* normal range */
    uint32_t e = (ax >> 23) - 112u;
    uint32_t m = ax & 0x7fffffu;
    uint32_t q = (e << 10) | (m >> 13);
    const uint32_t rem = m & 0x1fffu;
    if (rem > 0x1000u || (rem == 0x1000u && (q & 1u))) q++; /* carry may bump the exponent: still correct */
    return (uint16_t)(sign | q);
}

void orc_fp16_to_fp32_n(const uint16_t* src, float* dst, size_t n) {
    for (size_t i = 0; i < n; ++i) dst[i] = orc_fp16_to_fp32(src[i]);
}

void orc_fp32_to_fp16_n(const float* src, uint16_t* dst, size_t n) {
    for (size_t i = 0; i < n; ++i) dst[i] = orc_fp32_to_fp16(src[i]);
}

/* ---- cache writers ---------------------------------------------------------- */

void orc_kv_store_f32(float* kc, float* vc, const float* k, const float* v,
                      int n_kv, int head_dim, int n_ctx, int pos_base, int batch) {
    for (int b = 0; b < batch; ++b)
        for (int h = 0; h < n_kv; ++h) {
            const size_t dst = ((size_t)h * n_ctx + (size_t)(pos_base + b)) * head_dim;
            const size_t src = ((size_t)b * n_kv + h) * head_dim;
            memcpy(kc + dst, k + src, sizeof(float) * (size_t)head_dim);
            memcpy(vc + dst, v + src, sizeof(float) * (size_t)head_dim);
        }
}

void orc_kv_store_f16(uint16_t* kc, uint16_t* vc, const float* k, const float* v,
                      int n_kv, int head_dim, int n_ctx, int pos_base, int batch) {
    for (int b = 0; b < batch; ++b)
        for (int h = 0; h < n_kv; ++h) {
            const size_t dst = ((size_t)h * n_ctx + (size_t)(pos_base + b)) * head_dim;
            const size_t src = ((size_t)b * n_kv + h) * head_dim;
            orc_fp32_to_fp16_n(k + src, kc + dst, (size_t)head_dim);
            orc_fp32_to_fp16_n(v + src, vc + dst, (size_t)head_dim);
        }
}

/* Rolling-window shift of the whole cache (reference: src/model_cpu.cpp:321-338, which
 * states it on the CPU backend's fp32 cache; the device cache holds 16-bit elements,
 * src/kernels.cu:1682-1700): per layer and head, rows [n_keep + shift, n_ctx) move to
 * [n_keep, n_ctx - shift) and the last `shift` rows are cleared. */
void orc_kv_shift_u16(uint16_t* kc, uint16_t* vc, int n_layer, int n_kv, int head_dim, int n_ctx,
                      int n_keep, int shift) {
    const size_t d = (size_t)head_dim;
    const size_t per_layer = (size_t)n_kv * n_ctx * d;
    for (int l = 0; l < n_layer; ++l)
        for (int h = 0; h < n_kv; ++h) {
            uint16_t* kh = kc + l * per_layer + (size_t)h * n_ctx * d;
            uint16_t* vh = vc + l * per_layer + (size_t)h * n_ctx * d;
            memmove(kh + n_keep * d, kh + (n_keep + shift) * d, (size_t)(n_ctx - n_keep - shift) * d * sizeof(uint16_t));
            memmove(vh + n_keep * d, vh + (n_keep + shift) * d, (size_t)(n_ctx - n_keep - shift) * d * sizeof(uint16_t));
            memset(kh + (size_t)(n_ctx - shift) * d, 0, (size_t)shift * d * sizeof(uint16_t));
            memset(vh + (size_t)(n_ctx - shift) * d, 0, (size_t)shift * d * sizeof(uint16_t));
        }
}

/* ---- rotary position embedding ------------------------------------------------ */

/* One head row (reference: src/model_cpu.cpp:179-190 and :193-203).  std::pow, std::cos and
 * std::sin on float arguments are the float overloads. */
void orc_rope_neox_row(float* x, int n_rot, float theta, int pos, const float* freq_factors) {
    const int half = n_rot / 2;
    for (int i = 0; i < half; ++i) {
        float freq = powf(theta, -2.0f * i / n_rot);
        if (freq_factors) freq /= freq_factors[i];
        const float ang = (float)pos * freq;
        const float c = cosf(ang), s = sinf(ang);
        const float x0 = x[i], x1 = x[i + half];
        x[i] = x0 * c - x1 * s;
        x[i + half] = x0 * s + x1 * c;
    }
}

void orc_rope_normal_row(float* x, int n_rot, float theta, int pos, const float* freq_factors) {
    for (int i = 0; i < n_rot; i += 2) {
        float freq = powf(theta, -1.0f * i / n_rot);
        if (freq_factors) freq /= freq_factors[i / 2];
        const float ang = (float)pos * freq;
        const float c = cosf(ang), s = sinf(ang);
        const float x0 = x[i], x1 = x[i + 1];
        x[i] = x0 * c - x1 * s;
        x[i + 1] = x0 * s + x1 * c;
    }
}

/* All rows of a chunk: row = token * heads + head, position n_past + token (the loop of
 * src/model_cpu.cpp:264-275 over heads, run token by token as :314-319 does). */
void orc_rope_batch(float* x, int rows, int head_dim, int n_rot, float theta, int n_past, int heads,
                    const float* freq_factors, int neox) {
    for (int r = 0; r < rows; ++r) {
        const int pos = n_past + r / heads;
        if (neox) orc_rope_neox_row(x + (size_t)r * head_dim, n_rot, theta, pos, freq_factors);
        else orc_rope_normal_row(x + (size_t)r * head_dim, n_rot, theta, pos, freq_factors);
    }
}

/* ---- attention -------------------------------------------------------------- */

/* fp32 sequential dot product (reference: src/model_cpu.cpp:32-36). */
static float dot_f32(const float* a, const float* b, int n) {
    float s = 0.0f;
    for (int i = 0; i < n; ++i) s += a[i] * b[i];
    return s;
}

/* In-place softmax: max, expf, running fp32 sum, multiply by 1/sum
 * (reference: src/model_cpu.cpp:20-30). */
static void softmax_f32(float* x, int n) {
    float m = x[0];
    for (int i = 1; i < n; ++i) m = x[i] > m ? x[i] : m;
    float sum = 0.0f;
    for (int i = 0; i < n; ++i) {
        x[i] = expf(x[i] - m);
        sum += x[i];
    }
    const float inv = 1.0f / sum;
    for (int i = 0; i < n; ++i) x[i] *= inv;
}

void orc_attention_token_f32(const float* q, const float* kc, const float* vc, float* out,
                             int n_head, int n_kv, int head_dim, int n_ctx, int npos,
                             float scale, float* score) {
    const int d = head_dim;
    for (int h = 0; h < n_head; ++h) {
        const int kv = h * n_kv / n_head; /* GQA map, src/model_cpu.cpp:283 */
        const float* qh = q + (size_t)h * d;
        const float* kh = kc + (size_t)kv * n_ctx * d;
        const float* vh = vc + (size_t)kv * n_ctx * d;
        for (int j = 0; j < npos; ++j) score[j] = scale * dot_f32(qh, kh + (size_t)j * d, d);
        softmax_f32(score, npos);
        float* oh = out + (size_t)h * d;
        for (int jd = 0; jd < d; ++jd) {
            float s = 0.0f;
            for (int j = 0; j < npos; ++j) s += score[j] * vh[(size_t)j * d + jd];
            oh[jd] = s;
        }
    }
}

void orc_attention_token_f16(const float* q, const uint16_t* kc, const uint16_t* vc, float* out,
                             int n_head, int n_kv, int head_dim, int n_ctx, int npos,
                             float scale, float* score) {
    const int d = head_dim;
    float krow[512];
    for (int h = 0; h < n_head; ++h) {
        const int kv = h * n_kv / n_head;
        const float* qh = q + (size_t)h * d;
        const uint16_t* kh = kc + (size_t)kv * n_ctx * d;
        const uint16_t* vh = vc + (size_t)kv * n_ctx * d;
        for (int j = 0; j < npos; ++j) {
            orc_fp16_to_fp32_n(kh + (size_t)j * d, krow, (size_t)d);
            score[j] = scale * dot_f32(qh, krow, d);
        }
        softmax_f32(score, npos);
        float* oh = out + (size_t)h * d;
        for (int jd = 0; jd < d; ++jd) {
            float s = 0.0f;
            for (int j = 0; j < npos; ++j) s += score[j] * orc_fp16_to_fp32(vh[(size_t)j * d + jd]);
            oh[jd] = s;
        }
    }
}

void orc_attention_row_f16(const float* qh, const uint16_t* kc, const uint16_t* vc, float* outh,
                           int kv_head, int head_dim, int n_ctx, int npos,
                           float scale, float* score) {
    const int d = head_dim;
    float row[512];
    const uint16_t* kh = kc + (size_t)kv_head * n_ctx * d;
    const uint16_t* vh = vc + (size_t)kv_head * n_ctx * d;
    for (int j = 0; j < npos; ++j) {
        orc_fp16_to_fp32_n(kh + (size_t)j * d, row, (size_t)d);
        score[j] = scale * dot_f32(qh, row, d);
    }
    softmax_f32(score, npos);
    /* Each outh[jd] still receives its products in ascending j, one add at a time,
     * so the value is bit-identical to the output-outermost loop. */
    for (int jd = 0; jd < d; ++jd) outh[jd] = 0.0f;
    for (int j = 0; j < npos; ++j) {
        orc_fp16_to_fp32_n(vh + (size_t)j * d, row, (size_t)d);
        const float p = score[j];
        for (int jd = 0; jd < d; ++jd) outh[jd] += p * row[jd];
    }
}

void orc_flash_attention(const float* q, const uint16_t* kc, const uint16_t* vc, float* out,
                         int n_head, int n_kv, int head_dim, int n_ctx, int n_past, int batch,
                         float scale) {
    float* score = (float*)malloc(sizeof(float) * (size_t)(n_past + batch > 0 ? n_past + batch : 1));
    for (int b = 0; b < batch; ++b) {
        orc_attention_token_f16(q + (size_t)b * n_head * head_dim, kc, vc,
                                out + (size_t)b * n_head * head_dim,
                                n_head, n_kv, head_dim, n_ctx, n_past + b + 1, scale, score);
    }
    free(score);
}

void orc_flash_attention_decode_ind(const float* q, const uint16_t* kc, const uint16_t* vc, float* out,
                                    int n_head, int n_kv, int head_dim, int n_ctx, const int* pos,
                                    float scale) {
    const int npos = *pos + 1; /* src/model_cpu.cpp:281; GPU side reads it on device, src/kernels.cu:1127 */
    float* score = (float*)malloc(sizeof(float) * (size_t)npos);
    orc_attention_token_f16(q, kc, vc, out, n_head, n_kv, head_dim, n_ctx, npos, scale, score);
    free(score);
}

void orc_flash_attention_rows(const float* q, const uint16_t* kc, const uint16_t* vc, float* out_rows,
                              const int* rows, int n_rows,
                              int n_head, int n_kv, int head_dim, int n_ctx, int n_past,
                              float scale, int threads) {
    int max_npos = 1;
    for (int r = 0; r < n_rows; ++r) {
        const int np = n_past + rows[2 * r] + 1;
        if (np > max_npos) max_npos = np;
    }
#ifdef _OPENMP
    if (threads < 1) threads = 1;
#pragma omp parallel num_threads(threads)
#endif
    {
        float* score = (float*)malloc(sizeof(float) * (size_t)max_npos);
#ifdef _OPENMP
#pragma omp for schedule(dynamic, 1)
#endif
        for (int r = 0; r < n_rows; ++r) {
            const int tok = rows[2 * r], h = rows[2 * r + 1];
            const int kv = h * n_kv / n_head;
            orc_attention_row_f16(q + ((size_t)tok * n_head + h) * head_dim, kc, vc,
                                  out_rows + (size_t)r * head_dim, kv, head_dim, n_ctx,
                                  n_past + tok + 1, scale, score);
        }
        free(score);
    }
    (void)threads;
}

int orc_max_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}
