/*
 * CPU oracle for the decode layer around the attention path -- TEST INFRASTRUCTURE, NOT
 * PRODUCT CODE.  See layer_ref.h.  Built into liborin_oracle.so by oracle/Makefile with the same
 * flags as attention_ref.c (-O3 -ffp-contract=off, no fast-math).
 *
 * How each function is pinned (tests/test_oracle_layer.py):
 *   orc_dequantize_row, orc_gemv, orc_rms_norm, orc_swiglu
 *       bit-exact logits of the unmodified reference CPU build over small synthetic models whose
 *       matrices use every weight type (tests/golden/layer_reference.npz: two layers, projections
 *       with and without bias, with and without per-head q/k norms, tied and untied output
 *       matrix), through oracle/ref.py's decode_forward;
 *   orc_dequantize_row also against an independent whole-array numpy decoding of the same block
 *       formats, and orc_row_bytes against the block sizes (34/144/176/210 bytes).
 */
#include "layer_ref.h"

#include <math.h>
#include <string.h>

#include "attention_ref.h"

enum { kSuper = 256 }; /* elements per block of the three K types */

size_t orc_row_bytes(int type, int64_t n) {
    if (n < 0) return 0;
    switch (type) {
    case ORC_F32: return (size_t)n * 4;
    case ORC_F16: return (size_t)n * 2;
    case ORC_Q8_0: return n % 32 ? 0 : (size_t)(n / 32) * 34;
    case ORC_Q4_K: return n % kSuper ? 0 : (size_t)(n / kSuper) * 144;
    case ORC_Q5_K: return n % kSuper ? 0 : (size_t)(n / kSuper) * 176;
    case ORC_Q6_K: return n % kSuper ? 0 : (size_t)(n / kSuper) * 210;
    default: return 0;
    }
}

static float half_at(const uint8_t* p) {
    uint16_t h;
    memcpy(&h, p, 2);
    return orc_fp16_to_fp32(h);
}

/* The eight 6-bit (scale, min) pairs packed into 12 bytes (reference: src/model_cpu.cpp:38-47):
 * pairs 0..3 sit in the low six bits of bytes j and j + 4; pairs 4..7 take their low four bits from
 * the nibbles of byte j + 4 and their high two from the top bits of bytes j - 4 and j. */
static void unpack_pair(const uint8_t* s, int j, uint8_t* scale, uint8_t* min) {
    if (j < 4) {
        *scale = s[j] & 63;
        *min = s[j + 4] & 63;
    } else {
        *scale = (uint8_t)((s[j + 4] & 0x0f) | ((s[j - 4] >> 6) << 4));
        *min = (uint8_t)((s[j + 4] >> 4) | ((s[j] >> 6) << 4));
    }
}

/* Q4_K block, 144 bytes: d, dmin (fp16), 12 bytes of packed pairs, 128 bytes of nibbles.
 * Element 64 g + e takes the low nibble of byte 32 g + e for e < 32, else the high nibble of
 * byte 32 g + e - 32; its pair is 2 g + (e >= 32).  value = (d * scale) * q - dmin * min
 * (reference: src/model_cpu.cpp:70-89). */
static void decode_q4_k(const uint8_t* b, float* y) {
    const float d = half_at(b), dmin = half_at(b + 2);
    const uint8_t *s = b + 4, *q = b + 16;
    for (int p = 0; p < 8; ++p) {
        uint8_t sc, mn;
        unpack_pair(s, p, &sc, &mn);
        const float dp = d * sc, mp = dmin * mn;
        const uint8_t* qb = q + 32 * (p >> 1);
        for (int e = 0; e < 32; ++e) {
            const int v = (p & 1) ? qb[e] >> 4 : qb[e] & 0x0f;
            y[32 * p + e] = dp * v - mp;
        }
    }
}

/* Q5_K block, 176 bytes: as Q4_K with 32 bytes of fifth bits between the pairs and the nibbles;
 * bit p of byte e is the fifth bit of element 32 p + e (reference: src/model_cpu.cpp:91-113). */
static void decode_q5_k(const uint8_t* b, float* y) {
    const float d = half_at(b), dmin = half_at(b + 2);
    const uint8_t *s = b + 4, *hi = b + 16, *q = b + 48;
    for (int p = 0; p < 8; ++p) {
        uint8_t sc, mn;
        unpack_pair(s, p, &sc, &mn);
        const float dp = d * sc, mp = dmin * mn;
        const uint8_t* qb = q + 32 * (p >> 1);
        for (int e = 0; e < 32; ++e) {
            const int lo = (p & 1) ? qb[e] >> 4 : qb[e] & 0x0f;
            const int v = lo + ((hi[e] >> p) & 1 ? 16 : 0);
            y[32 * p + e] = dp * v - mp;
        }
    }
}

/* Q6_K block, 210 bytes: 128 bytes of low nibbles, 64 bytes of high bit pairs, 16 signed scales,
 * d (fp16).  Per half of 128 elements: element 32 c + l (c = 0..3) has its low nibble in byte
 * l + 32 (c & 1) of the half's 64 (low nibble for c < 2, high for c >= 2), its high two bits at
 * bits 2 c of high byte l, scale index 2 c + l / 16; value = (d * scale) * (q - 32)
 * (reference: src/model_cpu.cpp:115-142). */
static void decode_q6_k(const uint8_t* b, float* y) {
    const float d = half_at(b + 208);
    for (int h = 0; h < 2; ++h) {
        const uint8_t *lo = b + 64 * h, *hi = b + 128 + 32 * h;
        const int8_t* sc = (const int8_t*)(b + 192) + 8 * h;
        for (int c = 0; c < 4; ++c)
            for (int l = 0; l < 32; ++l) {
                const uint8_t byte = lo[l + 32 * (c & 1)];
                const int nib = c < 2 ? byte & 0x0f : byte >> 4;
                const int8_t q = (int8_t)((int8_t)(nib | (((hi[l] >> (2 * c)) & 3) << 4)) - 32);
                y[128 * h + 32 * c + l] = d * sc[2 * c + l / 16] * q;
            }
    }
}

/* Q8_0 block, 34 bytes: d (fp16), 32 signed bytes (reference: src/model_cpu.cpp:144-152). */
static void decode_q8_0(const uint8_t* b, float* y) {
    const float d = half_at(b);
    const int8_t* q = (const int8_t*)(b + 2);
    for (int l = 0; l < 32; ++l) y[l] = d * q[l];
}

int orc_dequantize_row(int type, const void* src, float* y, int64_t k) {
    const uint8_t* b = (const uint8_t*)src;
    switch (type) {
    case ORC_F32: memcpy(y, src, (size_t)k * 4); return 0;
    case ORC_F16:
        for (int64_t i = 0; i < k; ++i) y[i] = half_at(b + 2 * i);
        return 0;
    case ORC_Q8_0:
        for (int64_t i = 0; i < k / 32; ++i) decode_q8_0(b + 34 * i, y + 32 * i);
        return 0;
    case ORC_Q4_K:
        for (int64_t i = 0; i < k / kSuper; ++i) decode_q4_k(b + 144 * i, y + kSuper * i);
        return 0;
    case ORC_Q5_K:
        for (int64_t i = 0; i < k / kSuper; ++i) decode_q5_k(b + 176 * i, y + kSuper * i);
        return 0;
    case ORC_Q6_K:
        for (int64_t i = 0; i < k / kSuper; ++i) decode_q6_k(b + 210 * i, y + kSuper * i);
        return 0;
    default: return -1;
    }
}

int orc_gemv(int type, const void* w, const float* x, float* y, int n_in, int n_out, float* row) {
    const size_t rb = orc_row_bytes(type, n_in);
    if (rb == 0) return -1;
    for (int j = 0; j < n_out; ++j) {
        orc_dequantize_row(type, (const uint8_t*)w + (size_t)j * rb, row, n_in);
        float s = 0.0f;
        for (int i = 0; i < n_in; ++i) s += row[i] * x[i];
        y[j] = s;
    }
    return 0;
}

void orc_rms_norm(const float* x, const float* w, int n, float eps, float* y) {
    double ss = 0.0;
    for (int i = 0; i < n; ++i) ss += (double)x[i] * x[i];
    const double r = 1.0 / sqrt(ss / n + eps);
    for (int i = 0; i < n; ++i) y[i] = (float)(x[i] * r * w[i]);
}

void orc_swiglu(float* act, const float* gate, const float* up, int n) {
    for (int i = 0; i < n; ++i) {
        const float g = gate[i];
        act[i] = g / (1.0f + expf(-g)) * up[i];
    }
}
