// The small operators of the decode layer around attention for gfx950 (MI355X): RMS norm over a
// vector or over the rows of a matrix, the staging copy behind quantize_activation, and the
// decoding of one weight row (the token embedding).
//
// Replaces the reference's rms_norm_k / rms_norm_rows_k, quantize_q8_1_k and dequant_row_k with
// their launchers (reference: src/kernels.cu:133-205, 1570-1617, 2004-2013, 2029-2040).  All
// of them are launch-bound: a few kilobytes each.
#include "layer_common.hpp"

namespace orin_fa {
namespace {

// y = x / sqrt(mean(x^2) + eps) * w over each row of cols elements (reference CPU statement:
// src/model_cpu.cpp:13-18; w is shared by the rows).  One workgroup per row; y may be x: a thread
// writes only elements it has read itself.
template <int THREADS>
__global__ __launch_bounds__(THREADS) void rms_norm_kernel(const float* x, const float* __restrict__ w, int cols,
                                                            float eps, float* y) {
    __shared__ float sh[THREADS / 64];
    const float* xr = x + (size_t)blockIdx.x * cols;
    float* yr = y + (size_t)blockIdx.x * cols;
    float ss = 0.0f;
    for (int i = threadIdx.x; i < cols; i += THREADS) ss += xr[i] * xr[i];
    ss = wave_sum(ss);
    if constexpr (THREADS > 64) {
        if ((threadIdx.x & 63) == 0) sh[threadIdx.x >> 6] = ss;
        __syncthreads();
        ss = 0.0f;
#pragma unroll
        for (int k = 0; k < THREADS / 64; ++k) ss += sh[k];
    }
    const float rinv = 1.0f / sqrtf(ss / (float)cols + eps);
    for (int i = threadIdx.x; i < cols; i += THREADS) yr[i] = xr[i] * rinv * w[i];
}

__global__ __launch_bounds__(256) void stage_kernel(const float* __restrict__ x, float* __restrict__ stage, int n) {
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i < n) stage[i] = x[i];
}

// act = SiLU(gate) * up (reference CPU statement: src/model_cpu.cpp:11,302).
__global__ __launch_bounds__(256) void swiglu_kernel(float* act, const float* gate, const float* up, int n) {
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i < n) {
        const float g = gate[i];
        act[i] = g / (1.0f + expf(-g)) * up[i];
    }
}

__device__ __forceinline__ float half_at(const unsigned char* p) {
    return (float)__builtin_bit_cast(_Float16, *reinterpret_cast<const uint16_t*>(p));
}

__device__ __forceinline__ void pair_at(const unsigned char* s, int p, unsigned& sc, unsigned& mn) {
    if (p < 4) {
        sc = s[p] & 63u;
        mn = s[p + 4] & 63u;
    } else {
        sc = (s[p + 4] & 0x0fu) | ((unsigned)(s[p - 4] >> 6) << 4);
        mn = (unsigned)(s[p + 4] >> 4) | ((unsigned)(s[p] >> 6) << 4);
    }
}

// Element e of a row, decoded exactly as the reference's CPU backend decodes it
// (reference: src/model_cpu.cpp:70-167; block layouts src/quant.h:14-45).
__device__ float decode_element(int type, const unsigned char* row, int e) {
    switch (type) {
    case kF32: return reinterpret_cast<const float*>(row)[e];
    case kF16: return half_at(row + 2 * (size_t)e);
    case kQ8_0: {
        const unsigned char* b = row + (size_t)(e >> 5) * 34;
        return half_at(b) * (float)reinterpret_cast<const signed char*>(b + 2)[e & 31];
    }
    case kQ4_K:
    case kQ5_K: {
        const bool five = type == kQ5_K;
        const unsigned char* b = row + (size_t)(e >> 8) * (five ? 176 : 144);
        const int i = e & 255, p = i >> 5, l = i & 31;
        unsigned sc, mn;
        pair_at(b + 4, p, sc, mn);
        const unsigned char byte = b[(five ? 48 : 16) + 32 * (p >> 1) + l];
        int q = (p & 1) ? byte >> 4 : byte & 0x0f;
        if (five) q += ((b[16 + l] >> p) & 1) ? 16 : 0;
        const float d = half_at(b), dmin = half_at(b + 2);
        return (d * (float)sc) * (float)q - dmin * (float)mn;
    }
    case kQ6_K: {
        const unsigned char* b = row + (size_t)(e >> 8) * 210;
        const int i = e & 255, h = i >> 7, c = (i >> 5) & 3, l = i & 31;
        const unsigned char byte = b[64 * h + l + 32 * (c & 1)];
        const int nib = c < 2 ? byte & 0x0f : byte >> 4;
        const int q = (nib | (((b[128 + 32 * h + l] >> (2 * c)) & 3) << 4)) - 32;
        const float scale = (float)reinterpret_cast<const signed char*>(b + 192)[8 * h + 2 * c + l / 16];
        return half_at(b + 208) * scale * (float)q;
    }
    default: return 0.0f;
    }
}

__global__ __launch_bounds__(256) void dequant_row_kernel(int type, const unsigned char* __restrict__ src,
                                                          float* __restrict__ y, int n) {
#pragma clang fp contract(off)
    const int e = blockIdx.x * 256 + threadIdx.x;
    if (e < n) y[e] = decode_element(type, src, e);
}

} // namespace

hipError_t rms_norm_launch(const float* x, const float* w, int rows, int cols, float eps, float* y, hipStream_t stream) {
    drop_stale_error();
    if (cols <= 256)
        hipLaunchKernelGGL((rms_norm_kernel<64>), dim3(rows), dim3(64), 0, stream, x, w, cols, eps, y);
    else
        hipLaunchKernelGGL((rms_norm_kernel<1024>), dim3(rows), dim3(1024), 0, stream, x, w, cols, eps, y);
    return hipGetLastError();
}

hipError_t stage_launch(const float* x, float* stage, int n, hipStream_t stream) {
    drop_stale_error();
    hipLaunchKernelGGL(stage_kernel, dim3((n + 255) / 256), dim3(256), 0, stream, x, stage, n);
    return hipGetLastError();
}

hipError_t swiglu_launch(float* act, const float* gate, const float* up, int n, hipStream_t stream) {
    drop_stale_error();
    hipLaunchKernelGGL(swiglu_kernel, dim3((n + 255) / 256), dim3(256), 0, stream, act, gate, up, n);
    return hipGetLastError();
}

hipError_t dequant_row_launch(int type, const void* src, float* y, int n, hipStream_t stream) {
    drop_stale_error();
    hipLaunchKernelGGL(dequant_row_kernel, dim3((n + 255) / 256), dim3(256), 0, stream, type,
                       static_cast<const unsigned char*>(src), y, n);
    return hipGetLastError();
}

} // namespace orin_fa
