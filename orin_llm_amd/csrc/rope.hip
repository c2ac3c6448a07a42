// Rotary position embedding for gfx950 (MI355X), in place on fp32 rows [rows][head_dim].
//
// Replaces the reference's rope_neox_k / rope_normal_k and their four wrappers (reference:
// src/kernels.cu:1619-1657, 2059-2075; CPU statement src/model_cpu.cpp:179-203; call sites
// src/model_gpu.cu:277-279, 379-381).  Pair i of a row is rotated by the angle pos * freq_i,
// freq_i = theta^(-2i/n_rot) (divided by freq_factors[i] when given); "neox" pairs element i
// with i + n_rot/2, "normal" pairs 2i with 2i + 1; elements at or past n_rot are left alone.
// pos = n_past + row / heads (batch form) or *d_pos (single-token form, read on the device).
//
// Two kernels: rope4_kernel for the shapes models have (n_rot a multiple of 8, 16-byte aligned
// rows), all 128-bit accesses, and rope_kernel for any even n_rot.  In rope_kernel,
// every head of a token shares the token's angles, so one thread owns (token, pair, group of up
// to 8 heads): the block's first threads compute the frequency of each pair once into LDS, each
// thread forms its angle and one sine/cosine, then rotates its heads; all loads are issued
// before any of that arithmetic -- where the reference spends a power, a sine and a cosine per
// element pair of every head.
// Arithmetic (rope_freq, rope_rotate in fa_common.hpp) follows the CPU statement operation by
// operation in fp32.  Sine and cosine are the accurate library versions (full range
// reduction), not the fast hardware approximations the reference's GPU path uses.
#include "fa_common.hpp"

namespace orin_fa {
namespace {

constexpr int kHeadsPerThread = 8;

// The rotated rows and the cache rows are read next by another kernel, on other compute units:
// streaming stores send them on instead of leaving them dirty in this die's cache until the
// kernel ends.
__device__ __forceinline__ void store_stream(float* p, const float4& v) {
    __builtin_nontemporal_store(f4{v.x, v.y, v.z, v.w}, reinterpret_cast<f4*>(p));
}

template <bool NEOX, bool IND>
__global__ __launch_bounds__(256) void rope_kernel(float* x, int tokens, int heads, int head_dim, int n_rot,
                                                   float theta, int n_past, const int* d_pos,
                                                   const float* freq_factors) {
#pragma clang fp contract(off)
    __shared__ float sh_freq[128];
    const int half = n_rot / 2;
    const int n_hgroups = (heads + kHeadsPerThread - 1) / kHeadsPerThread;
    // pair index fastest, then head group, then token; a block covers whole runs of pairs when
    // half divides 256, otherwise every thread computes its own frequency
    const bool shared_freq = half <= 128 && (256 % half) == 0;
    const long long t = (long long)blockIdx.x * 256 + threadIdx.x;
    const bool active = t < (long long)tokens * n_hgroups * half;
    const int i = (int)(t % half);
    const long long th = t / half;
    const int hgroup = (int)(th % n_hgroups), token = (int)(th / n_hgroups);
    const int h0 = hgroup * kHeadsPerThread;
    float* row = x + ((size_t)token * heads + h0) * head_dim;
    const int i0 = NEOX ? i : 2 * i, i1 = NEOX ? i + half : 2 * i + 1;
    // The loads go out first: nothing they need depends on the angle, and the power, sine and
    // cosine below then run while the rows are on their way.
    float x0[kHeadsPerThread], x1[kHeadsPerThread];
#pragma unroll
    for (int u = 0; u < kHeadsPerThread; ++u)
        if (active && h0 + u < heads) {
            x0[u] = row[(size_t)u * head_dim + i0];
            x1[u] = row[(size_t)u * head_dim + i1];
        }
    const int pos = IND ? *d_pos : n_past + token;
    if (shared_freq && (int)threadIdx.x < half) {
        sh_freq[threadIdx.x] = rope_freq(threadIdx.x, n_rot, theta, freq_factors);
    }
    if (shared_freq) __syncthreads();
    if (!active) return;
    float freq;
    if (shared_freq) {
        freq = sh_freq[i];
    } else {
        freq = rope_freq(i, n_rot, theta, freq_factors);
    }
    const float ang = (float)pos * freq;
    const float c = cosf(ang), s = sinf(ang);
#pragma unroll
    for (int u = 0; u < kHeadsPerThread; ++u)
        if (h0 + u < heads) {
            rope_rotate(x0[u], x1[u], c, s);
            row[(size_t)u * head_dim + i0] = x0[u];
            row[(size_t)u * head_dim + i1] = x1[u];
        }
}

// The same rotation for the common shapes (n_rot a multiple of 8, rows 16-byte aligned), moved in
// 16-byte pieces: a thread owns four adjacent pairs of (token, group of up to 4 heads) -- "neox":
// elements 4j..4j+3 and the four n_rot/2 further on; "normal": elements 8j..8j+7 -- so every
// load and store is a full 128-bit access that a wave makes on whole cache lines, all of a
// thread's loads are in flight before its four sines and cosines are formed, and an angle is
// computed once per four heads.  The frequencies come from a table the block's first n_rot/2
// threads fill.  Arithmetic per element as in rope_kernel.
constexpr int kHeadsPerThread4 = 4;

template <bool NEOX, bool IND>
__global__ __launch_bounds__(256) void rope4_kernel(float* x, int tokens, int heads, int head_dim, int n_rot,
                                                    float theta, int n_past, const int* d_pos,
                                                    const float* freq_factors) {
#pragma clang fp contract(off)
    __shared__ float sh_freq[256];
    const int half = n_rot / 2, quads = half / 4;
    const int n_hgroups = (heads + kHeadsPerThread4 - 1) / kHeadsPerThread4;
    const long long t = (long long)blockIdx.x * 256 + threadIdx.x;
    const bool active = t < (long long)tokens * n_hgroups * quads;
    const int qi = (int)(t % quads);
    const long long th = t / quads;
    const int hgroup = (int)(th % n_hgroups), token = (int)(th / n_hgroups);
    const int h0 = hgroup * kHeadsPerThread4;
    float* row = x + ((size_t)token * heads + h0) * head_dim;
    const int o0 = NEOX ? 4 * qi : 8 * qi, o1 = NEOX ? 4 * qi + half : 8 * qi + 4;
    float4 a[kHeadsPerThread4], b[kHeadsPerThread4];
#pragma unroll
    for (int u = 0; u < kHeadsPerThread4; ++u)
        if (active && h0 + u < heads) {
            a[u] = *reinterpret_cast<const float4*>(row + (size_t)u * head_dim + o0);
            b[u] = *reinterpret_cast<const float4*>(row + (size_t)u * head_dim + o1);
        }
    const int pos = IND ? *d_pos : n_past + token;
    if ((int)threadIdx.x < half) sh_freq[threadIdx.x] = rope_freq(threadIdx.x, n_rot, theta, freq_factors);
    __syncthreads();
    if (!active) return;
    float c[4], sn[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        const float ang = (float)pos * sh_freq[4 * qi + e];
        c[e] = cosf(ang);
        sn[e] = sinf(ang);
    }
#pragma unroll
    for (int u = 0; u < kHeadsPerThread4; ++u)
        if (h0 + u < heads) {
            if (NEOX) {
                rope_rotate(a[u].x, b[u].x, c[0], sn[0]);
                rope_rotate(a[u].y, b[u].y, c[1], sn[1]);
                rope_rotate(a[u].z, b[u].z, c[2], sn[2]);
                rope_rotate(a[u].w, b[u].w, c[3], sn[3]);
            } else {
                rope_rotate(a[u].x, a[u].y, c[0], sn[0]);
                rope_rotate(a[u].z, a[u].w, c[1], sn[1]);
                rope_rotate(b[u].x, b[u].y, c[2], sn[2]);
                rope_rotate(b[u].z, b[u].w, c[3], sn[3]);
            }
            store_stream(row + (size_t)u * head_dim + o0, a[u]);
            store_stream(row + (size_t)u * head_dim + o1, b[u]);
        }
}

// The three launches a prefill layer makes ahead of its attention (reference call sites:
// src/model_gpu.cu:378-382) in one: blocks [0, nbq) rotate the Q rows as rope4_kernel does,
// blocks [nbq, nbq + nbk) rotate the K rows, write them back and store them to the cache as
// fp16 (rounded from the rotated fp32 value, as the store kernel rounds what the rotary kernel
// wrote), the remaining blocks store the V rows.  n_rot = head_dim, a multiple of 8.
typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));

template <bool NEOX>
__global__ __launch_bounds__(256) void rope_store_kernel(float* q, float* k, const float* v, uint16_t* kc, uint16_t* vc,
                                                         int tokens, int n_head, int n_kv, int head_dim, int n_ctx,
                                                         int n_past, float theta, const float* freq_factors,
                                                         unsigned nbq, unsigned nbk) {
#pragma clang fp contract(off)
    __shared__ float sh_freq[256];
    if (blockIdx.x >= nbq + nbk) { // ---- V rows -> cache ----
        const int per_row = head_dim / 8;
        const long long j = (long long)(blockIdx.x - nbq - nbk) * 256 + threadIdx.x;
        if (j >= (long long)tokens * n_kv * per_row) return;
        const long long row = j / per_row; // = token * n_kv + head
        const int piece = (int)(j % per_row), head = (int)(row % n_kv), pos = n_past + (int)(row / n_kv);
        const float* src = v + row * head_dim + piece * 8;
        const float4 x0 = *reinterpret_cast<const float4*>(src);
        const float4 x1 = *reinterpret_cast<const float4*>(src + 4);
        half8_t h;
        h[0] = (_Float16)x0.x; h[1] = (_Float16)x0.y; h[2] = (_Float16)x0.z; h[3] = (_Float16)x0.w;
        h[4] = (_Float16)x1.x; h[5] = (_Float16)x1.y; h[6] = (_Float16)x1.z; h[7] = (_Float16)x1.w;
        __builtin_nontemporal_store(h, reinterpret_cast<half8_t*>(vc + ((size_t)head * n_ctx + pos) * head_dim + piece * 8));
        return;
    }
    const bool is_k = blockIdx.x >= nbq;
    float* const x = is_k ? k : q;
    const int heads = is_k ? n_kv : n_head;
    const int n_rot = head_dim, half = n_rot / 2, quads = half / 4;
    const int n_hgroups = (heads + kHeadsPerThread4 - 1) / kHeadsPerThread4;
    const long long t = (long long)(blockIdx.x - (is_k ? nbq : 0u)) * 256 + threadIdx.x;
    const bool active = t < (long long)tokens * n_hgroups * quads;
    const int qi = (int)(t % quads);
    const long long th = t / quads;
    const int hgroup = (int)(th % n_hgroups), token = (int)(th / n_hgroups);
    const int h0 = hgroup * kHeadsPerThread4;
    float* row = x + ((size_t)token * heads + h0) * head_dim;
    const int o0 = NEOX ? 4 * qi : 8 * qi, o1 = NEOX ? 4 * qi + half : 8 * qi + 4;
    float4 a[kHeadsPerThread4], b[kHeadsPerThread4];
#pragma unroll
    for (int u = 0; u < kHeadsPerThread4; ++u)
        if (active && h0 + u < heads) {
            a[u] = *reinterpret_cast<const float4*>(row + (size_t)u * head_dim + o0);
            b[u] = *reinterpret_cast<const float4*>(row + (size_t)u * head_dim + o1);
        }
    const int pos = n_past + token;
    if ((int)threadIdx.x < half) sh_freq[threadIdx.x] = rope_freq(threadIdx.x, n_rot, theta, freq_factors);
    __syncthreads();
    if (!active) return;
    float c[4], sn[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        const float ang = (float)pos * sh_freq[4 * qi + e];
        c[e] = cosf(ang);
        sn[e] = sinf(ang);
    }
#pragma unroll
    for (int u = 0; u < kHeadsPerThread4; ++u)
        if (h0 + u < heads) {
            if (NEOX) {
                rope_rotate(a[u].x, b[u].x, c[0], sn[0]);
                rope_rotate(a[u].y, b[u].y, c[1], sn[1]);
                rope_rotate(a[u].z, b[u].z, c[2], sn[2]);
                rope_rotate(a[u].w, b[u].w, c[3], sn[3]);
            } else {
                rope_rotate(a[u].x, a[u].y, c[0], sn[0]);
                rope_rotate(a[u].z, a[u].w, c[1], sn[1]);
                rope_rotate(b[u].x, b[u].y, c[2], sn[2]);
                rope_rotate(b[u].z, b[u].w, c[3], sn[3]);
            }
            store_stream(row + (size_t)u * head_dim + o0, a[u]);
            store_stream(row + (size_t)u * head_dim + o1, b[u]);
            if (is_k) {
                uint16_t* dst = kc + ((size_t)(h0 + u) * n_ctx + pos) * head_dim;
                half4_t ha, hb;
                ha[0] = (_Float16)a[u].x; ha[1] = (_Float16)a[u].y; ha[2] = (_Float16)a[u].z; ha[3] = (_Float16)a[u].w;
                hb[0] = (_Float16)b[u].x; hb[1] = (_Float16)b[u].y; hb[2] = (_Float16)b[u].z; hb[3] = (_Float16)b[u].w;
                __builtin_nontemporal_store(ha, reinterpret_cast<half4_t*>(dst + o0));
                __builtin_nontemporal_store(hb, reinterpret_cast<half4_t*>(dst + o1));
            }
        }
}

// (cos, sin) of every pair at the position *d_pos: what each thread of rope_kernel forms for
// itself, written out once for callers that rotate several rows of one token (every layer of a
// decode step rotates by the same angles).
__global__ __launch_bounds__(64) void rope_angles_kernel(float* angles, int n_rot, float theta, const int* d_pos,
                                                         const float* freq_factors) {
#pragma clang fp contract(off)
    const int i = blockIdx.x * 64 + threadIdx.x;
    if (i >= n_rot / 2) return;
    const float ang = (float)*d_pos * rope_freq(i, n_rot, theta, freq_factors);
    angles[2 * i] = cosf(ang);
    angles[2 * i + 1] = sinf(ang);
}

} // namespace

hipError_t rope_angles_launch(float* angles, int n_rot, float theta, const int* d_pos, const float* freq_factors,
                              hipStream_t stream) {
    drop_stale_error();
    const unsigned grid = (unsigned)((n_rot / 2 + 63) / 64);
    if (grid == 0) return hipSuccess;
    hipLaunchKernelGGL(rope_angles_kernel, dim3(grid), dim3(64), 0, stream, angles, n_rot, theta, d_pos, freq_factors);
    return hipGetLastError();
}

bool rope_store_fused_ok(const float* q, const float* k, const float* v, const uint16_t* kc, const uint16_t* vc,
                         int head_dim, int n_rot) {
    const uintptr_t bits = reinterpret_cast<uintptr_t>(q) | reinterpret_cast<uintptr_t>(k) | reinterpret_cast<uintptr_t>(v) |
                           reinterpret_cast<uintptr_t>(kc) | reinterpret_cast<uintptr_t>(vc);
    return n_rot == head_dim && head_dim % 8 == 0 && head_dim / 2 <= 256 && (bits & 15u) == 0;
}

hipError_t rope_store_launch(float* q, float* k, const float* v, uint16_t* kc, uint16_t* vc, int tokens, int n_head,
                             int n_kv, int head_dim, int n_ctx, int n_past, float theta, const float* freq_factors,
                             bool neox, hipStream_t stream) {
    drop_stale_error();
    const int quads = head_dim / 8;
    auto blocks = [](long long threads) { return (unsigned)((threads + 255) / 256); };
    const unsigned nbq = blocks((long long)tokens * ((n_head + kHeadsPerThread4 - 1) / kHeadsPerThread4) * quads);
    const unsigned nbk = blocks((long long)tokens * ((n_kv + kHeadsPerThread4 - 1) / kHeadsPerThread4) * quads);
    const unsigned nbv = blocks((long long)tokens * n_kv * (head_dim / 8));
    if (nbq + nbk + nbv == 0) return hipSuccess;
    if (neox)
        hipLaunchKernelGGL(rope_store_kernel<true>, dim3(nbq + nbk + nbv), dim3(256), 0, stream, q, k, v, kc, vc, tokens,
                           n_head, n_kv, head_dim, n_ctx, n_past, theta, freq_factors, nbq, nbk);
    else
        hipLaunchKernelGGL(rope_store_kernel<false>, dim3(nbq + nbk + nbv), dim3(256), 0, stream, q, k, v, kc, vc, tokens,
                           n_head, n_kv, head_dim, n_ctx, n_past, theta, freq_factors, nbq, nbk);
    return hipGetLastError();
}

hipError_t rope_launch(float* x, int rows, int head_dim, int n_rot, float theta, int n_past, int heads,
                       const int* d_pos, const float* freq_factors, bool neox, hipStream_t stream) {
    drop_stale_error();
    // batch form: rows = tokens * heads; single-token form: every row belongs to the one token
    const int tokens = d_pos ? 1 : rows / heads;
    const int heads_per_token = d_pos ? rows : heads;
    if (n_rot % 8 == 0 && n_rot / 2 <= 256 && head_dim % 4 == 0 && (reinterpret_cast<uintptr_t>(x) & 15u) == 0) {
        const int n_hgroups4 = (heads_per_token + kHeadsPerThread4 - 1) / kHeadsPerThread4;
        const long long threads4 = (long long)tokens * n_hgroups4 * (n_rot / 8);
        const unsigned grid4 = (unsigned)((threads4 + 255) / 256);
        if (grid4 == 0) return hipSuccess;
#define ORIN_ROPE4_LAUNCH(NEOX, IND) \
    hipLaunchKernelGGL((rope4_kernel<NEOX, IND>), dim3(grid4), dim3(256), 0, stream, x, tokens, heads_per_token, \
                       head_dim, n_rot, theta, n_past, d_pos, freq_factors)
        if (neox) { if (d_pos) ORIN_ROPE4_LAUNCH(true, true); else ORIN_ROPE4_LAUNCH(true, false); }
        else      { if (d_pos) ORIN_ROPE4_LAUNCH(false, true); else ORIN_ROPE4_LAUNCH(false, false); }
#undef ORIN_ROPE4_LAUNCH
        return hipGetLastError();
    }
    const int n_hgroups = (heads_per_token + kHeadsPerThread - 1) / kHeadsPerThread;
    const long long threads = (long long)tokens * n_hgroups * (n_rot / 2);
    const unsigned grid = (unsigned)((threads + 255) / 256);
    if (grid == 0) return hipSuccess;
#define ORIN_ROPE_LAUNCH(NEOX, IND) \
    hipLaunchKernelGGL((rope_kernel<NEOX, IND>), dim3(grid), dim3(256), 0, stream, x, tokens, heads_per_token, \
                       head_dim, n_rot, theta, n_past, d_pos, freq_factors)
    if (neox) { if (d_pos) ORIN_ROPE_LAUNCH(true, true); else ORIN_ROPE_LAUNCH(true, false); }
    else      { if (d_pos) ORIN_ROPE_LAUNCH(false, true); else ORIN_ROPE_LAUNCH(false, false); }
#undef ORIN_ROPE_LAUNCH
    return hipGetLastError();
}

} // namespace orin_fa
