// Matrix-vector products over quantised weight rows for gfx950 (MI355X): y = W x for one token,
// the weights streamed from HBM once and decoded in registers.
//
// Replaces the reference's gemv_dp4a_k / gemv_dp4a_smallk_k / gemv_plain_k /
// gemv_fused_gate_up_swiglu_k and their launchers (reference: src/kernels.cu:207-509,
// 1786-1835, 1944-1954).  The reference rounds the activation to int8 in blocks of 32 first and
// multiplies integers; here the activation stays fp32 and the weights are decoded to the exact
// fp32 values the reference's CPU backend decodes them to (reference: src/model_cpu.cpp:70-167),
// so the result differs from that backend's only by the order of the fp32 sum.
//
//   * Unit of work ("slot"): 32 elements of a row, chosen per weight type so that one lane's
//     loads are whole 16- or 8-byte pieces of a block (Q4_K/Q5_K: one 16-byte piece of nibbles,
//     i.e. 16 low-nibble and 16 high-nibble elements; Q6_K: 8 columns of the block's four
//     32-element strips; Q8_0: one block; F16/F32: 32 consecutive elements).  A lane keeps the
//     same slots for every row it works on, so its 32 activations per slot -- and their sums,
//     which the minimum / offset terms of the block formats multiply -- sit in registers for
//     the whole kernel: the vector cache and LDS carry weight bytes only.
//   * A row is covered by a team of 1, 2 or 4 waves (64 * slots-per-lane * 32 elements per
//     wave); a workgroup is 4 waves, i.e. 4, 2 or 1 teams on different rows.  Partial sums are
//     reduced inside the wave by lane exchanges and, for teams of several waves, through LDS.
//   * Several rows are in flight per lane at once (all loads of an iteration are issued before
//     the first is used).
//   * Folded into the same launch where the caller asks: the RMS norm of the activation in the
//     prologue (every workgroup needs the whole activation anyway), a bias or the accumulation
//     into y in the epilogue, two matrices with SiLU(gate) * up, and up to three matrices of one
//     type that share the activation (the q, k, v projections).
#include "layer_common.hpp"

#include <stdlib.h>

namespace orin_fa {
namespace {

__device__ __forceinline__ float half_bits(unsigned h) { return (float)__builtin_bit_cast(_Float16, (uint16_t)h); }
__device__ __forceinline__ float ub(unsigned v, int k) { return (float)((v >> (8 * k)) & 0xffu); }
__device__ __forceinline__ float sb(unsigned v, int k) { return (float)((int)(v << (24 - 8 * k)) >> 24); }

template <typename V>
struct __attribute__((packed, aligned(2))) Loose { // a vector at an address that is only 2-byte aligned
    V v;
};
template <typename V>
__device__ __forceinline__ V load_loose(const unsigned char* p) {
    return reinterpret_cast<const Loose<V>*>(p)->v;
}

// Per weight type: kRuns runs of kRunLen consecutive activations make up a slot's 32; run_start
// says where run r of slot s begins in the row; Raw holds a slot's bytes of one row; load
// requests them; dot multiplies them out against the slot's activations x[32] (run after run) and
// their per-run sums xs[kRuns].
template <int T>
struct Fmt;

// Q4_K block (reference: src/quant.h:14-21): d, dmin (fp16), 12 bytes of six-bit (scale, min)
// pairs, 128 bytes of nibbles.  Slot s of a block (0..7) = nibble bytes 16 s .. 16 s + 15: the low
// nibbles are elements 64 (s / 2) + 16 (s % 2) + e of pair 2 (s / 2), the high ones the same + 32 of
// pair 2 (s / 2) + 1.
__device__ __forceinline__ void pair_of(unsigned s0, unsigned s1, unsigned s2, int p, float& scale, float& min) {
    const int k = 8 * (p & 3);
    const unsigned b0 = (s0 >> k) & 0xffu, b1 = (s1 >> k) & 0xffu, b2 = (s2 >> k) & 0xffu;
    const unsigned sc = p < 4 ? b0 & 63u : (b2 & 0x0fu) | ((b0 >> 6) << 4);
    const unsigned mn = p < 4 ? b1 & 63u : (b2 >> 4) | ((b1 >> 6) << 4);
    scale = (float)sc;
    min = (float)mn;
}

template <>
struct Fmt<kQ4_K> {
    static constexpr int kRuns = 2, kRunLen = 16, kAlign = 16;
    struct Raw {
        u32x4 hdr, qs;
    };
    static __device__ __forceinline__ int run_start(int s, int r) {
        const int b = s >> 3, c = s & 7;
        return b * 256 + (c >> 1) * 64 + (c & 1) * 16 + r * 32;
    }
    static __device__ __forceinline__ void load(const unsigned char* row, int s, Raw& w) {
        const unsigned char* blk = row + (size_t)(s >> 3) * 144;
        w.hdr = *reinterpret_cast<const u32x4*>(blk);
        w.qs = *reinterpret_cast<const u32x4*>(blk + 16 + (s & 7) * 16);
    }
    static __device__ __forceinline__ float dot(const Raw& w, int s, const float* x, const float* xs) {
        const float d = half_bits(w.hdr.x & 0xffffu), dmin = half_bits(w.hdr.x >> 16);
        const int p = (s & 7) >> 1 << 1;
        float sc0, mn0, sc1, mn1;
        pair_of(w.hdr.y, w.hdr.z, w.hdr.w, p, sc0, mn0);
        pair_of(w.hdr.y, w.hdr.z, w.hdr.w, p + 1, sc1, mn1);
        float a0 = 0.0f, a1 = 0.0f;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const unsigned lo = w.qs[i] & 0x0f0f0f0fu, hi = (w.qs[i] >> 4) & 0x0f0f0f0fu;
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                a0 += ub(lo, k) * x[4 * i + k];
                a1 += ub(hi, k) * x[16 + 4 * i + k];
            }
        }
        return (d * sc0) * a0 - (dmin * mn0) * xs[0] + ((d * sc1) * a1 - (dmin * mn1) * xs[1]);
    }
};

// Q5_K block (reference: src/quant.h:24-31): as Q4_K with 32 bytes of fifth bits behind the pairs;
// bit p of byte e belongs to element 32 p + e.  A slot needs bytes 16 (s % 2) .. + 15 of them.
template <>
struct Fmt<kQ5_K> {
    static constexpr int kRuns = 2, kRunLen = 16, kAlign = 16;
    struct Raw {
        u32x4 hdr, qh, qs;
    };
    static __device__ __forceinline__ int run_start(int s, int r) { return Fmt<kQ4_K>::run_start(s, r); }
    static __device__ __forceinline__ void load(const unsigned char* row, int s, Raw& w) {
        const unsigned char* blk = row + (size_t)(s >> 3) * 176;
        w.hdr = *reinterpret_cast<const u32x4*>(blk);
        w.qh = *reinterpret_cast<const u32x4*>(blk + 16 + (s & 1) * 16);
        w.qs = *reinterpret_cast<const u32x4*>(blk + 48 + (s & 7) * 16);
    }
    static __device__ __forceinline__ float dot(const Raw& w, int s, const float* x, const float* xs) {
        const float d = half_bits(w.hdr.x & 0xffffu), dmin = half_bits(w.hdr.x >> 16);
        const int p = (s & 7) >> 1 << 1;
        float sc0, mn0, sc1, mn1;
        pair_of(w.hdr.y, w.hdr.z, w.hdr.w, p, sc0, mn0);
        pair_of(w.hdr.y, w.hdr.z, w.hdr.w, p + 1, sc1, mn1);
        float a0 = 0.0f, a1 = 0.0f;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const unsigned h = w.qh[i] >> p;
            const unsigned lo = (w.qs[i] & 0x0f0f0f0fu) | ((h & 0x01010101u) << 4);
            const unsigned hi = ((w.qs[i] >> 4) & 0x0f0f0f0fu) | ((h & 0x02020202u) << 3);
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                a0 += ub(lo, k) * x[4 * i + k];
                a1 += ub(hi, k) * x[16 + 4 * i + k];
            }
        }
        return (d * sc0) * a0 - (dmin * mn0) * xs[0] + ((d * sc1) * a1 - (dmin * mn1) * xs[1]);
    }
};

// Q6_K block (reference: src/quant.h:34-40), 210 bytes and therefore only 2-byte aligned: 128 bytes
// of low nibbles, 64 of high bit pairs, 16 signed scales, d (fp16).  Per half h of 128 elements,
// strip c (0..3) is elements 32 c + l; its low nibbles sit in bytes l + 32 (c & 1) of the half's 64
// (low nibble for c < 2), its high bits at bits 2 c of high byte l, its scales at 2 c + l / 16.
// Slot s of a block = (h, columns l = 8 (s & 3) .. + 7 of all four strips): four runs of 8.
template <>
struct Fmt<kQ6_K> {
    static constexpr int kRuns = 4, kRunLen = 8, kAlign = 2;
    struct Raw {
        u32x2 la, lb, qh, sc;
        unsigned d;
    };
    static __device__ __forceinline__ int run_start(int s, int r) {
        const int b = s >> 3, h = (s >> 2) & 1, lq = s & 3;
        return b * 256 + h * 128 + r * 32 + lq * 8;
    }
    static __device__ __forceinline__ void load(const unsigned char* row, int s, Raw& w) {
        const unsigned char* blk = row + (size_t)(s >> 3) * 210;
        const int h = (s >> 2) & 1, lq = s & 3;
        w.la = load_loose<u32x2>(blk + 64 * h + 8 * lq);
        w.lb = load_loose<u32x2>(blk + 64 * h + 32 + 8 * lq);
        w.qh = load_loose<u32x2>(blk + 128 + 32 * h + 8 * lq);
        w.sc = load_loose<u32x2>(blk + 192 + 8 * h);
        w.d = *reinterpret_cast<const uint16_t*>(blk + 208);
    }
    static __device__ __forceinline__ float dot(const Raw& w, int s, const float* x, const float* xs) {
        const float d = half_bits(w.d);
        const int odd = (s & 3) >> 1; // l / 16
        float out = 0.0f;
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            const u32x2 src = (c & 1) ? w.lb : w.la;
            float a = 0.0f;
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                const unsigned nib = (c < 2 ? src[i] : src[i] >> 4) & 0x0f0f0f0fu;
                const unsigned v = nib | (((w.qh[i] >> (2 * c)) & 0x03030303u) << 4);
#pragma unroll
                for (int k = 0; k < 4; ++k) a += ub(v, k) * x[8 * c + 4 * i + k];
            }
            // scale byte 2 c + odd of the half's eight
            const int idx = 2 * c + odd;
            const unsigned word = idx < 4 ? w.sc.x : w.sc.y;
            const float scale = (float)((int)(word << (24 - 8 * (idx & 3))) >> 24);
            out += (d * scale) * (a - 32.0f * xs[c]);
        }
        return out;
    }
};

// Q8_0 block (reference: src/quant.h:42-45), 34 bytes: d (fp16) and 32 signed bytes.  Slot = block.
template <>
struct Fmt<kQ8_0> {
    static constexpr int kRuns = 1, kRunLen = 32, kAlign = 2;
    struct Raw {
        u32x4 a, b;
        unsigned d;
    };
    static __device__ __forceinline__ int run_start(int s, int) { return s * 32; }
    static __device__ __forceinline__ void load(const unsigned char* row, int s, Raw& w) {
        const unsigned char* blk = row + (size_t)s * 34;
        w.d = *reinterpret_cast<const uint16_t*>(blk);
        w.a = load_loose<u32x4>(blk + 2);
        w.b = load_loose<u32x4>(blk + 18);
    }
    static __device__ __forceinline__ float dot(const Raw& w, int, const float* x, const float*) {
        float a = 0.0f;
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                a += sb(w.a[i], k) * x[4 * i + k];
                a += sb(w.b[i], k) * x[16 + 4 * i + k];
            }
        return half_bits(w.d) * a;
    }
};

template <>
struct Fmt<kF16> {
    static constexpr int kRuns = 1, kRunLen = 32, kAlign = 16;
    struct Raw {
        h8 v[4];
    };
    static __device__ __forceinline__ int run_start(int s, int) { return s * 32; }
    static __device__ __forceinline__ void load(const unsigned char* row, int s, Raw& w) {
#pragma unroll
        for (int i = 0; i < 4; ++i) w.v[i] = *reinterpret_cast<const h8*>(row + (size_t)s * 64 + i * 16);
    }
    static __device__ __forceinline__ float dot(const Raw& w, int, const float* x, const float*) {
        float a = 0.0f;
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int k = 0; k < 8; ++k) a += (float)w.v[i][k] * x[8 * i + k];
        return a;
    }
};

template <>
struct Fmt<kF32> {
    static constexpr int kRuns = 1, kRunLen = 32, kAlign = 16;
    struct Raw {
        f4 v[8];
    };
    static __device__ __forceinline__ int run_start(int s, int) { return s * 32; }
    static __device__ __forceinline__ void load(const unsigned char* row, int s, Raw& w) {
#pragma unroll
        for (int i = 0; i < 8; ++i) w.v[i] = *reinterpret_cast<const f4*>(row + (size_t)s * 128 + i * 16);
    }
    static __device__ __forceinline__ float dot(const Raw& w, int, const float* x, const float*) {
        float a = 0.0f;
#pragma unroll
        for (int i = 0; i < 8; ++i)
#pragma unroll
            for (int k = 0; k < 4; ++k) a += w.v[i][k] * x[4 * i + k];
        return a;
    }
};

constexpr int kGemvWaves = 4;

// T: weight type.  SLOTS: slots per lane.  DUAL: two matrices (gate, up) and SiLU(gate) * up.
// Grid: (workgroups, matrices).  A workgroup walks row groups g = blockIdx.x, + gridDim.x, ...; a row
// group is RB rows for each of the workgroup's teams.  The rows of group g + gridDim.x are requested
// before those of group g are multiplied out, and the first group before the activation is even
// loaded, so a workgroup always has two groups of weight bytes on their way.
template <int T, int SLOTS, bool DUAL>
__global__ __launch_bounds__(kGemvWaves * 64) void gemv_kernel(const GemvArgs a) {
    using F = Fmt<T>;
    constexpr int RB = SLOTS == 1 ? 2 : 1;
    constexpr int M = DUAL ? 2 : 1;
    __shared__ float sh_red[kGemvWaves][M * RB];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int kw = a.team_waves;                 // waves per row: 1, 2 or 4
    const int team = wave / kw, n_teams = kGemvWaves / kw;
    const int tt = (wave % kw) * 64 + lane, ts = kw * 64;
    const int n_slots = a.n_in >> 5;
    const GemvSeg seg = a.seg[blockIdx.y];
    const size_t row_bytes = a.row_bytes;
    const unsigned char* const w0 = static_cast<const unsigned char*>(seg.w);
    const unsigned char* const w1 = static_cast<const unsigned char*>(DUAL ? a.w_up : seg.w);
    const int last = seg.n_out - 1;
    const int per_group = n_teams * RB;
    const int n_groups = (seg.n_out + per_group - 1) / per_group;
    if ((int)blockIdx.x >= n_groups) return; // (whole workgroup: a shorter matrix of a shared launch)

    bool live[SLOTS];
    int slot[SLOTS];
#pragma unroll
    for (int i = 0; i < SLOTS; ++i) {
        live[i] = i * ts + tt < n_slots;
        slot[i] = live[i] ? i * ts + tt : 0; // (idle lanes repeat slot 0 and count for nothing)
    }
    typedef typename F::Raw Raw;
    Raw raw_a[M][RB][SLOTS], raw_b[M][RB][SLOTS];
    auto request = [&](Raw (&raw)[M][RB][SLOTS], int g) {
        g = min(g, n_groups - 1); // (past the end: the last group once more, from the cache; never used)
#pragma unroll
        for (int b = 0; b < RB; ++b) {
            const int row = min(g * per_group + team * RB + b, last);
#pragma unroll
            for (int i = 0; i < SLOTS; ++i) {
                F::load(w0 + (size_t)row * row_bytes, slot[i], raw[0][b][i]);
                if constexpr (DUAL) F::load(w1 + (size_t)row * row_bytes, slot[i], raw[1][b][i]);
            }
        }
    };
    request(raw_a, blockIdx.x);
    __builtin_amdgcn_sched_barrier(0);

    // ---- this lane's activations, once ----
    float x[SLOTS][32], xs[SLOTS][F::kRuns];
    float ss = 0.0f;
#pragma unroll
    for (int i = 0; i < SLOTS; ++i) {
#pragma unroll
        for (int r = 0; r < F::kRuns; ++r) {
            const int e0 = F::run_start(slot[i], r);
#pragma unroll
            for (int j = 0; j < F::kRunLen; j += 4) {
                const float4 v = *reinterpret_cast<const float4*>(a.x + e0 + j);
                float4 g = float4{1.f, 1.f, 1.f, 1.f};
                if (a.norm_w) g = *reinterpret_cast<const float4*>(a.norm_w + e0 + j);
                const float m = live[i] ? 1.0f : 0.0f;
                float* dst = &x[i][r * F::kRunLen + j];
                dst[0] = v.x * m; dst[1] = v.y * m; dst[2] = v.z * m; dst[3] = v.w * m;
                if (a.norm_w) {
                    ss += dst[0] * dst[0] + dst[1] * dst[1] + dst[2] * dst[2] + dst[3] * dst[3];
                    dst[0] *= g.x; dst[1] *= g.y; dst[2] *= g.z; dst[3] *= g.w;
                }
            }
        }
    }
    if (a.norm_w) {
        // x / sqrt(mean(x^2) + eps) * w (reference: src/kernels.cu:1596-1604, CPU src/model_cpu.cpp:13-18)
        ss = wave_sum(ss);
        if (kw > 1) {
            if (lane == 0) sh_red[wave][0] = ss;
            __syncthreads();
            ss = 0.0f;
            for (int w = 0; w < kw; ++w) ss += sh_red[team * kw + w][0];
            __syncthreads();
        }
        const float rinv = 1.0f / sqrtf(ss / (float)a.n_in + a.eps);
#pragma unroll
        for (int i = 0; i < SLOTS; ++i)
#pragma unroll
            for (int e = 0; e < 32; ++e) x[i][e] *= rinv;
    }
#pragma unroll
    for (int i = 0; i < SLOTS; ++i)
#pragma unroll
        for (int r = 0; r < F::kRuns; ++r) {
            float t = 0.0f;
#pragma unroll
            for (int e = 0; e < F::kRunLen; ++e) t += x[i][r * F::kRunLen + e];
            xs[i][r] = t;
        }

    auto finish = [&](const Raw (&raw)[M][RB][SLOTS], int g) {
        float acc[M][RB];
#pragma unroll
        for (int m = 0; m < M; ++m)
#pragma unroll
            for (int b = 0; b < RB; ++b) {
                float t = 0.0f;
#pragma unroll
                for (int i = 0; i < SLOTS; ++i) {
                    const float part = F::dot(raw[m][b][i], slot[i], x[i], xs[i]);
                    t += live[i] ? part : 0.0f;
                }
                acc[m][b] = wave_sum(t);
            }
        if (kw > 1) { // the team's waves meet in LDS (every wave of the workgroup walks the same groups)
            if (lane == 0)
#pragma unroll
                for (int m = 0; m < M; ++m)
#pragma unroll
                    for (int b = 0; b < RB; ++b) sh_red[wave][m * RB + b] = acc[m][b];
            __syncthreads();
#pragma unroll
            for (int m = 0; m < M; ++m)
#pragma unroll
                for (int b = 0; b < RB; ++b) {
                    float t = 0.0f;
                    for (int w = 0; w < kw; ++w) t += sh_red[team * kw + w][m * RB + b];
                    acc[m][b] = t;
                }
            __syncthreads();
        }
        if (lane == 0 && wave % kw == 0) {
#pragma unroll
            for (int b = 0; b < RB; ++b) {
                const int row = g * per_group + team * RB + b;
                if (row > last) continue;
                float v = acc[0][b];
                if constexpr (DUAL) {
                    // SiLU(gate) * up (reference: src/kernels.cu:396-492, CPU src/model_cpu.cpp:11,302)
                    v = v / (1.0f + expf(-v)) * acc[1][b];
                }
                if (seg.bias) v += seg.bias[row];
                if (a.accumulate) v += seg.y[row];
                seg.y[row] = v;
            }
        }
    };
    const int stride = gridDim.x;
    for (int g = blockIdx.x; g < n_groups; g += 2 * stride) {
        request(raw_b, g + stride);
        finish(raw_a, g);
        if (g + stride >= n_groups) break;
        request(raw_a, g + 2 * stride);
        finish(raw_b, g + stride);
    }
}

template <int T, int SLOTS>
hipError_t launch_slots(const GemvArgs& a, dim3 grid, hipStream_t stream) {
    if (a.w_up)
        hipLaunchKernelGGL((gemv_kernel<T, SLOTS, true>), grid, dim3(kGemvWaves * 64), 0, stream, a);
    else
        hipLaunchKernelGGL((gemv_kernel<T, SLOTS, false>), grid, dim3(kGemvWaves * 64), 0, stream, a);
    return hipGetLastError();
}

template <int T>
hipError_t launch_type(GemvArgs& a, int cu_count, hipStream_t stream) {
    const int n_slots = a.n_in / 32;
    // Fewest waves per row that keep a lane at three slots or fewer (96 activations in registers); rows past
    // what four waves cover that way (24576 elements) take a fourth slot.
    int kw = 1;
    while (kw < kGemvWaves && n_slots > kw * 64 * 3) kw *= 2;
    const int slots = (n_slots + kw * 64 - 1) / (kw * 64);
    if (slots > 4) return hipErrorInvalidValue;
    a.team_waves = kw;
    const int per_group = (kGemvWaves / kw) * (slots == 1 ? 2 : 1);
    int max_out = 0;
    for (int i = 0; i < a.n_seg; ++i) max_out = max(max_out, a.seg[i].n_out);
    // At most kGemvWgsPerCu workgroups per CU, each walking its share of the row groups: the activation is
    // fetched once per workgroup, so fewer, longer-lived workgroups keep that traffic below the weights'.
    const int n_groups = (max_out + per_group - 1) / per_group;
    const int wgs = min(n_groups, cu_count * a.wgs_per_cu);
    const dim3 grid(wgs, a.n_seg);
    switch (slots) {
    case 1: return launch_slots<T, 1>(a, grid, stream);
    case 2: return launch_slots<T, 2>(a, grid, stream);
    case 3: return launch_slots<T, 3>(a, grid, stream);
    default: return launch_slots<T, 4>(a, grid, stream);
    }
}

} // namespace

// Workgroups per CU of a launch (ORIN_GEMV_WGS_PER_CU overrides, for tuning runs).
int gemv_wgs_per_cu() {
    static const int v = [] {
        const char* e = getenv("ORIN_GEMV_WGS_PER_CU");
        const int n = e ? atoi(e) : 0;
        return n >= 1 && n <= 16 ? n : 2;
    }();
    return v;
}

// Workgroups per CU of the matrix-core kernel (0: one per 16-row tile; ORIN_GEMV_MFMA_WGS_PER_CU overrides).
int gemv_mfma_wgs_per_cu() {
    static const int v = [] {
        const char* e = getenv("ORIN_GEMV_MFMA_WGS_PER_CU");
        const int n = e ? atoi(e) : -1;
        return n >= 0 && n <= 16 ? n : 2;
    }();
    return v;
}

// Whether block types go to the matrix-core kernel (default) or stay on the vector-ALU kernel
// (orin_gemv_use_matrix_cores(0), or ORIN_GEMV_NO_MFMA=1 in the environment: for comparisons and tests).
static int g_use_mfma = -1;
bool gemv_use_mfma() {
    if (g_use_mfma < 0) {
        const char* e = getenv("ORIN_GEMV_NO_MFMA");
        g_use_mfma = !(e && e[0] == '1');
    }
    return g_use_mfma != 0;
}
void gemv_set_use_mfma(bool on) { g_use_mfma = on ? 1 : 0; }

// Shares of a row that an accumulating projection may be cut into (0: the launcher chooses 1, 2 or 4 by shape;
// 1: never cut, which makes `y += W x` a plain sum with a fixed order; orin_gemv_row_shares(), or ORIN_GEMV_KSPLIT in
// the environment as the initial value).
static int g_row_shares = -1;
int gemv_row_shares() {
    if (g_row_shares < 0) {
        const char* e = getenv("ORIN_GEMV_KSPLIT");
        const int n = e ? atoi(e) : 0;
        g_row_shares = n >= 0 && n <= 4 ? n : 0;
    }
    return g_row_shares;
}
void gemv_set_row_shares(int n) { g_row_shares = n >= 0 && n <= 4 ? n : 0; }

size_t weight_row_bytes(int type, int n) {
    switch (type) {
    case kF32: return (size_t)n * 4;
    case kF16: return (size_t)n * 2;
    case kQ8_0: return n % 32 ? 0 : (size_t)(n / 32) * 34;
    case kQ4_K: return n % 256 ? 0 : (size_t)(n / 256) * 144;
    case kQ5_K: return n % 256 ? 0 : (size_t)(n / 256) * 176;
    case kQ6_K: return n % 256 ? 0 : (size_t)(n / 256) * 210;
    default: return 0;
    }
}

int weight_align(int type) { return type == kQ6_K || type == kQ8_0 ? 2 : 16; }

hipError_t gemv_launch(int type, GemvArgs a, int cu_count, hipStream_t stream) {
    drop_stale_error();
    a.row_bytes = weight_row_bytes(type, a.n_in);
    if (a.row_bytes == 0 || a.n_in % 32 != 0 || a.n_seg < 1 || a.n_seg > 3) return hipErrorInvalidValue;
    if (a.wgs_per_cu < 1) a.wgs_per_cu = gemv_wgs_per_cu();
    a.mfma_wgs_per_cu = gemv_mfma_wgs_per_cu();
    a.k_split_override = gemv_row_shares();
    if (gemv_use_mfma() && gemv_mfma_ok(type, a)) return gemv_mfma_launch(type, a, cu_count, stream);
    switch (type) {
    case kF32: return launch_type<kF32>(a, cu_count, stream);
    case kF16: return launch_type<kF16>(a, cu_count, stream);
    case kQ8_0: return launch_type<kQ8_0>(a, cu_count, stream);
    case kQ4_K: return launch_type<kQ4_K>(a, cu_count, stream);
    case kQ5_K: return launch_type<kQ5_K>(a, cu_count, stream);
    case kQ6_K: return launch_type<kQ6_K>(a, cu_count, stream);
    default: return hipErrorInvalidValue;
    }
}

// Matrices of different types over one activation: one launch when every one of them is Q4_K or Q6_K and the
// matrix-core kernel takes the shape; hipErrorNotSupported otherwise (the caller then launches them one by one).
hipError_t gemv_mixed_launch(GemvArgs a, int cu_count, hipStream_t stream) {
    drop_stale_error();
    if (!gemv_use_mfma() || a.w_up || a.n_seg < 1 || a.n_seg > 3) return hipErrorNotSupported;
    for (int i = 0; i < a.n_seg; ++i) {
        if (!gemv_mfma_ok(a.seg[i].type, a)) return hipErrorNotSupported;
        a.seg[i].row_bytes = weight_row_bytes(a.seg[i].type, a.n_in);
    }
    a.mfma_wgs_per_cu = gemv_mfma_wgs_per_cu();
    return gemv_mfma_mixed_launch(a, cu_count, stream);
}

} // namespace orin_fa
