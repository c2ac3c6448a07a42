// GQA flash attention for gfx950 (MI355X): causal chunked prefill and split-KV
// single-token decode over the fp16 KV cache, plus the C ABI of include/orin_fa.h.
//
// Replaces the reference's flash_attention_prefill_mma_k / flash_attention_decode_mma_k
// and their host wrappers (reference: src/kernels.cu:1105-1568, 1956-2000).
//
// Shape of the computation (one template serves both operators):
//   * A workgroup is 4 wave64s that own one KV head, a block of query columns
//     (prefill: TQ tokens x the head group; decode: the head group of the one token)
//     and a contiguous range of 32-row KV tiles.  Wave w takes tiles w, w+4, ... and
//     keeps its own online-softmax state, so the main loop has no workgroup barrier.
//   * Per tile a wave streams 32 K rows and 32 V rows from global memory with
//     coalesced 128-bit loads (next tile prefetched into registers while this one is
//     consumed), parks them in its private LDS slice, and reads them back in MFMA
//     operand order.
//   * S^T = K Q^T and O^T = V^T P run on v_mfma_f32_16x16x32_f16.  The accumulator
//     layout of the first product (lane = query column, 4 KV rows per lane-group) is
//     the B-operand layout of the second once the 32 KV rows of a tile are numbered
//     (lane-group, sub-tile, row) -- no shuffle of P is needed, and every rescale
//     factor is a per-lane scalar.
//   * Row maxima / sums over the four lane-groups use two xor-shuffles.
//   * The four waves' (m, l, O) are merged through LDS; decode then writes one
//     partial per KV split and a second kernel merges the splits (log-sum-exp combine).
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>

#include "../../include/orin_fa.h"

namespace {

typedef _Float16 h8 __attribute__((ext_vector_type(8)));
typedef float f4 __attribute__((ext_vector_type(4)));

constexpr int kWaves = 4;             // waves per workgroup
constexpr int kThreads = kWaves * 64;
constexpr int kTile = 32;             // KV rows per wave tile
constexpr float kLog2e = 1.4426950408889634f;
constexpr float kPShift = 12.0f;      // P is scaled by 2^12 before fp16 rounding (keeps small weights normal)
constexpr size_t kWorkspaceBytes = 8u << 20;
constexpr int kMaxSplits = 512;

struct FaArgs {
    const float* q;
    const uint16_t* kc;
    const uint16_t* vc;
    float* out;
    float* part_o;    // [split][n_head][D]
    float* part_ml;   // [split][n_head][2] = (running max in log2 units, row sum)
    const int* d_pos; // decode only
    int n_head, n_kv, n_ctx;
    int n_past, batch; // prefill only
    int r;             // query heads per KV head
    int n_hgroups;     // head groups per KV head
    int n_ttiles;      // prefill: token tiles
    int n_splits;      // decode: KV splits
    float scale_log2e;
};

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

__device__ __forceinline__ float xor_max(float v) {
    v = fmaxf(v, __shfl_xor(v, 16));
    v = fmaxf(v, __shfl_xor(v, 32));
    return v;
}
__device__ __forceinline__ float xor_sum(float v) {
    v += __shfl_xor(v, 16);
    v += __shfl_xor(v, 32);
    return v;
}

// Orders this wave's LDS writes before its later LDS reads (lanes of one wave
// exchange data through the wave-private LDS slice).
__device__ __forceinline__ void wave_lds_sync() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

template <int D, int NQB>
struct Geom {
    static constexpr int kSteps = D / 32;            // MFMA k-steps over head_dim
    static constexpr int kDBlk = D / 16;             // 16-wide output blocks over head_dim
    static constexpr int kRowB = D * 2 + 16;         // bytes per KV row in LDS (16 B pad: conflict-free b128 reads)
    static constexpr int kChunksPerRow = D / 8;      // 16-byte chunks per KV row
    static constexpr int kLoads = kTile * kChunksPerRow / 64; // 16-byte loads per lane per matrix per tile
    static constexpr int kTileB = kTile * kRowB;     // bytes of one K (or V) tile in LDS
    static constexpr int kOStride = D + 4;           // floats per column in the merge buffer
    static constexpr int kMergeB = NQB * 16 * kOStride * 4;
    static constexpr int kWaveB = (2 * kTileB > kMergeB) ? 2 * kTileB : kMergeB;
    static constexpr int kMlOff = kWaves * kWaveB;   // (m, l) per wave per column follow the wave slices
    static constexpr int kLdsB = kMlOff + kWaves * NQB * 16 * 2 * 4;
};

// D: head_dim; NQB: 16-column query blocks per workgroup; TQ: tokens per workgroup
// (column c = local_head * TQ + local_token); PRECISE: carry Q and P as fp16 hi+lo
// pairs (decode, where the matrix pipe is idle anyway); DECODE: position from *d_pos,
// KV splits across workgroups, partial outputs.
template <int D, int NQB, int TQ, bool PRECISE, bool DECODE>
__global__ __launch_bounds__(kThreads) void fa_fwd_kernel(const FaArgs a) {
    using G = Geom<D, NQB>;
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];

    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int col = lane & 15; // MFMA column (query column) / row (KV row or head_dim index) owned by the lane
    const int grp = lane >> 4; // lane-group: 8-wide k slice of an operand, 4-row slice of an accumulator

    // Workgroup id -> (KV head, head group, token tile | split).  The KV head varies
    // fastest so that the workgroups an XCD receives (id mod 8) share one KV head.
    int id = blockIdx.x;
    const int kvh = id % a.n_kv;
    id /= a.n_kv;
    const int hg = id % a.n_hgroups;
    id /= a.n_hgroups;

    int n_past, batch, t0;
    if (DECODE) {
        int p = *a.d_pos;
        p = p < 0 ? 0 : p;
        n_past = p > a.n_ctx - 1 ? a.n_ctx - 1 : p;
        batch = 1;
        t0 = 0;
    } else {
        n_past = a.n_past;
        batch = a.batch;
        t0 = (a.n_ttiles - 1 - id) * TQ; // longest rows first
    }
    constexpr int kHeadsPerGroup = NQB * 16 / TQ;
    const int head_lo = hg * kHeadsPerGroup;
    const int tok_hi = (t0 + TQ < batch) ? t0 + TQ : batch;
    const int kv_end = n_past + tok_hi;     // the workgroup's columns see rows [0, kv_end) at most
    const int full_end = n_past + t0 + 1;   // rows below this are visible to every column
    const int n_tiles = (kv_end + kTile - 1) / kTile;
    int tile_lo = 0, tile_hi = n_tiles;
    if (DECODE) {
        const int tps = (n_tiles + a.n_splits - 1) / a.n_splits;
        tile_lo = id * tps;
        tile_hi = (tile_lo + tps < n_tiles) ? tile_lo + tps : n_tiles;
        if (tile_lo >= tile_hi) return; // inactive split: the combine kernel never reads it
    }

    // ---- query columns -> B operands (fp16, optionally hi + lo) ----
    h8 qhi[NQB][G::kSteps];
    h8 qlo[PRECISE ? NQB : 1][PRECISE ? G::kSteps : 1];
    int limit[NQB];
#pragma unroll
    for (int qb = 0; qb < NQB; ++qb) {
        const int c = qb * 16 + col;
        const int tok = t0 + c % TQ;
        const int hl = head_lo + c / TQ;
        const bool valid = (hl < a.r) && (tok < batch);
        limit[qb] = valid ? n_past + tok + 1 : 0x7fffffff;
        const float* qp = a.q + ((size_t)(valid ? tok : 0) * a.n_head + (size_t)(valid ? kvh * a.r + hl : 0)) * D;
#pragma unroll
        for (int kk = 0; kk < G::kSteps; ++kk) {
            const float4 x0 = *reinterpret_cast<const float4*>(qp + kk * 32 + grp * 8);
            const float4 x1 = *reinterpret_cast<const float4*>(qp + kk * 32 + grp * 8 + 4);
            const float x[8] = {x0.x, x0.y, x0.z, x0.w, x1.x, x1.y, x1.z, x1.w};
            h8 hi, lo;
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const float xe = valid ? x[e] : 0.0f;
                hi[e] = (_Float16)xe;
                lo[e] = (_Float16)(xe - (float)hi[e]);
            }
            qhi[qb][kk] = hi;
            if (PRECISE) qlo[qb][kk] = lo;
        }
    }

    unsigned char* const ks = smem + wave * G::kWaveB;
    unsigned char* const vs = ks + G::kTileB;
    const _Float16* const kbase = reinterpret_cast<const _Float16*>(a.kc) + (size_t)kvh * a.n_ctx * D;
    const _Float16* const vbase = reinterpret_cast<const _Float16*>(a.vc) + (size_t)kvh * a.n_ctx * D;

    float m_run[NQB], l_run[NQB];
    f4 o[NQB][G::kDBlk];
#pragma unroll
    for (int qb = 0; qb < NQB; ++qb) {
        m_run[qb] = -INFINITY;
        l_run[qb] = 0.0f;
#pragma unroll
        for (int db = 0; db < G::kDBlk; ++db) o[qb][db] = f4{0.f, 0.f, 0.f, 0.f};
    }

    uint4 kreg[G::kLoads], vreg[G::kLoads];
    auto fetch = [&](int tile) {
#pragma unroll
        for (int i = 0; i < G::kLoads; ++i) {
            const int c = i * 64 + lane;
            const int row = tile * kTile + c / G::kChunksPerRow;
            const int ch = c % G::kChunksPerRow;
            if (row < kv_end) { // rows past the visible range are never read: the cache tail may hold anything
                kreg[i] = *reinterpret_cast<const uint4*>(kbase + (size_t)row * D + ch * 8);
                vreg[i] = *reinterpret_cast<const uint4*>(vbase + (size_t)row * D + ch * 8);
            } else {
                kreg[i] = uint4{0u, 0u, 0u, 0u};
                vreg[i] = uint4{0u, 0u, 0u, 0u};
            }
        }
    };

    int tile = tile_lo + wave;
    if (tile < tile_hi) fetch(tile);
    for (; tile < tile_hi; tile += kWaves) {
        // registers -> this wave's LDS slice
#pragma unroll
        for (int i = 0; i < G::kLoads; ++i) {
            const int c = i * 64 + lane;
            const int off = (c / G::kChunksPerRow) * G::kRowB + (c % G::kChunksPerRow) * 16;
            *reinterpret_cast<uint4*>(ks + off) = kreg[i];
            *reinterpret_cast<uint4*>(vs + off) = vreg[i];
        }
        if (tile + kWaves < tile_hi) fetch(tile + kWaves);
        wave_lds_sync();

        // ---- S^T = K Q^T : rows = KV row (sub-tile t, row col), columns = query column ----
        f4 s[2][NQB];
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int qb = 0; qb < NQB; ++qb) s[t][qb] = f4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int kk = 0; kk < G::kSteps; ++kk) {
#pragma unroll
            for (int t = 0; t < 2; ++t) {
                const h8 ka = *reinterpret_cast<const h8*>(ks + (t * 16 + col) * G::kRowB + (kk * 4 + grp) * 16);
#pragma unroll
                for (int qb = 0; qb < NQB; ++qb) {
                    s[t][qb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(ka, qhi[qb][kk], s[t][qb], 0, 0, 0);
                    if (PRECISE) s[t][qb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(ka, qlo[qb][kk], s[t][qb], 0, 0, 0);
                }
            }
        }

        // ---- online softmax; lane (col, grp) holds rows t*16 + grp*4 + i of its column ----
        const bool need_mask = (tile * kTile + kTile > full_end);
        h8 phi[NQB];
        h8 plo[PRECISE ? NQB : 1];
#pragma unroll
        for (int qb = 0; qb < NQB; ++qb) {
            float v[8];
#pragma unroll
            for (int t = 0; t < 2; ++t)
#pragma unroll
                for (int i = 0; i < 4; ++i) v[t * 4 + i] = s[t][qb][i] * a.scale_log2e;
            if (need_mask) {
#pragma unroll
                for (int t = 0; t < 2; ++t)
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        const int row = tile * kTile + t * 16 + grp * 4 + i;
                        if (row >= limit[qb]) v[t * 4 + i] = -INFINITY;
                    }
            }
            float mx = v[0];
#pragma unroll
            for (int e = 1; e < 8; ++e) mx = fmaxf(mx, v[e]);
            mx = xor_max(mx);
            const float m_new = fmaxf(m_run[qb], mx);
            const float m_use = (m_new == -INFINITY) ? 0.0f : m_new;
            const float alpha = fast_exp2(m_run[qb] - m_use);
            m_run[qb] = m_new;
            float sum = 0.0f;
            h8 ph, pl;
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const float p = fast_exp2(v[e] - m_use + kPShift);
                sum += p;
                ph[e] = (_Float16)p;
                pl[e] = (_Float16)(p - (float)ph[e]);
            }
            l_run[qb] = l_run[qb] * alpha + sum;
            phi[qb] = ph;
            if (PRECISE) plo[qb] = pl;
#pragma unroll
            for (int db = 0; db < G::kDBlk; ++db) o[qb][db] *= alpha;
        }

        // ---- O^T += V^T P : rows = head_dim index, columns = query column, k = the tile's 32 KV rows
        //      in the order (grp, t, i) that matches the layout P already has ----
#pragma unroll
        for (int db = 0; db < G::kDBlk; ++db) {
            h8 va;
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const int row = (e >> 2) * 16 + grp * 4 + (e & 3);
                va[e] = *reinterpret_cast<const _Float16*>(vs + row * G::kRowB + (db * 16 + col) * 2);
            }
#pragma unroll
            for (int qb = 0; qb < NQB; ++qb) {
                o[qb][db] = __builtin_amdgcn_mfma_f32_16x16x32_f16(va, phi[qb], o[qb][db], 0, 0, 0);
                if (PRECISE) o[qb][db] = __builtin_amdgcn_mfma_f32_16x16x32_f16(va, plo[qb], o[qb][db], 0, 0, 0);
            }
        }
        wave_lds_sync(); // the slice is overwritten at the top of the next iteration
    }

    // ---- merge the four waves through LDS ----
    float* const ml = reinterpret_cast<float*>(smem + G::kMlOff);
    float* const obuf = reinterpret_cast<float*>(smem + wave * G::kWaveB);
#pragma unroll
    for (int qb = 0; qb < NQB; ++qb) {
        const float l_tot = xor_sum(l_run[qb]);
        if (grp == 0) {
            ml[(wave * NQB * 16 + qb * 16 + col) * 2 + 0] = m_run[qb];
            ml[(wave * NQB * 16 + qb * 16 + col) * 2 + 1] = l_tot;
        }
#pragma unroll
        for (int db = 0; db < G::kDBlk; ++db)
            *reinterpret_cast<f4*>(obuf + (qb * 16 + col) * G::kOStride + db * 16 + grp * 4) = o[qb][db];
    }
    __syncthreads();

    constexpr int kCols = NQB * 16;
    for (int idx = threadIdx.x; idx < kCols * (D / 4); idx += kThreads) {
        const int c = idx / (D / 4);
        const int d4 = (idx % (D / 4)) * 4;
        const int tok = t0 + c % TQ;
        const int hl = head_lo + c / TQ;
        if (hl >= a.r || tok >= batch) continue;
        float mw[kWaves], lw[kWaves];
        float m_all = -INFINITY;
#pragma unroll
        for (int w = 0; w < kWaves; ++w) {
            mw[w] = ml[(w * kCols + c) * 2 + 0];
            lw[w] = ml[(w * kCols + c) * 2 + 1];
            m_all = fmaxf(m_all, mw[w]);
        }
        float l_all = 0.0f;
        f4 acc = f4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int w = 0; w < kWaves; ++w) {
            const float wgt = fast_exp2(mw[w] - m_all); // a wave that saw no visible row has m = -inf -> weight 0
            l_all += lw[w] * wgt;
            const f4 ow = *reinterpret_cast<const f4*>(smem + w * G::kWaveB + ((size_t)c * G::kOStride + d4) * 4);
            acc += ow * wgt;
        }
        const int head = kvh * a.r + hl;
        if (DECODE && a.n_splits > 1) {
            const size_t pi = (size_t)id * a.n_head + head;
            *reinterpret_cast<f4*>(a.part_o + pi * D + d4) = acc;
            if (d4 == 0) {
                a.part_ml[pi * 2 + 0] = m_all;
                a.part_ml[pi * 2 + 1] = l_all;
            }
        } else {
            const float inv = l_all > 0.0f ? 1.0f / l_all : 0.0f;
            *reinterpret_cast<f4*>(a.out + ((size_t)tok * a.n_head + head) * D + d4) = acc * inv;
        }
    }
}

// Log-sum-exp merge of the decode splits: one workgroup per query head.
template <int D>
__global__ __launch_bounds__(256) void fa_decode_combine_kernel(const FaArgs a) {
    constexpr int kGroups = 256 / D;
    __shared__ float sh_o[kGroups][D];
    __shared__ float sh_m[kGroups];
    __shared__ float sh_l[kGroups];
    const int head = blockIdx.x;
    const int d = threadIdx.x % D;
    const int sg = threadIdx.x / D;

    int p = *a.d_pos;
    p = p < 0 ? 0 : p;
    const int npos = (p > a.n_ctx - 1 ? a.n_ctx - 1 : p) + 1;
    const int n_tiles = (npos + kTile - 1) / kTile;
    const int tps = (n_tiles + a.n_splits - 1) / a.n_splits;
    const int n_active = (n_tiles + tps - 1) / tps;

    float m = -INFINITY, l = 0.0f, acc = 0.0f;
    for (int s = sg; s < n_active; s += kGroups) {
        const size_t pi = (size_t)s * a.n_head + head;
        const float ms = a.part_ml[pi * 2 + 0];
        const float ls = a.part_ml[pi * 2 + 1];
        const float os = a.part_o[pi * D + d];
        const float m_new = fmaxf(m, ms);
        const float wa = fast_exp2(m - m_new);
        const float wb = fast_exp2(ms - m_new);
        acc = acc * wa + os * wb;
        l = l * wa + ls * wb;
        m = m_new;
    }
    sh_o[sg][d] = acc;
    if (d == 0) {
        sh_m[sg] = m;
        sh_l[sg] = l;
    }
    __syncthreads();
    if (sg == 0) {
        float m_all = sh_m[0];
#pragma unroll
        for (int g = 1; g < kGroups; ++g) m_all = fmaxf(m_all, sh_m[g]);
        float l_all = 0.0f, o_all = 0.0f;
#pragma unroll
        for (int g = 0; g < kGroups; ++g) {
            const float w = fast_exp2(sh_m[g] - m_all); // a group with no split has m = -inf -> weight 0
            l_all += sh_l[g] * w;
            o_all += sh_o[g][d] * w;
        }
        a.out[(size_t)head * D + d] = l_all > 0.0f ? o_all / l_all : 0.0f;
    }
}

// ---------------------------------------------------------------------------
// host side
// ---------------------------------------------------------------------------

struct State {
    bool ready = false;
    int device = 0;
    int cu_count = 0;
    hipStream_t stream = nullptr;
    void* own_ws = nullptr; // allocated by init
    void* ws = nullptr;     // active workspace
    size_t ws_bytes = 0;
};
State g_state;

inline int hip_code(hipError_t e) { return e == hipSuccess ? ORIN_FA_OK : ORIN_FA_E_HIP - (int)e; }

template <int D, int NQB, int TQ, bool PRECISE, bool DECODE>
int launch_fwd(const FaArgs& a, int grid) {
    using G = Geom<D, NQB>;
    hipLaunchKernelGGL((fa_fwd_kernel<D, NQB, TQ, PRECISE, DECODE>), dim3(grid), dim3(kThreads), G::kLdsB,
                       g_state.stream, a);
    return hip_code(hipGetLastError());
}

// The kernels use more than 64 KB of dynamic LDS; the opt-in is set once per kernel at
// init so that no launch path touches function attributes (decode runs under capture).
template <int D, int NQB, int TQ, bool PRECISE, bool DECODE>
hipError_t allow_lds() {
    return hipFuncSetAttribute(reinterpret_cast<const void*>(fa_fwd_kernel<D, NQB, TQ, PRECISE, DECODE>),
                               hipFuncAttributeMaxDynamicSharedMemorySize, Geom<D, NQB>::kLdsB);
}

template <int D>
hipError_t allow_lds_all() {
    hipError_t e;
    if ((e = allow_lds<D, 1, 16, false, false>()) != hipSuccess) return e;
    if ((e = allow_lds<D, 2, 16, false, false>()) != hipSuccess) return e;
    if ((e = allow_lds<D, 3, 16, false, false>()) != hipSuccess) return e;
    if ((e = allow_lds<D, 4, 16, false, false>()) != hipSuccess) return e;
    if ((e = allow_lds<D, 3, 8, false, false>()) != hipSuccess) return e;
    if ((e = allow_lds<D, 4, 8, false, false>()) != hipSuccess) return e;
    return allow_lds<D, 1, 1, true, true>();
}

template <int D>
int launch_prefill(FaArgs a) {
    // Column packing per GQA ratio: (16-column blocks, tokens per workgroup).
    // r <= 4: 16 tokens x r heads; r in 5..8: 8 tokens x up to 8 heads; larger ratios
    // are cut into groups of 8 heads that each re-read the KV head.
    const int r = a.r;
    int nqb, tq;
    if (r <= 4) { nqb = r; tq = 16; }
    else if (r <= 6) { nqb = 3; tq = 8; }
    else { nqb = 4; tq = 8; }
    const int heads_per_group = nqb * 16 / tq;
    a.n_hgroups = (r + heads_per_group - 1) / heads_per_group;
    a.n_ttiles = (a.batch + tq - 1) / tq;
    const int grid = a.n_kv * a.n_hgroups * a.n_ttiles;
    switch (nqb * 100 + tq) {
        case 116: return launch_fwd<D, 1, 16, false, false>(a, grid);
        case 216: return launch_fwd<D, 2, 16, false, false>(a, grid);
        case 316: return launch_fwd<D, 3, 16, false, false>(a, grid);
        case 416: return launch_fwd<D, 4, 16, false, false>(a, grid);
        case 308: return launch_fwd<D, 3, 8, false, false>(a, grid);
        default:  return launch_fwd<D, 4, 8, false, false>(a, grid);
    }
}

int decode_splits(int n_head, int n_kv, int head_dim, int n_ctx) {
    const int r = n_head / n_kv;
    const int n_hgroups = (r + 15) / 16;
    const int cus = g_state.cu_count > 0 ? g_state.cu_count : 256;
    int s = (2 * cus) / (n_kv * n_hgroups);
    const int by_ctx = (n_ctx + kWaves * kTile - 1) / (kWaves * kTile);
    if (s > by_ctx) s = by_ctx;
    if (s > kMaxSplits) s = kMaxSplits;
    const size_t per_split = (size_t)n_head * (head_dim + 2) * sizeof(float);
    const size_t ws = g_state.ws ? g_state.ws_bytes : kWorkspaceBytes;
    if ((size_t)s * per_split > ws) s = (int)(ws / per_split);
    return s < 1 ? 1 : s;
}

template <int D>
int launch_decode(FaArgs a) {
    a.n_hgroups = (a.r + 15) / 16;
    a.n_splits = decode_splits(a.n_head, a.n_kv, D, a.n_ctx);
    if (a.n_splits > 1) {
        if (!g_state.ws) return ORIN_FA_E_WORKSPACE;
        a.part_o = static_cast<float*>(g_state.ws);
        a.part_ml = a.part_o + (size_t)a.n_splits * a.n_head * D;
    }
    const int grid = a.n_kv * a.n_hgroups * a.n_splits;
    int rc = launch_fwd<D, 1, 1, true, true>(a, grid);
    if (rc != ORIN_FA_OK || a.n_splits == 1) return rc;
    hipLaunchKernelGGL(fa_decode_combine_kernel<D>, dim3(a.n_head), dim3(256), 0, g_state.stream, a);
    return hip_code(hipGetLastError());
}

int check_common(const void* q, const void* kc, const void* vc, const void* out,
                 int n_head, int n_kv, int head_dim, int n_ctx) {
    if (!g_state.ready) return ORIN_FA_E_NOT_INIT;
    if (!q || !kc || !vc || !out) return ORIN_FA_E_INVALID;
    if (n_head <= 0 || n_kv <= 0 || n_ctx <= 0 || n_head % n_kv != 0) return ORIN_FA_E_INVALID;
    if (head_dim != 64 && head_dim != 128) return ORIN_FA_E_HEAD_DIM;
    if ((reinterpret_cast<uintptr_t>(q) | reinterpret_cast<uintptr_t>(kc) | reinterpret_cast<uintptr_t>(vc) |
         reinterpret_cast<uintptr_t>(out)) & 15u)
        return ORIN_FA_E_INVALID; // 128-bit loads and stores
    return ORIN_FA_OK;
}

} // namespace

extern "C" {

int orin_fa_init(int device) {
    hipError_t e = hipSetDevice(device);
    if (e != hipSuccess) {
        fprintf(stderr, "[orin_fa] hipSetDevice(%d) failed: %s\n", device, hipGetErrorString(e));
        return hip_code(e);
    }
    hipDeviceProp_t prop;
    e = hipGetDeviceProperties(&prop, device);
    if (e != hipSuccess) return hip_code(e);
    g_state.device = device;
    g_state.cu_count = prop.multiProcessorCount;
    if ((e = allow_lds_all<128>()) != hipSuccess) return hip_code(e);
    if ((e = allow_lds_all<64>()) != hipSuccess) return hip_code(e);
    if (!g_state.own_ws) {
        e = hipMalloc(&g_state.own_ws, kWorkspaceBytes);
        if (e != hipSuccess) return hip_code(e);
    }
    if (!g_state.ws) {
        g_state.ws = g_state.own_ws;
        g_state.ws_bytes = kWorkspaceBytes;
    }
    g_state.ready = true;
    return ORIN_FA_OK;
}

void orin_fa_set_stream(void* stream) { g_state.stream = static_cast<hipStream_t>(stream); }

size_t orin_fa_workspace_bytes(void) { return kWorkspaceBytes; }

int orin_fa_set_workspace(void* dev_ptr, size_t bytes) {
    if (!dev_ptr) { // back to the library's own block
        g_state.ws = g_state.own_ws;
        g_state.ws_bytes = g_state.own_ws ? kWorkspaceBytes : 0;
        return ORIN_FA_OK;
    }
    if ((reinterpret_cast<uintptr_t>(dev_ptr) & 255u) != 0) return ORIN_FA_E_INVALID;
    if (bytes < kWorkspaceBytes) return ORIN_FA_E_WORKSPACE;
    g_state.ws = dev_ptr;
    g_state.ws_bytes = bytes;
    return ORIN_FA_OK;
}

int orin_fa_prefill(const float* q, const uint16_t* kc, const uint16_t* vc, float* out,
                    int n_head, int n_kv, int head_dim, int n_ctx, int n_past, int batch, float scale) {
    int rc = check_common(q, kc, vc, out, n_head, n_kv, head_dim, n_ctx);
    if (rc != ORIN_FA_OK) return rc;
    if (batch < 0 || n_past < 0 || (long long)n_past + batch > n_ctx) return ORIN_FA_E_INVALID;
    if (batch == 0) return ORIN_FA_OK;
    FaArgs a{};
    a.q = q; a.kc = kc; a.vc = vc; a.out = out;
    a.n_head = n_head; a.n_kv = n_kv; a.n_ctx = n_ctx; a.n_past = n_past; a.batch = batch;
    a.r = n_head / n_kv;
    a.n_splits = 1;
    a.scale_log2e = scale * kLog2e;
    return head_dim == 128 ? launch_prefill<128>(a) : launch_prefill<64>(a);
}

int orin_fa_decode_ind(const float* q, const uint16_t* kc, const uint16_t* vc, float* out,
                       int n_head, int n_kv, int head_dim, int n_ctx, const int* d_pos, float scale) {
    int rc = check_common(q, kc, vc, out, n_head, n_kv, head_dim, n_ctx);
    if (rc != ORIN_FA_OK) return rc;
    if (!d_pos) return ORIN_FA_E_INVALID;
    FaArgs a{};
    a.q = q; a.kc = kc; a.vc = vc; a.out = out; a.d_pos = d_pos;
    a.n_head = n_head; a.n_kv = n_kv; a.n_ctx = n_ctx; a.batch = 1;
    a.r = n_head / n_kv;
    a.scale_log2e = scale * kLog2e;
    return head_dim == 128 ? launch_decode<128>(a) : launch_decode<64>(a);
}

int orin_fa_decode_splits(int n_head, int n_kv, int head_dim, int n_ctx) {
    if (n_head <= 0 || n_kv <= 0 || n_ctx <= 0 || n_head % n_kv != 0) return 0;
    if (head_dim != 64 && head_dim != 128) return 0;
    return decode_splits(n_head, n_kv, head_dim, n_ctx);
}

int orin_fa_cu_count(void) { return g_state.cu_count; }

const char* orin_fa_error_string(int code) {
    switch (code) {
        case ORIN_FA_OK: return "ok";
        case ORIN_FA_E_INVALID: return "invalid argument (shape, alignment or null pointer)";
        case ORIN_FA_E_HEAD_DIM: return "unsupported head_dim (64 and 128 only)";
        case ORIN_FA_E_WORKSPACE: return "split-KV workspace missing or too small";
        case ORIN_FA_E_NOT_INIT: return "orin_fa_init has not been called";
        default: break;
    }
    if (code <= ORIN_FA_E_HIP) return hipGetErrorString(static_cast<hipError_t>(ORIN_FA_E_HIP - code));
    return "unknown error";
}

} // extern "C"
