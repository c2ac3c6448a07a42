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
typedef _Float16 h4 __attribute__((ext_vector_type(4)));
typedef __fp16 fp16x4 __attribute__((ext_vector_type(4)));
typedef float f4 __attribute__((ext_vector_type(4)));

constexpr int kPrefillWaves = 4;      // waves per prefill workgroup (one per SIMD: the kernel fills the register file)
constexpr int kDecodeWaves = 8;       // waves per decode workgroup (two per SIMD, one workgroup per CU)
constexpr int kTile = 32;             // KV rows per wave tile
constexpr float kLog2e = 1.4426950408889634f;
// Softmax weights are computed against a reference maximum that is only moved when a
// tile's maximum exceeds it by more than kLazy (log2 units), so the O accumulators are
// rescaled on a handful of early tiles instead of every tile.  P = 2^(s - m_ref + kPShift)
// therefore lies in (0, 2^(kLazy + kPShift)] = (0, 2^15], inside fp16 range, and the
// common factor cancels in O / l.
constexpr float kLazy = 8.0f;
constexpr float kPShift = 7.0f;
constexpr float kUnsetRef = -1.0e30f; // prefill: reference maximum of a column that has seen no visible key yet
constexpr size_t kWorkspaceBytes = 8u << 20;
constexpr int kMaxSplits = 256;
#ifndef FA_PREFILL_KDIRECT
#define FA_PREFILL_KDIRECT 0
#endif
#ifndef FA_DECODE_KDIRECT
#define FA_DECODE_KDIRECT 1
#endif
constexpr bool kPrefillKDirect = FA_PREFILL_KDIRECT;
constexpr bool kDecodeKDirect = FA_DECODE_KDIRECT;

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
    float c;           // |scale| * log2(e), clamped away from zero
    float qsign;       // sign of scale, folded into Q
};

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

__device__ __forceinline__ float max2(float x, float y);
typedef unsigned u32x2 __attribute__((ext_vector_type(2)));
typedef unsigned u32x4 __attribute__((ext_vector_type(4)));

// All-reduce over the four 16-lane groups of a wave (lanes l, l^16, l^32, l^48) with the
// gfx950 lane-swap instructions: v_permlane32_swap exchanges the upper half of one register
// with the lower half of the other, v_permlane16_swap does the same for odd/even 16-lane rows.
__device__ __forceinline__ float xor_max(float v) {
    u32x2 s = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    v = fmaxf(__uint_as_float(s.x), __uint_as_float(s.y));
    s = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    return fmaxf(__uint_as_float(s.x), __uint_as_float(s.y));
}
__device__ __forceinline__ float xor_max_fast(float v) { // same, for inputs that are never NaN
    u32x2 s = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    float r = max2(__uint_as_float(s.x), __uint_as_float(s.y));
    s = __builtin_amdgcn_permlane16_swap(__float_as_uint(r), __float_as_uint(r), false, false);
    return max2(__uint_as_float(s.x), __uint_as_float(s.y));
}
__device__ __forceinline__ float xor_sum(float v) {
    u32x2 s = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    v = __uint_as_float(s.x) + __uint_as_float(s.y);
    s = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    return __uint_as_float(s.x) + __uint_as_float(s.y);
}

// 16-byte load through a buffer descriptor: the hardware returns zeros for offsets at or
// past the descriptor's byte count, so cache rows beyond the visible range (which may hold
// anything, NaN patterns included) are never fetched and need no branch.
__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void* base, unsigned bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, bytes, 0x00020000);
}
// (The whole offset travels in the vector operand: the scalar offset operand is not range-checked.)
// STREAM marks data that is read once (decode): the load carries the non-temporal hint so the
// stream does not displace useful lines in L2 / Infinity Cache (measured 5-7% faster).
template <bool STREAM>
__device__ __forceinline__ u32x4 buf_load16(__amdgpu_buffer_rsrc_t r, int byte_off) {
    return __builtin_amdgcn_raw_buffer_load_b128(r, byte_off, 0, STREAM ? 2 : 0);
}

// ds_read_b64_tr_b16: within each group of 16 lanes, lane i receives element (i % 4) of the
// 8 bytes addressed by lanes i/4, i/4 + 4, i/4 + 8, i/4 + 12 -- a 4x16 transpose on the way
// out of LDS.  With lane i pointing at row (i / 4), 8-byte column (i % 4) of a row-major
// fp16 tile, lane i ends up with rows 0..3 at column i: an MFMA operand whose k index runs
// down the tile's rows.
__device__ __forceinline__ h4 lds_read_tr(const unsigned char* p) {
    const fp16x4 t = __builtin_amdgcn_ds_read_tr16_b64_v4f16(
        (__attribute__((address_space(3))) fp16x4*)(p));
    return __builtin_bit_cast(h4, t);
}

// Orders this wave's LDS writes before its later LDS reads (lanes of one wave
// exchange data through the wave-private LDS slice).
__device__ __forceinline__ void wave_lds_sync() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

template <int D, int NQB, int NW, bool KDIRECT>
struct Geom {
    static constexpr int kSteps = D / 32;            // MFMA k-steps over head_dim
    static constexpr int kDBlk = D / 16;             // 16-wide output blocks over head_dim
    static constexpr int kRowBK = D * 2 + 16;        // bytes per K row in LDS (16 B pad: conflict-free b128 row reads)
    static constexpr int kRowBV = D * 2 + 32;        // bytes per V row in LDS (32 B pad: spreads the transposing reads)
    static constexpr int kChunksPerRow = D / 8;      // 16-byte chunks per KV row
    static constexpr int kLoads = kTile * kChunksPerRow / 64; // 16-byte loads per lane per matrix per tile
    static constexpr int kTileBK = kTile * kRowBK;   // bytes of one K tile in LDS
    static constexpr int kTileBV = kTile * kRowBV;   // bytes of one V tile in LDS
    static constexpr int kOStride = D + 4;           // floats per column in the merge buffer
    static constexpr int kMergeB = NQB * 16 * kOStride * 4;
    static constexpr int kTilesB = (KDIRECT ? 0 : kTileBK) + kTileBV; // K skips LDS when it is loaded in operand order
    static constexpr int kWaveB = (kTilesB > kMergeB) ? kTilesB : kMergeB;
    static constexpr int kMlOff = NW * kWaveB;       // (m, l) per wave per column follow the wave slices
    static constexpr int kLdsB = kMlOff + NW * NQB * 16 * 2 * 4;
};

// D: head_dim; NQB: 16-column query blocks per workgroup; TQ: tokens per workgroup
// (column c = local_head * TQ + local_token); PRECISE: carry Q and P as fp16 hi+lo
// pairs (decode, where the matrix pipe is idle anyway); DECODE: position from *d_pos,
// KV splits across workgroups, partial outputs.
template <int D, int NQB, int TQ, bool PRECISE, bool DECODE, bool KDIRECT>
__global__ __launch_bounds__((DECODE ? kDecodeWaves : kPrefillWaves) * 64) void fa_fwd_kernel(const FaArgs a) {
    constexpr int kWaves = DECODE ? kDecodeWaves : kPrefillWaves;
    constexpr int kThreads = kWaves * 64;
    using G = Geom<D, NQB, kWaves, KDIRECT>;
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
    // Wave w of split s takes tiles s*4 + w, then every (4 * n_splits)-th tile after it.
    const int tile_first = (DECODE ? id * kWaves : 0) + wave;
    const int tile_step = DECODE ? kWaves * a.n_splits : kWaves;
    if (DECODE && id * kWaves >= n_tiles) return; // inactive split: the combine kernel never reads it

    unsigned char* const ks = smem + wave * G::kWaveB;
    unsigned char* const vs = ks + (KDIRECT ? 0 : G::kTileBK);
    const __amdgpu_buffer_rsrc_t krs = make_rsrc(a.kc + (size_t)kvh * a.n_ctx * D, (unsigned)kv_end * D * 2);
    const __amdgpu_buffer_rsrc_t vrs = make_rsrc(a.vc + (size_t)kvh * a.n_ctx * D, (unsigned)kv_end * D * 2);

    // K: either coalesced 16-byte chunks bound for LDS, or (KDIRECT) straight into MFMA A-operand
    // order -- lane (col, grp) takes row t*16 + col, bytes (kk*4 + grp)*16 .. +16 -- so that the
    // score product needs no LDS round trip.  V always goes through LDS (it is read transposed).
    constexpr int kKRegs = KDIRECT ? 2 * G::kSteps : G::kLoads;
    u32x4 kreg[kKRegs], vreg[G::kLoads];
    auto fetch_k = [&](int tile) {
        const int soff = tile * kTile * D * 2;
        if (KDIRECT) {
#pragma unroll
            for (int t = 0; t < 2; ++t)
#pragma unroll
                for (int kk = 0; kk < G::kSteps; ++kk)
                    kreg[t * G::kSteps + kk] = buf_load16<DECODE>(krs, soff + (t * 16 + col) * D * 2 + (kk * 4 + grp) * 16);
        } else {
#pragma unroll
            for (int i = 0; i < G::kLoads; ++i) kreg[i] = buf_load16<DECODE>(krs, soff + (i * 64 + lane) * 16);
        }
    };
    auto fetch_v = [&](int tile) {
        const int soff = tile * kTile * D * 2;
#pragma unroll
        for (int i = 0; i < G::kLoads; ++i) vreg[i] = buf_load16<DECODE>(vrs, soff + (i * 64 + lane) * 16);
    };
    int tile = tile_first;
    if (tile < n_tiles) { // in flight while the query columns are loaded and converted
        fetch_k(tile);
        fetch_v(tile);
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
        const float qmul = valid ? a.qsign : 0.0f;
#pragma unroll
        for (int kk = 0; kk < G::kSteps; ++kk) {
            const float4 x0 = *reinterpret_cast<const float4*>(qp + kk * 32 + grp * 8);
            const float4 x1 = *reinterpret_cast<const float4*>(qp + kk * 32 + grp * 8 + 4);
            const float x[8] = {x0.x, x0.y, x0.z, x0.w, x1.x, x1.y, x1.z, x1.w};
            h8 hi, lo;
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const float xe = x[e] * qmul;
                hi[e] = (_Float16)xe;
                lo[e] = (_Float16)(xe - (float)hi[e]);
            }
            qhi[qb][kk] = hi;
            if (PRECISE) qlo[qb][kk] = lo;
        }
    }

    // m_ref: reference maximum of the raw scores (S units, before the scale); l_run: this lane's
    // share of the row sum; o: O^T accumulators, lane (col, grp) holds head_dim rows db*16 + grp*4 + i.
    float m_ref[NQB], l_run[NQB];
    f4 o[NQB][G::kDBlk];
#pragma unroll
    for (int qb = 0; qb < NQB; ++qb) {
        m_ref[qb] = -INFINITY;
        l_run[qb] = 0.0f;
#pragma unroll
        for (int db = 0; db < G::kDBlk; ++db) o[qb][db] = f4{0.f, 0.f, 0.f, 0.f};
    }

    // per-lane LDS read offsets
    const int k_rd = col * G::kRowBK + grp * 16;                              // + t*16 rows, + kk*64 bytes
    const int v_rd = (grp * 4 + (col >> 2)) * G::kRowBV + (col & 3) * 8;      // + h*16 rows, + db*32 bytes

    for (; tile < n_tiles; tile += tile_step) {
        const bool more = tile + tile_step < n_tiles;
        // registers -> this wave's LDS slice
#pragma unroll
        for (int i = 0; i < G::kLoads; ++i) {
            const int c = i * 64 + lane;
            if (!KDIRECT)
                *reinterpret_cast<u32x4*>(ks + (c / G::kChunksPerRow) * G::kRowBK + (c % G::kChunksPerRow) * 16) = kreg[i];
            *reinterpret_cast<u32x4*>(vs + (c / G::kChunksPerRow) * G::kRowBV + (c % G::kChunksPerRow) * 16) = vreg[i];
        }
        if (!KDIRECT && more) fetch_k(tile + tile_step);
        if (more) fetch_v(tile + tile_step);
        wave_lds_sync();

        // ---- S^T = K Q^T : rows = KV row (sub-tile t, row col), columns = query column ----
        f4 s[2][NQB];
        f4 s2[PRECISE ? 2 : 1][PRECISE ? NQB : 1]; // the Q-lo product runs as its own accumulation chain
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int qb = 0; qb < NQB; ++qb) {
                s[t][qb] = f4{0.f, 0.f, 0.f, 0.f};
                if (PRECISE) s2[t][qb] = f4{0.f, 0.f, 0.f, 0.f};
            }
#pragma unroll
        for (int kk = 0; kk < G::kSteps; ++kk) {
#pragma unroll
            for (int t = 0; t < 2; ++t) {
                h8 ka;
                if (KDIRECT) ka = __builtin_bit_cast(h8, kreg[t * G::kSteps + kk]);
                else ka = *reinterpret_cast<const h8*>(ks + k_rd + t * 16 * G::kRowBK + kk * 64);
#pragma unroll
                for (int qb = 0; qb < NQB; ++qb) {
                    s[t][qb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(ka, qhi[qb][kk], s[t][qb], 0, 0, 0);
                    if (PRECISE) s2[t][qb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(ka, qlo[qb][kk], s2[t][qb], 0, 0, 0);
                }
            }
        }
        if (PRECISE) {
#pragma unroll
            for (int t = 0; t < 2; ++t)
#pragma unroll
                for (int qb = 0; qb < NQB; ++qb) s[t][qb] += s2[t][qb];
        }
        if (KDIRECT && more) fetch_k(tile + tile_step); // the operand registers are free again

        // ---- softmax weights; lane (col, grp) holds rows t*16 + grp*4 + i of its column ----
        const bool need_mask = (tile * kTile + kTile > full_end);
        h8 phi[NQB];
        h8 plo[PRECISE ? NQB : 1];
#pragma unroll
        for (int qb = 0; qb < NQB; ++qb) {
            float v[8];
#pragma unroll
            for (int t = 0; t < 2; ++t)
#pragma unroll
                for (int i = 0; i < 4; ++i) v[t * 4 + i] = s[t][qb][i];
            if (need_mask) {
#pragma unroll
                for (int t = 0; t < 2; ++t)
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        const int row = tile * kTile + t * 16 + grp * 4 + i;
                        if (row >= limit[qb]) v[t * 4 + i] = -INFINITY;
                    }
            }
            float mx = fmaxf(fmaxf(v[0], v[1]), v[2]);
            mx = fmaxf(fmaxf(mx, v[3]), v[4]);
            mx = fmaxf(fmaxf(mx, v[5]), v[6]);
            mx = xor_max(fmaxf(mx, v[7]));
            // move the reference only when this tile's maximum is far above it (or it is unset)
            const bool move = (mx - m_ref[qb]) * a.c > kLazy || (m_ref[qb] == -INFINITY && mx > -INFINITY);
            if (__builtin_amdgcn_ballot_w64(move) != 0) {
                const float alpha = move ? fast_exp2((m_ref[qb] - mx) * a.c) : 1.0f; // unset reference -> 0
                if (move) m_ref[qb] = mx;
                l_run[qb] *= alpha;
#pragma unroll
                for (int db = 0; db < G::kDBlk; ++db) o[qb][db] *= alpha;
            }
            // exponent = s*c - m_ref*c + shift; a column that has seen no visible row keeps weight 0
            const float nb = (m_ref[qb] == -INFINITY) ? kPShift : kPShift - m_ref[qb] * a.c;
            float sum = 0.0f;
            h8 ph, pl;
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const float p = fast_exp2(__builtin_fmaf(v[e], a.c, nb));
                sum += p;
                ph[e] = (_Float16)p;
                pl[e] = (_Float16)(p - (float)ph[e]);
            }
            l_run[qb] += sum;
            phi[qb] = ph;
            if (PRECISE) plo[qb] = pl;
        }

        // ---- O^T += V^T P : rows = head_dim index, columns = query column, k = the tile's 32 KV rows
        //      in the order (grp, t, i) that matches the layout P already has.  The LDS transpose
        //      read hands lane (col, grp) the four rows h*16 + grp*4 + 0..3 at head_dim index db*16 + col. ----
#pragma unroll
        for (int db = 0; db < G::kDBlk; ++db) {
            const h4 v0 = lds_read_tr(vs + v_rd + db * 32);
            const h4 v1 = lds_read_tr(vs + v_rd + 16 * G::kRowBV + db * 32);
            const h8 va = __builtin_shufflevector(v0, v1, 0, 1, 2, 3, 4, 5, 6, 7);
#pragma unroll
            for (int qb = 0; qb < NQB; ++qb) {
                o[qb][db] = __builtin_amdgcn_mfma_f32_16x16x32_f16(va, phi[qb], o[qb][db], 0, 0, 0);
                if (PRECISE) o[qb][db] = __builtin_amdgcn_mfma_f32_16x16x32_f16(va, plo[qb], o[qb][db], 0, 0, 0);
            }
        }
        wave_lds_sync(); // the slice is overwritten at the top of the next iteration
    }

    float m_run[NQB]; // reference maximum in log2 units, as the merge steps expect
#pragma unroll
    for (int qb = 0; qb < NQB; ++qb) m_run[qb] = (m_ref[qb] == -INFINITY) ? -INFINITY : m_ref[qb] * a.c;

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

// ---------------------------------------------------------------------------
// Prefill: software-pipelined kernel.
//
// Same decomposition as above (4 waves split the KV tiles of one KV head between them and
// share a block of NQB*16 query columns), but the three stages of a tile
//     A: S = K Q^T (MFMA)      B: P = 2^(S*c - m) (VALU)      C: O += V^T P (MFMA)
// run skewed -- iteration t issues A(t+1), B(t) and C(t-1), which are independent of one
// another, so the matrix pipe works while the vector pipe exponentiates.  K rows are loaded
// straight into MFMA operand order (two register sets, filled two tiles ahead); V tiles are
// copied global->LDS by the load unit itself (no staging registers, two buffers per wave) in
// an XOR-swizzled layout that both the 1 KB copy bursts and the transposing reads hit
// conflict-free.  Each wave walks its tiles from the diagonal backwards, so the only tile
// that can need the causal mask is handled in the prologue and the steady state is mask-free.
// ---------------------------------------------------------------------------
template <int D, int NQB>
struct PGeom {
    static constexpr int kSteps = D / 32;
    static constexpr int kDBlk = D / 16;
    static constexpr int kRowB = D * 2;               // bytes per K/V row in LDS (no padding; chunks are XOR-swizzled)
    static constexpr int kChunks = D / 8;             // 16-byte chunks per row
    static constexpr int kTileB = kTile * kRowB;      // one K or V tile
    static constexpr int kCopies = kTileB / 1024;     // one LDS copy instruction moves 64 lanes x 16 B
    static constexpr int kRowsPerCopy = 1024 / kRowB; // 4 (d=128) or 8 (d=64)
    static constexpr int kKOff = 0;                   // wave slice: K buffers 0/1, then V buffers 0/1
    static constexpr int kVOff = 2 * kTileB;
    static constexpr int kOStride = D + 4;
    static constexpr int kMergeB = NQB * 16 * kOStride * 4;
    static constexpr int kScratchOff = 4 * kTileB;    // 1 KB per wave: 16 bytes per lane for the rare O rescale
    static constexpr int kWaveB = (4 * kTileB + 1024 > kMergeB) ? 4 * kTileB + 1024 : kMergeB;
    static constexpr int kMlOff = kPrefillWaves * kWaveB;
    static constexpr int kLdsB = kMlOff + kPrefillWaves * NQB * 16 * 2 * 4;
};

template <int N> struct IntC { static constexpr int value = N; };

// Matrix instructions with the register file of each operand spelled out.  The prefill kernel
// keeps its score accumulators in ordinary vector registers (the exponentials read them with no
// copy) and its output accumulators in the accumulation-register file, and it fixes the issue
// order of matrix and vector work by hand -- neither of which the builtin form allows.  The
// price: the compiler knows nothing about the hazards of these.  (1) Result latency: every place
// where a non-matrix instruction reads an accumulator is either a pipeline stage away or behind
// settle().  (2) A matrix instruction must not read an operand in the two cycles after a vector
// instruction wrote it, and the compiler is free to sink such a write (the fp16 conversion of P,
// a register copy) right in front of the asm block: each block starts with the two wait states.
__device__ __forceinline__ void mfma_v(f4& acc, h8 a_op, h8 b_op) {
    asm volatile("s_nop 1\n\tv_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+v"(acc) : "v"(a_op), "v"(b_op));
}
__device__ __forceinline__ void mfma_v_zero(f4& acc, h8 a_op, h8 b_op) { // acc = A B
    // early clobber: the destination must not share registers with an operand that dies here
    asm volatile("s_nop 1\n\tv_mfma_f32_16x16x32_f16 %0, %1, %2, 0" : "=&v"(acc) : "v"(a_op), "v"(b_op));
}
__device__ __forceinline__ void mfma_a(f4& acc, h8 a_op, h8 b_op) {
    asm volatile("s_nop 1\n\tv_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+a"(acc) : "v"(a_op), "v"(b_op));
}
// Lets the matrix pipe drain (32 wait states, more than any 16x16x32 result needs) and stops the
// compiler from moving anything across.
__device__ __forceinline__ void settle() {
    __builtin_amdgcn_sched_barrier(0);
    asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");
    __builtin_amdgcn_sched_barrier(0);
}
// 16 bytes between LDS and the accumulation-register file, without a detour through vector
// registers.  The output accumulators of the prefill kernel are only ever touched by these and
// by mfma_a, which keeps them in that file for the whole kernel.
__device__ __forceinline__ void lds_store_acc(unsigned lds_addr, const f4& acc) {
    asm volatile("ds_write_b128 %0, %1\n\ts_waitcnt lgkmcnt(0)" : : "v"(lds_addr), "a"(acc) : "memory");
}
__device__ __forceinline__ void lds_load_acc(f4& acc, unsigned lds_addr) {
    asm volatile("s_waitcnt lgkmcnt(0)\n\tds_read_b128 %0, %1\n\ts_waitcnt lgkmcnt(0)" : "=a"(acc) : "v"(lds_addr) : "memory");
}
template <int I, int N, class F>
__device__ __forceinline__ void static_for(F&& f) {
    if constexpr (I < N) {
        f(IntC<I>{});
        static_for<I + 1, N>(f);
    }
}

// three-input maximum without the NaN-quieting moves the library fmaxf carries
__device__ __forceinline__ float max3(float x, float y, float z) {
    float r;
    asm("v_max3_f32 %0, %1, %2, %3" : "=v"(r) : "v"(x), "v"(y), "v"(z));
    return r;
}
// (trailing wait state: the result may feed a lane-swap instruction, which must not read a
// register in the cycle after a vector instruction wrote it, and the compiler cannot see that
// this block is one)
__device__ __forceinline__ float max2(float x, float y) {
    float r;
    asm("v_max_f32 %0, %1, %2\n\ts_nop 1" : "=v"(r) : "v"(x), "v"(y));
    return r;
}

typedef int i32x4 __attribute__((ext_vector_type(4)));

// Buffer descriptor words for the global->LDS copies below: base address, stride 0, byte
// count, raw 32-bit format.  Offsets at or past the byte count are not fetched.
__device__ __forceinline__ i32x4 make_desc(const void* base, unsigned bytes) {
    const unsigned long long b = reinterpret_cast<unsigned long long>(base);
    return i32x4{(int)(unsigned)b, (int)((unsigned)(b >> 32) & 0xffffu), (int)bytes, 0x00020000};
}

// Four 1 KB global->LDS copies (buffer_load ... lds): lane l of copy i fetches 16 bytes at
// global offset off_i + i*1024 and the load unit writes them to LDS byte lds_base + i*1024 +
// l*16 (the immediate offset advances both addresses).  They count on the vector-memory
// counter and complete in issue order; callers wait with s_waitcnt vmcnt(n).  Written as one
// asm block so that M0 (the LDS base) cannot change between the copies.
__device__ __forceinline__ void lds_copy_4k(i32x4 desc, unsigned lds_base, int off_even, int off_odd) {
    asm volatile(
        "s_mov_b32 m0, %0\n\t"
        "buffer_load_dwordx4 %1, %3, 0 offen lds\n\t"
        "buffer_load_dwordx4 %2, %3, 0 offen offset:1024 lds\n\t"
        "buffer_load_dwordx4 %1, %3, 0 offen offset:2048 lds\n\t"
        "buffer_load_dwordx4 %2, %3, 0 offen offset:3072 lds"
        :
        : "s"(lds_base), "v"(off_even), "v"(off_odd), "s"(desc)
        : "memory", "m0");
}

template <int D, int NQB, int TQ>
__global__ __launch_bounds__(kPrefillWaves * 64) void fa_prefill_kernel(const FaArgs a) {
    using G = PGeom<D, NQB>;
    constexpr int kWaves = kPrefillWaves;
    constexpr int kThreads = kWaves * 64;
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];

    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int col = lane & 15;
    const int grp = lane >> 4;

    int id = blockIdx.x;
    const int kvh = id % a.n_kv;
    id /= a.n_kv;
    const int hg = id % a.n_hgroups;
    id /= a.n_hgroups;
    const int n_past = a.n_past, batch = a.batch;
    const int t0 = (a.n_ttiles - 1 - id) * TQ; // longest rows first
    constexpr int kHeadsPerGroup = NQB * 16 / TQ;
    const int head_lo = hg * kHeadsPerGroup;
    const int tok_hi = (t0 + TQ < batch) ? t0 + TQ : batch;
    const int kv_end = n_past + tok_hi;
    const int full_end = n_past + t0 + 1;
    const int n_tiles = (kv_end + kTile - 1) / kTile;
    // Wave w owns tiles w, w+4, ...; step j visits them from the highest down.  Steps past the
    // end map to negative tiles, whose copies fall outside the buffer descriptor and fetch nothing.
    const int n_mine = n_tiles > wave ? (n_tiles - 1 - wave) / kWaves + 1 : 0;
    auto tile_of = [&](int j) { return wave + kWaves * (n_mine - 1 - j); };

    unsigned char* const ws = smem + wave * G::kWaveB; // this wave's LDS slice
    // wave-uniform by construction; readfirstlane tells the compiler so (it has to live in a scalar register)
    const unsigned ws_addr = __builtin_amdgcn_readfirstlane(
        (unsigned)(size_t)(__attribute__((address_space(3))) unsigned char*)ws);
    const i32x4 kdesc = make_desc(a.kc + (size_t)kvh * a.n_ctx * D, (unsigned)kv_end * D * 2);
    const i32x4 vdesc = make_desc(a.vc + (size_t)kvh * a.n_ctx * D, (unsigned)kv_end * D * 2);

    // ---- per-lane offsets ----
    // Copy: lane l of copy i lands at LDS byte i*1024 + l*16 = row i*R + l/C, physical chunk l%C,
    // and physical chunk p of row r holds logical chunk p ^ (r & 7).
    int g_off[2];
    {
        const int r_in = lane / G::kChunks, pc = lane % G::kChunks;
#pragma unroll
        for (int par = 0; par < 2; ++par) {
            const int sw = (par * G::kRowsPerCopy + r_in) & 7;
            g_off[par] = r_in * G::kRowB + ((pc ^ sw) & (G::kChunks - 1)) * 16;
        }
    }
    constexpr int kOdd = (G::kRowsPerCopy == 4) ? 1 : 0;
    // K operand read: lane (col, grp) takes row t*16 + col, logical chunk kk*4 + grp.
    int k_rd[G::kSteps];
#pragma unroll
    for (int kk = 0; kk < G::kSteps; ++kk) k_rd[kk] = col * G::kRowB + (((kk * 4 + grp) ^ (col & 7)) * 16);
    // V transposing read: lane (col, grp) addresses row grp*4 + col/4 (+16 for the second half),
    // 8-byte column db*4 + col%4.
    int v_rd[G::kDBlk];
    {
        const int r0 = grp * 4 + (col >> 2), sw = r0 & 7;
#pragma unroll
        for (int db = 0; db < G::kDBlk; ++db)
            v_rd[db] = r0 * G::kRowB + (((db * 2 + ((col & 3) >> 1)) ^ sw) * 16) + (col & 1) * 8;
    }

    auto copy_tile = [&](i32x4 desc, unsigned lds_dst, int tile) { // kCopies (4 or 8) copies
        const int base = tile * G::kTileB;
        lds_copy_4k(desc, lds_dst, base + g_off[0], base + g_off[kOdd]);
        if (G::kCopies > 4) lds_copy_4k(desc, lds_dst + 4096, base + 4096 + g_off[0], base + 4096 + g_off[kOdd]);
    };
    auto fetch_k = [&](auto par, int tile) { copy_tile(kdesc, ws_addr + G::kKOff + decltype(par)::value * G::kTileB, tile); };
    auto fetch_v = [&](auto par, int tile) { copy_tile(vdesc, ws_addr + G::kVOff + decltype(par)::value * G::kTileB, tile); };

    // ---- state ----
    h8 q[NQB][G::kSteps];
    int limit[NQB];
    float m_ref[NQB], l_run[NQB];
    f4 o[NQB][G::kDBlk];
    f4 s[2][2][NQB]; // [parity][sub-tile][query block]
    h8 pw[2][NQB];   // [parity][query block]
    // Zero the slice once: a copy whose rows lie past the visible range fetches nothing, and must
    // not expose stale bit patterns (their weights are zero, and 0 * NaN is not).  The output
    // accumulators are cleared from the same zeros.
#pragma unroll
    for (int i = 0; i < (4 * G::kTileB + 1024) / 1024; ++i)
        *reinterpret_cast<u32x4*>(ws + i * 1024 + lane * 16) = u32x4{0u, 0u, 0u, 0u};
    __builtin_amdgcn_s_waitcnt(0xC07F); // lgkmcnt(0): the zero fill is done before the first copy can land
    wave_lds_sync();
    const unsigned scratch_addr = (unsigned)(size_t)(__attribute__((address_space(3))) unsigned char*)(ws + G::kScratchOff) + lane * 16;
#pragma unroll
    for (int qb = 0; qb < NQB; ++qb) {
        m_ref[qb] = kUnsetRef;
        l_run[qb] = 0.0f;
#pragma unroll
        for (int db = 0; db < G::kDBlk; ++db) lds_load_acc(o[qb][db], scratch_addr);
    }

    auto stage_a = [&](auto kpar, auto spar) { // S[spar] = K[kpar] Q^T (prologue form: not interleaved)
        constexpr int KP = decltype(kpar)::value, SP = decltype(spar)::value;
        const unsigned char* const kb = ws + G::kKOff + KP * G::kTileB;
#pragma unroll
        for (int kk = 0; kk < G::kSteps; ++kk)
#pragma unroll
            for (int t = 0; t < 2; ++t) {
                const h8 ka = *reinterpret_cast<const h8*>(kb + t * 16 * G::kRowB + k_rd[kk]);
#pragma unroll
                for (int qb = 0; qb < NQB; ++qb) {
                    if (kk == 0) mfma_v_zero(s[SP][t][qb], ka, q[qb][kk]);
                    else mfma_v(s[SP][t][qb], ka, q[qb][kk]);
                    // With few query blocks the next k-step of the same accumulator is only a
                    // couple of instructions away; give the result time to leave the pipe.
                    if (2 * NQB < 8) asm volatile("s_nop 15");
                }
            }
    };

    float alpha[NQB];
    // P[par] = 2^(S[par]*c - m_ref*c + shift); returns whether any column moved its reference
    auto stage_b = [&](auto par, auto masked, int tile) -> bool {
        constexpr int P = decltype(par)::value;
        bool any_move = false;
#pragma unroll
        for (int qb = 0; qb < NQB; ++qb) {
            float v[8];
#pragma unroll
            for (int t = 0; t < 2; ++t)
#pragma unroll
                for (int i = 0; i < 4; ++i) v[t * 4 + i] = s[P][t][qb][i];
            if (decltype(masked)::value) {
#pragma unroll
                for (int t = 0; t < 2; ++t)
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        const int row = tile * kTile + t * 16 + grp * 4 + i;
                        if (row >= limit[qb]) v[t * 4 + i] = -INFINITY;
                    }
            }
            float mx = max3(v[0], v[1], v[2]);
            mx = max3(mx, v[3], v[4]);
            mx = max3(mx, v[5], v[6]);
            mx = xor_max_fast(max2(mx, v[7]));
            const bool move = (mx - m_ref[qb]) * a.c > kLazy; // an unset reference is far below any score
            alpha[qb] = fast_exp2(move ? (m_ref[qb] - mx) * a.c : 0.0f);
            m_ref[qb] = move ? mx : m_ref[qb];
            any_move |= move;
            const float nb = kPShift - m_ref[qb] * a.c;
            float sum = 0.0f;
            h8 ph;
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const float p = fast_exp2(__builtin_fmaf(v[e], a.c, nb));
                sum += p;
                ph[e] = (_Float16)p;
            }
            l_run[qb] = l_run[qb] * alpha[qb] + sum;
            pw[P][qb] = ph;
        }
        return __builtin_amdgcn_ballot_w64(any_move) != 0;
    };

    auto stage_c = [&](auto par) { // O += V[par]^T P[par]
        constexpr int P = decltype(par)::value;
        const unsigned char* const vb = ws + G::kVOff + P * G::kTileB;
#pragma unroll
        for (int db = 0; db < G::kDBlk; ++db) {
            const h4 v0 = lds_read_tr(vb + v_rd[db]);
            const h4 v1 = lds_read_tr(vb + 16 * G::kRowB + v_rd[db]);
            const h8 va = __builtin_shufflevector(v0, v1, 0, 1, 2, 3, 4, 5, 6, 7);
#pragma unroll
            for (int qb = 0; qb < NQB; ++qb) mfma_a(o[qb][db], va, pw[P][qb]);
        }
    };
    // Rare (a column's reference maximum moved): O *= alpha, one accumulator at a time through a
    // 16-byte-per-lane LDS scratch so that O never becomes an operand of an ordinary vector instruction.
    auto rescale = [&]() {
        settle(); // the last accumulation into O has left the matrix pipe
        f4* const scratch = reinterpret_cast<f4*>(ws + G::kScratchOff) + lane;
#pragma unroll
        for (int qb = 0; qb < NQB; ++qb)
#pragma unroll
            for (int db = 0; db < G::kDBlk; ++db) {
                lds_store_acc(scratch_addr, o[qb][db]);
                f4 x = *scratch;
                x *= alpha[qb];
                *scratch = x;
                lds_load_acc(o[qb][db], scratch_addr);
            }
        settle();
    };
    // The copies are tracked by the vector-memory counter and complete in issue order: waiting
    // until at most `newer` younger ones are outstanding guarantees a tile has landed.
    auto wait_copies = [&](auto newer) {
        constexpr int n = decltype(newer)::value;
        __builtin_amdgcn_s_waitcnt(0x0F70 | (n & 15) | ((n >> 4) << 14)); // vmcnt(n), other counters untouched
        wave_lds_sync();
    };
    constexpr int kC = G::kCopies;

    if (n_mine > 0) {
        fetch_k(IntC<0>{}, tile_of(0));
        fetch_v(IntC<0>{}, tile_of(0));
        fetch_k(IntC<1>{}, tile_of(1));
        fetch_v(IntC<1>{}, tile_of(1));

        // ---- query columns -> B operands ----
#pragma unroll
        for (int qb = 0; qb < NQB; ++qb) {
            const int c = qb * 16 + col;
            const int tok = t0 + c % TQ;
            const int hl = head_lo + c / TQ;
            const bool valid = (hl < a.r) && (tok < batch);
            limit[qb] = valid ? n_past + tok + 1 : 0x7fffffff;
            const float* qp = a.q + ((size_t)(valid ? tok : 0) * a.n_head + (size_t)(valid ? kvh * a.r + hl : 0)) * D;
            const float qmul = valid ? a.qsign : 0.0f;
#pragma unroll
            for (int kk = 0; kk < G::kSteps; ++kk) {
                const float4 x0 = *reinterpret_cast<const float4*>(qp + kk * 32 + grp * 8);
                const float4 x1 = *reinterpret_cast<const float4*>(qp + kk * 32 + grp * 8 + 4);
                const float x[8] = {x0.x, x0.y, x0.z, x0.w, x1.x, x1.y, x1.z, x1.w};
                h8 hv;
#pragma unroll
                for (int e = 0; e < 8; ++e) hv[e] = (_Float16)(x[e] * qmul);
                q[qb][kk] = hv;
            }
        }

        // Copy issue order: K0 V0 K1 V1 | K2 (step 0) | K3 V2 (step 1) | K4 V3 (step 2) | ...
        // ---- step 0: the diagonal tile, the only one that can need the causal mask ----
        const int R = n_mine - 1; // steps after step 0
        wait_copies(IntC<3 * kC>{});               // K0 landed (V0 K1 V1 may be in flight)
        stage_a(IntC<0>{}, IntC<0>{});             // S(0)
        __builtin_amdgcn_s_waitcnt(0xC07F);        // its LDS reads have returned: K buffer 0 is free
        fetch_k(IntC<0>{}, tile_of(2));
        if (R > 0) {
            wait_copies(IntC<2 * kC>{});           // K1 landed (V1 K2 may be in flight)
            stage_a(IntC<1>{}, IntC<1>{});         // S(1)
        }
        settle();
        if (tile_of(0) * kTile + kTile > full_end) stage_b(IntC<0>{}, IntC<1>{}, tile_of(0));
        else stage_b(IntC<0>{}, IntC<0>{}, tile_of(0));
        // (O is still zero: no rescale)

        // ---- steps t >= 1: A(t+1), B(t) and C(t-1) share one hand-ordered instruction stream.
        // The 2 * kGroups/2 * NQB matrix instructions of A and C are cut into groups of NQB that
        // share an LDS operand (A: one (k-step, sub-tile) of K; C: one 16-wide block of V^T),
        // ordered A0 C0 A1 C1 ...; the vector work of B is cut into 16 sites per query block and
        // each site is followed by its share of the matrix instructions, so the matrix pipe is
        // fed while the exponentials run.  Operands are read from LDS two groups ahead.
        // `newer` = copies issued after K(t+1): K(t+2) only at t == 1 (step 0 issued no V),
        // V(t) and K(t+2) afterwards. ----
        constexpr int kGroups = 2 * G::kSteps + G::kDBlk; // 2*kSteps == kDBlk
        static_assert(2 * G::kSteps == G::kDBlk, "A and C groups alternate one to one");
        auto body = [&](auto tpar, auto has_next, auto newer, int t) {
            constexpr int TP = decltype(tpar)::value; // t & 1
            constexpr bool HN = decltype(has_next)::value;
            // (Every LDS read of the previous step has been consumed by a matrix instruction that
            // was issued before this point, so the K buffer A(t) read is free.)
            fetch_k(IntC<TP>{}, tile_of(t + 2));                       // K(t+2) -> the buffer A(t) read
            wait_copies(newer);                                         // K(t+1) landed; V(t-1) is older
            const unsigned char* const kb = ws + G::kKOff + (TP ^ 1) * G::kTileB;
            const unsigned char* const vb = ws + G::kVOff + (TP ^ 1) * G::kTileB;
            h8 gop[kGroups];
            auto issue_read = [&](auto gc) {
                constexpr int g = decltype(gc)::value;
                if constexpr (g % 2 == 0) {
                    constexpr int kk = (g / 2) / 2, tt = (g / 2) % 2;
                    if (HN) gop[g] = *reinterpret_cast<const h8*>(kb + tt * 16 * G::kRowB + k_rd[kk]);
                } else {
                    constexpr int db = g / 2;
                    const h4 v0 = lds_read_tr(vb + v_rd[db]);
                    const h4 v1 = lds_read_tr(vb + 16 * G::kRowB + v_rd[db]);
                    gop[g] = __builtin_shufflevector(v0, v1, 0, 1, 2, 3, 4, 5, 6, 7);
                }
            };
            auto ticket = [&](auto ic) {
                constexpr int i = decltype(ic)::value;
                constexpr int g = i / NQB, m = i % NQB;
                if constexpr (m == 0 && g + 2 < kGroups) issue_read(IntC<g + 2>{});
                if constexpr (g % 2 == 0) {
                    constexpr int kk = (g / 2) / 2, tt = (g / 2) % 2;
                    if (HN) {
                        if constexpr (kk == 0) mfma_v_zero(s[TP ^ 1][tt][m], gop[g], q[m][kk]);
                        else mfma_v(s[TP ^ 1][tt][m], gop[g], q[m][kk]);
                    }
                } else {
                    mfma_a(o[m][g / 2], gop[g], pw[TP ^ 1][m]);
                }
            };
            issue_read(IntC<0>{});
            issue_read(IntC<1>{});
            // Matrix instruction tickets: NQB go to phase 0 (one per query block), the rest are
            // spread over the 10 vector sites of each query block in phase 1.
            constexpr int kPerQb = kGroups - 1;
            auto tickets = [&](auto loc, auto hic) {
                __builtin_amdgcn_sched_barrier(0);
                static_for<decltype(loc)::value, decltype(hic)::value>(ticket);
                __builtin_amdgcn_sched_barrier(0);
            };
            // ---- phase 0: has any score outgrown its column's reference maximum?  Lane-local
            // maxima only (no lane exchange, no execution-mask games: both stall the matrix pipe);
            // the answer is "no" on all but the first few tiles.
            float lmax[NQB];
            float excess = -INFINITY;
            static_for<0, NQB>([&](auto qbc) {
                constexpr int qb = decltype(qbc)::value;
                float mx = max3(s[TP][0][qb][0], s[TP][0][qb][1], s[TP][0][qb][2]);
                mx = max3(mx, s[TP][0][qb][3], s[TP][1][qb][0]);
                mx = max3(mx, s[TP][1][qb][1], s[TP][1][qb][2]);
                mx = max2(mx, s[TP][1][qb][3]);
                lmax[qb] = mx;
                excess = max2(excess, (mx - m_ref[qb]) * a.c);
                tickets(IntC<qb>{}, IntC<qb + 1>{});
            });
            bool moved = false;
            if (__builtin_amdgcn_ballot_w64(excess > kLazy) != 0) {
                moved = true;
#pragma unroll
                for (int qb = 0; qb < NQB; ++qb) {
                    const float mx = xor_max_fast(lmax[qb]);
                    const bool move = (mx - m_ref[qb]) * a.c > kLazy;
                    alpha[qb] = fast_exp2(move ? (m_ref[qb] - mx) * a.c : 0.0f);
                    m_ref[qb] = move ? mx : m_ref[qb];
                    l_run[qb] *= alpha[qb];
                }
            }
            // ---- phase 1: P(t) = 2^(S*c - m_ref*c + shift), row sums, fp16 ----
            static_for<0, NQB>([&](auto qbc) {
                constexpr int qb = decltype(qbc)::value;
                constexpr int base = NQB + qb * kPerQb;
                auto site = [&](auto jc) {
                    constexpr int j = decltype(jc)::value;
                    tickets(IntC<base + j * kPerQb / 10>{}, IntC<base + (j + 1) * kPerQb / 10>{});
                };
                const float nb = kPShift - m_ref[qb] * a.c;
                float sum = 0.0f;
                h8 ph;
                static_for<0, 8>([&](auto ec) {
                    constexpr int e = decltype(ec)::value;
                    float pe = fast_exp2(__builtin_fmaf(s[TP][e / 4][qb][e % 4], a.c, nb));
                    // An empty volatile block that "rewrites" the value: it keeps its order among
                    // the matrix instructions, so the exponential stays at this site instead of
                    // being sunk into the next iteration next to its first use.
                    asm volatile("" : "+v"(pe));
                    sum += pe;
                    ph[e] = (_Float16)pe;
                    site(IntC<e>{});
                });
                asm volatile("" : "+v"(ph));
                l_run[qb] += sum;
                pw[TP][qb] = ph;
                site(IntC<8>{});
                site(IntC<9>{});
            });
            fetch_v(IntC<TP ^ 1>{}, tile_of(t + 1));                   // V(t+1) -> the buffer C(t-1) read (all consumed)
            if (moved) rescale();
        };
        if (R >= 1) {
            if (R == 1) body(IntC<1>{}, IntC<0>{}, IntC<kC>{}, 1);
            else body(IntC<1>{}, IntC<1>{}, IntC<kC>{}, 1);
        }
        int t = 2;
        while (t + 1 < R) { // t even
            body(IntC<0>{}, IntC<1>{}, IntC<2 * kC>{}, t);
            body(IntC<1>{}, IntC<1>{}, IntC<2 * kC>{}, t + 1);
            t += 2;
        }
        if (t < R) { // steps t (even) and t + 1 == R
            body(IntC<0>{}, IntC<1>{}, IntC<2 * kC>{}, t);
            body(IntC<1>{}, IntC<0>{}, IntC<2 * kC>{}, t + 1);
        } else if (t == R) {
            body(IntC<0>{}, IntC<0>{}, IntC<2 * kC>{}, t);
        }
        // ---- drain: C(R) ----
        wait_copies(IntC<0>{});
        settle(); // P(R) was converted just above
        if (R & 1) stage_c(IntC<1>{});
        else stage_c(IntC<0>{});
        __builtin_amdgcn_s_waitcnt(0xC07F); // every read of the tile buffers has returned: the merge reuses them
        settle();                            // and O is out of the matrix pipe
        wave_lds_sync();
    }

    // ---- merge the four waves through LDS ----
    float* const ml = reinterpret_cast<float*>(smem + G::kMlOff);
    const unsigned obuf_addr = (unsigned)(size_t)(__attribute__((address_space(3))) unsigned char*)(smem + wave * G::kWaveB);
#pragma unroll
    for (int qb = 0; qb < NQB; ++qb) {
        const float l_tot = xor_sum(l_run[qb]);
        if (grp == 0) {
            ml[(wave * NQB * 16 + qb * 16 + col) * 2 + 0] = m_ref[qb] * a.c; // unset: hugely negative, weight 0
            ml[(wave * NQB * 16 + qb * 16 + col) * 2 + 1] = l_tot;
        }
#pragma unroll
        for (int db = 0; db < G::kDBlk; ++db)
            lds_store_acc(obuf_addr + ((qb * 16 + col) * G::kOStride + db * 16 + grp * 4) * 4, o[qb][db]);
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
        const float inv = l_all > 0.0f ? 1.0f / l_all : 0.0f;
        *reinterpret_cast<f4*>(a.out + ((size_t)tok * a.n_head + kvh * a.r + hl) * D + d4) = acc * inv;
    }
}

// Log-sum-exp merge of the decode splits.  One workgroup per (query head, 32-wide slice of
// head_dim); 8 lane-groups of 32 take the splits round-robin.  Every global load -- the
// position, the (m, l) pairs and this thread's share of the partial outputs -- is issued
// before anything is waited on, so the kernel is one memory round trip deep.  Slots of
// splits that were inactive for this position hold stale data and are masked after the load.
template <int D>
__global__ __launch_bounds__(256) void fa_decode_combine_kernel(const FaArgs a) {
    constexpr int kSlices = D / 32;
    constexpr int kGroups = 8;
    constexpr int kPer = kMaxSplits / kGroups; // partial-output loads per thread, at most
    __shared__ float sh_w[kMaxSplits];
    __shared__ float sh_red[kGroups][32];
    __shared__ float sh_wave[4][2];
    const int head = blockIdx.x / kSlices;
    const int d = (blockIdx.x % kSlices) * 32 + (threadIdx.x & 31);
    const int sg = threadIdx.x >> 5;
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int n_splits = a.n_splits;

    // loads first
    const int s_mine = threadIdx.x; // kMaxSplits == 256 == blockDim.x
    float m_s = -INFINITY, l_s = 0.0f;
    if (s_mine < n_splits) {
        const float2 ml = *reinterpret_cast<const float2*>(a.part_ml + ((size_t)s_mine * a.n_head + head) * 2);
        m_s = ml.x;
        l_s = ml.y;
    }
    float x[kPer];
    const float* po = a.part_o + (size_t)head * D + d;
    const size_t stride = (size_t)a.n_head * D;
#pragma unroll
    for (int j = 0; j < kPer; ++j) {
        const int s = sg + j * kGroups;
        x[j] = s < n_splits ? po[s * stride] : 0.0f;
    }
    int p = *a.d_pos;
    p = p < 0 ? 0 : p;
    const int npos = (p > a.n_ctx - 1 ? a.n_ctx - 1 : p) + 1;
    const int n_tiles = (npos + kTile - 1) / kTile;
    const int by_tiles = (n_tiles + kDecodeWaves - 1) / kDecodeWaves;
    const int n_active = by_tiles < n_splits ? by_tiles : n_splits;

    // weights w_s = 2^(m_s - max m) and the total row sum
    if (s_mine >= n_active) {
        m_s = -INFINITY;
        l_s = 0.0f;
    }
    float m_all = m_s;
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) m_all = fmaxf(m_all, __shfl_xor(m_all, off));
    if (lane == 0) sh_wave[wave][0] = m_all;
    __syncthreads();
    m_all = fmaxf(fmaxf(sh_wave[0][0], sh_wave[1][0]), fmaxf(sh_wave[2][0], sh_wave[3][0]));
    const float w = fast_exp2(m_s - m_all); // every active split has seen a visible row, so m_all is finite
    sh_w[s_mine] = w;                       // 0 for inactive slots
    float l_all = w * l_s;
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) l_all += __shfl_xor(l_all, off);
    if (lane == 0) sh_wave[wave][1] = l_all;
    __syncthreads();
    l_all = (sh_wave[0][1] + sh_wave[1][1]) + (sh_wave[2][1] + sh_wave[3][1]);

    float acc = 0.0f;
#pragma unroll
    for (int j = 0; j < kPer; ++j) {
        const int s = sg + j * kGroups;
        if (s < n_active) acc = __builtin_fmaf(x[j], sh_w[s], acc);
    }
    sh_red[sg][threadIdx.x & 31] = acc;
    __syncthreads();
    if (sg == 0) {
        float tot = 0.0f;
#pragma unroll
        for (int g = 0; g < kGroups; ++g) tot += sh_red[g][threadIdx.x];
        a.out[(size_t)head * D + d] = l_all > 0.0f ? tot / l_all : 0.0f;
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

// The kernels take max over raw scores and scale afterwards, which needs a positive
// multiplier: the sign of `scale` moves into Q and a zero scale becomes a vanishing one.
inline void set_scale(FaArgs& a, float scale) {
    const float c = scale * kLog2e;
    a.qsign = c < 0.0f ? -1.0f : 1.0f;
    a.c = c < 0.0f ? -c : c;
    if (!(a.c >= 1e-30f)) a.c = 1e-30f;
}

template <int D, int NQB, int TQ, bool PRECISE, bool DECODE, bool KDIRECT>
int launch_fwd(const FaArgs& a, int grid) {
    constexpr int kWaves = DECODE ? kDecodeWaves : kPrefillWaves;
    using G = Geom<D, NQB, kWaves, KDIRECT>;
    hipLaunchKernelGGL((fa_fwd_kernel<D, NQB, TQ, PRECISE, DECODE, KDIRECT>), dim3(grid), dim3(kWaves * 64), G::kLdsB,
                       g_state.stream, a);
    return hip_code(hipGetLastError());
}

// The kernels use more than 64 KB of dynamic LDS; the opt-in is set once per kernel at
// init so that no launch path touches function attributes (decode runs under capture).
template <int D, int NQB, int TQ>
int launch_prefill_kernel(const FaArgs& a, int grid) {
    constexpr int lds = PGeom<D, NQB>::kLdsB;
    hipLaunchKernelGGL((fa_prefill_kernel<D, NQB, TQ>), dim3(grid), dim3(kPrefillWaves * 64), lds, g_state.stream, a);
    return hip_code(hipGetLastError());
}

// The kernels use more than 64 KB of dynamic LDS; the opt-in is set once per kernel at
// init so that no launch path touches function attributes (decode runs under capture).
template <int D, int NQB, int TQ>
hipError_t allow_lds_prefill() {
    return hipFuncSetAttribute(reinterpret_cast<const void*>(fa_prefill_kernel<D, NQB, TQ>),
                               hipFuncAttributeMaxDynamicSharedMemorySize, PGeom<D, NQB>::kLdsB);
}

template <int D>
hipError_t allow_lds_all() {
    hipError_t e;
    if ((e = allow_lds_prefill<D, 1, 16>()) != hipSuccess) return e;
    if ((e = allow_lds_prefill<D, 2, 16>()) != hipSuccess) return e;
    if ((e = allow_lds_prefill<D, 3, 16>()) != hipSuccess) return e;
    if ((e = allow_lds_prefill<D, 4, 16>()) != hipSuccess) return e;
    if ((e = allow_lds_prefill<D, 3, 8>()) != hipSuccess) return e;
    if ((e = allow_lds_prefill<D, 4, 8>()) != hipSuccess) return e;
    return hipFuncSetAttribute(
        reinterpret_cast<const void*>(fa_fwd_kernel<D, 1, 1, true, true, kDecodeKDirect>),
        hipFuncAttributeMaxDynamicSharedMemorySize, Geom<D, 1, kDecodeWaves, kDecodeKDirect>::kLdsB);
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
        case 116: return launch_prefill_kernel<D, 1, 16>(a, grid);
        case 216: return launch_prefill_kernel<D, 2, 16>(a, grid);
        case 316: return launch_prefill_kernel<D, 3, 16>(a, grid);
        case 416: return launch_prefill_kernel<D, 4, 16>(a, grid);
        case 308: return launch_prefill_kernel<D, 3, 8>(a, grid);
        default:  return launch_prefill_kernel<D, 4, 8>(a, grid);
    }
}

int decode_splits(int n_head, int n_kv, int head_dim, int n_ctx) {
    const int r = n_head / n_kv;
    const int n_hgroups = (r + 15) / 16;
    const int cus = g_state.cu_count > 0 ? g_state.cu_count : 256;
    int s = cus / (n_kv * n_hgroups); // one 8-wave workgroup per CU
    const int by_ctx = (n_ctx + kDecodeWaves * kTile - 1) / (kDecodeWaves * kTile);
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
    int rc = launch_fwd<D, 1, 1, true, true, kDecodeKDirect>(a, grid);
    if (rc != ORIN_FA_OK || a.n_splits == 1) return rc;
    hipLaunchKernelGGL(fa_decode_combine_kernel<D>, dim3(a.n_head * (D / 32)), dim3(256), 0, g_state.stream, a);
    return hip_code(hipGetLastError());
}

int check_common(const void* q, const void* kc, const void* vc, const void* out,
                 int n_head, int n_kv, int head_dim, int n_ctx) {
    if (!g_state.ready) return ORIN_FA_E_NOT_INIT;
    if (!q || !kc || !vc || !out) return ORIN_FA_E_INVALID;
    if (n_head <= 0 || n_kv <= 0 || n_ctx <= 0 || n_head % n_kv != 0) return ORIN_FA_E_INVALID;
    if (head_dim != 64 && head_dim != 128) return ORIN_FA_E_HEAD_DIM;
    if ((long long)n_ctx * head_dim * 2 >= (1ll << 31)) return ORIN_FA_E_INVALID; // 32-bit byte offsets per KV head
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
    set_scale(a, scale);
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
    set_scale(a, scale);
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
