// Single-token GQA attention over the fp16 KV cache for gfx950 (MI355X): a split-KV kernel
// spread over every CU plus a log-sum-exp combine kernel.
//
// Replaces the reference's flash_attention_decode_mma_k and its launcher (reference:
// src/kernels.cu:1105-1345, 1983-2000), which runs one block per KV head.
//
//   * The visible cache rows [0, *d_pos] of one KV head are cut into 32-row tiles.  Workgroup
//     (KV head, split s) is 8 wave64s; wave w takes tile s*8 + w and then every
//     (8 * n_splits)-th tile after it (runs shorter than 8 at a short position in a long cache,
//     see the kernel), so at 32k context each wave streams one or two tiles and
//     every byte of K and V is fetched exactly once, by 128-bit loads with the non-temporal hint.
//   * K rows go straight from memory into MFMA A-operand order (lane (col, grp) takes row col,
//     bytes (kk*4 + grp)*16): the score product needs no LDS round trip.  V rows are loaded
//     coalesced, parked in the wave's LDS slice and read back transposed (ds_read_b64_tr_b16).
//   * All query heads of the KV head's group (up to 16 per workgroup) are the 16 columns of
//     S^T = K Q^T and O^T = V^T P on v_mfma_f32_16x16x32_f16, so the group shares one pass
//     over K and V.  The matrix pipe is idle most of the time here, so Q and P are carried as
//     fp16 hi + lo pairs and the result is accurate to fp32 rounding.
//   * The position is read on the device; the launch shape depends only on by-value arguments,
//     so the launch can be captured in a graph and replayed after the position changes.  The
//     position and the query heads are requested together, first thing; a split that the
//     position leaves without a tile exits without having touched the cache (at a short
//     position in a long cache that is nearly all of them).  Tiles are fetched whole: rows at
//     or past the position are masked (K) or zeroed on their way into LDS (V).
//   * Partials (reference maximum, row sum, O) of the 8 waves are merged through LDS and
//     written per split; the combine kernel merges the splits that were active.
#include "fa_common.hpp"

// Stage marks: wall-clock stamps in the timeline build, nothing otherwise (fa_common.hpp).
#ifdef ORIN_FA_STAMPS
namespace orin_fa {
__device__ long long g_decode_stamps[kStampWgs * kDecodeWaves * kStampSlots];
}
#define FA_STAMP(i) ORIN_FA_STAMP_STORE(orin_fa::g_decode_stamps, orin_fa::kDecodeWaves, i)
#else
#define FA_STAMP(i)
#endif

// Cut-off builds (-DORIN_FA_DECODE_PROBE=flags, liborin_fa_probe_<flags>.so; measurement aids whose RESULTS ARE
// WRONG by design): the split kernel with parts taken out, so that bench.py's cut-off workload can say
// what each part costs.  1: no combine launch.  2: the kernel leaves once its first tile has arrived
// (no products, no merge, no partial).  4: the position is n_ctx - 1, not read from memory.
// 8: no query loads.  16: K fetched whole lines at a time like V (its contents then in the wrong
// lanes).  0 in the library proper, where none of this exists.
#ifndef ORIN_FA_DECODE_PROBE
#define ORIN_FA_DECODE_PROBE 0
#endif

namespace orin_fa {
namespace {
constexpr int kProbe = ORIN_FA_DECODE_PROBE;
constexpr bool kProbeNoCombine = (kProbe & 1) != 0, kProbeCutOff = (kProbe & 2) != 0, kProbeConstPos = (kProbe & 4) != 0,
               kProbeNoQuery = (kProbe & 8) != 0, kProbeKWholeLines = (kProbe & 16) != 0;

template <int D>
struct DGeom {
    static constexpr int kSteps = D / 32;                      // MFMA k-steps over head_dim
    static constexpr int kDBlk = D / 16;                       // 16-wide output blocks over head_dim
    static constexpr int kRowBV = D * 2 + 32;                  // bytes per V row in LDS (32 B pad spreads the transposing reads)
    static constexpr int kChunksPerRow = D / 8;                // 16-byte chunks per KV row
    static constexpr int kLoads = kTile * kChunksPerRow / 64;  // 16-byte V loads per lane per tile
    static constexpr int kTileBV = kTile * kRowBV;             // one V tile in LDS
    static constexpr int kOStride = D + 4;                     // floats per column in the merge buffer
    static constexpr int kMergeB = 16 * kOStride * 4;
    static constexpr int kWaveB = (kTileBV > kMergeB) ? kTileBV : kMergeB;
    static constexpr int kMlOff = kDecodeWaves * kWaveB;       // (m, l) per wave per column follow the wave slices
    static constexpr int kQOff = kMlOff + kDecodeWaves * 16 * 2 * 4; // the group's query heads, fp32 [16][kQStride]
    static constexpr int kQStride = D + 4;                     // floats per head (4 of padding: the operand reads of 16 heads miss each other's banks)
    static constexpr int kLdsB = kQOff + 16 * kQStride * 4;
};

// MODE 1 (store): the current token's K and V rows arrive as fp32 beside the cache (FaArgs::k_new,
// v_new).  The wave whose tile holds row *d_pos takes that row from them -- rounded to fp16 exactly
// as the store kernel rounds -- instead of from the cache, and writes it to the cache on the way:
// the store kernel's launch is saved and the result is the same bit for bit.
// MODE 2 (rotate + store): q and k_new arrive before the rotary embedding, and every workgroup
// rotates them itself (the inputs stay as they are): the first n_rot/2 lanes of every wave put
// the angles' cosines and sines (computed, or read from the caller's table) into the wave's own
// LDS table while the first tile is on its way, and the pairs a lane rotates are ones it holds
// anyway -- "normal" pairs are neighbours, and for "neox" with
// n_rot = head_dim element e pairs with e + head_dim/2, the same lane's k-step two (one, at
// head_dim 64) further on.  Same arithmetic as the rotary kernel, so again bit for bit what the
// separate launches give, four launches in the place of seven.
template <int D, int MODE>
__global__ __launch_bounds__(kDecodeWaves * 64) void fa_decode_split_kernel(
    // What the first loads need comes first, as scalars: the leading kernel arguments are handed
    // to a wave in registers when it starts (kernel-argument preload), so the position and the
    // query can be requested at once instead of behind a trip to memory for their addresses.
    // (no __restrict__ on these: loads the compiler knows to be invariant are free to sink past
    // the statements below that hold them in place)
    // Plain decode needs nothing but these 14 words: no trip to the launch's argument block at
    // all, which is slower than the trip for the position (the caches hold that).  So: the grid
    // is (KV head, head group, split) and says what n_kv and n_hgroups would; n_splits and r share
    // a word (splits_r = n_splits | r << 16); the scale carries the sign that goes into Q
    // (c_signed = |scale| log2(e) with the sign of scale; c2 below is its magnitude); dst is where this kernel writes: the
    // partial outputs (followed by the (m, l) pairs) when there are splits, else `out` itself.
    const int* d_pos, const float* q, const uint16_t* kc, const uint16_t* vc,
    const int n_ctx, const unsigned splits_r, const float c_signed, float* dst, const int n_head,
    const FaArgs a) { // (a: what the store and rotate variants need besides)
    using G = DGeom<D>;
    constexpr int kWaves = kDecodeWaves;
    constexpr int kThreads = kWaves * 64;
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    FA_STAMP(0);

    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int col = lane & 15; // MFMA column (query head of the group) / row (KV row or head_dim index) of the lane
    const int grp = lane >> 4; // lane-group: 8-wide k slice of an operand, 4-row slice of an accumulator

    const int n_splits = splits_r & 0xffffu, r = splits_r >> 16;
    const float c2 = __builtin_fabsf(c_signed), qsign = c_signed < 0.0f ? -1.0f : 1.0f;
    // Workgroup -> (KV head, head group, split); the KV head varies fastest in dispatch order.
    const int kvh = blockIdx.x, hg = blockIdx.y, id = blockIdx.z;
    float* const part_o = dst;
    float* const part_ml = dst + (size_t)n_splits * n_head * D; // [n_head][split][2]

    unsigned char* const vs = smem + wave * G::kWaveB;
    const __amdgpu_buffer_rsrc_t krs = make_rsrc(kc + (size_t)kvh * n_ctx * D, (unsigned)n_ctx * D * 2);
    const __amdgpu_buffer_rsrc_t vrs = make_rsrc(vc + (size_t)kvh * n_ctx * D, (unsigned)n_ctx * D * 2);

    u32x4 kreg[2 * G::kSteps], vreg[G::kLoads];
    auto fetch_k = [&](int tile) {
        const int soff = tile * kTile * D * 2;
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int kk = 0; kk < G::kSteps; ++kk)
                kreg[t * G::kSteps + kk] = buf_load16<true>(krs, kProbeKWholeLines ? soff + ((t * G::kSteps + kk) * 64 + lane) * 16
                                                                                    : soff + (t * 16 + col) * D * 2 + (kk * 4 + grp) * 16);
    };
    auto fetch_v = [&](int tile) {
        const int soff = tile * kTile * D * 2;
#pragma unroll
        for (int i = 0; i < G::kLoads; ++i) vreg[i] = buf_load16<true>(vrs, soff + (i * 64 + lane) * 16);
    };
    // ---- query heads: requested before the first tile, so that they arrive before it (a wave's
    // loads complete in order) and the score product can start while V is still on its way ----
    const int pos = kProbeConstPos ? n_ctx - 1 - (d_pos == nullptr) : *d_pos; // (read here, ahead of the statement below that may write memory: a scalar load)
    const int hl = hg * 16 + col;
    const bool valid = hl < r;
    // Columns past the group's heads are padding: their loads carry an offset past the descriptor's
    // end, which the hardware answers with zeros without going to memory.  (Every wave of every
    // workgroup reads its group's heads: fetched for all 16 columns that was as many bytes through
    // the L2 as the K rows.)
    // The workgroup fetches its group's heads once: wave w asks for one 16-byte piece per lane --
    // piece (w & 1) of k-step (w >> 1) -- and the pieces meet in LDS further down.  (Every wave
    // fetching all of them itself was seven more load instructions a wave whose lanes each count
    // as a look-up of their own in the vector cache, a quarter again of the kernel's look-ups, all
    // of them in the queue ahead of the tile requests: 0.4 us per launch.)
    const __amdgpu_buffer_rsrc_t qrs = make_rsrc(q, 0x7ffffff0u);
    const int q_off = valid ? ((kvh * r + hl) * D + grp * 8) * 4 : 0x7ffffff8;
    const float qmul = valid ? qsign : 0.0f;
    static_assert(kWaves % (2 * G::kSteps) == 0, "a piece per wave (the same piece twice at head_dim 64)");
    const int q_piece = __builtin_amdgcn_readfirstlane(wave) & (2 * G::kSteps - 1);
    const float4 q_share = kProbeNoQuery ? float4{1.f, 2.f, (float)q_off, (float)lane}
                                         : __builtin_bit_cast(float4, __builtin_amdgcn_raw_buffer_load_b128(qrs, q_off, (q_piece >> 1) * 128 + (q_piece & 1) * 16, 0));
    constexpr bool STORE = MODE != 0, ROPE = MODE == 2;
    // (rotate + store) lane i < n_rot/2 of every wave fetches what pair i's angle needs: its
    // cosine and sine when the caller supplies them, else its frequency factor if there is one.
    // Both loads are made by every lane, from an address that can be read either way (the query,
    // when the array is absent): a load under a branch makes the compiler wait for every load
    // issued so far where the branch ends.
    float2 cs_given = float2{1.0f, 0.0f};
    float ff_given = 1.0f;
    if constexpr (ROPE) {
        const int pi = min(lane, a.n_rot / 2 - 1);
        const float* anp = a.rope_angles ? a.rope_angles + 2 * pi : q;
        const float* ffp = a.freq_factors ? a.freq_factors + pi : q;
        cs_given = *reinterpret_cast<const float2*>(anp);
        ff_given = *ffp;
    }
    // (store, rotate + store) The new row, in as few loads as will do, by every wave: only the one whose tiles
    // include the row's uses it (at its last tile), but which wave that is depends on the position, which is
    // still on its way, and a load issued later, while the CU's tiles stream in, holds its wave up for a few
    // hundred cycles each (three of them: 0.5 us between the query's arrival and its conversion).  Here they
    // are small loads ahead of the flood, hits in the cache for all but the first wave to ask.  K: elements
    // 4*lane .. 4*lane+3 (the lanes hand each other the pieces they hold of a K row through LDS then); V: piece
    // lane % (D/8), which is what the lane holds of a V row.
    float4 k_raw = float4{0.f, 0.f, 0.f, 0.f}, v_raw[2] = {k_raw, k_raw};
    if constexpr (STORE) {
        const float* kp4 = a.k_new + (size_t)kvh * D + (lane % (D / 4)) * 4;
        const float* vp8 = a.v_new + (size_t)kvh * D + (lane % G::kChunksPerRow) * 8;
        k_raw = *reinterpret_cast<const float4*>(kp4);
        v_raw[0] = *reinterpret_cast<const float4*>(vp8);
        v_raw[1] = *reinterpret_cast<const float4*>(vp8 + 4);
    }
    __builtin_amdgcn_sched_barrier(0); // the small loads first: they return first, and nothing that needs them waits for a tile

    // The query loads above are used only behind the early return below, and left alone the
    // compiler moves them there, behind the wait for the position.  A statement that may write
    // memory keeps them on this side of the branch, where they overlap the load of the position.
    // The first tile is NOT requested here: a workgroup that turns out to be inactive would pull
    // 128 KB of cache rows for nothing -- at a short position in a long cache, all of them but a
    // few, tens of megabytes per launch that the active ones then queue behind.
    asm volatile("" ::: "memory");
    // (store and rotate variants) The arguments that did not arrive in registers are fetched
    // here, in the trip to memory that brings the position: left alone, the compiler fetches
    // each where it is first used, behind the first tile's arrival.  (Fetched behind the tile
    // requests instead, they queue behind the chip's 33 MB of tile traffic: 0.5 us per layer.)
    if constexpr (MODE != 0) {
        const void *p0 = a.k_new, *p1 = a.v_new;
        asm volatile("" ::"s"(p0), "s"(p1), "s"(a.n_rot), "s"(a.neox), "s"(pos));
    }
    __builtin_amdgcn_sched_barrier(0);

    int p = pos < 0 ? 0 : pos;
    const int npos = (p > n_ctx - 1 ? n_ctx - 1 : p) + 1; // rows [0, npos) are visible
    const bool store = STORE && pos >= 0 && pos < n_ctx;   // (a position outside the cache stores nothing, as the store kernel)
    const int n_tiles = (npos + kTile - 1) / kTile;
    // Tiles go to the splits in runs of `wu` consecutive tiles, one per wave: eight when there are
    // enough tiles to keep every wave of every split busy (runs of 128 KB of K and of V), fewer
    // at a short position in a long cache, whose few tiles then spread over as many workgroups
    // (CUs, each with its own 64 B/clk into the vector cache) as there are instead of filling a
    // few workgroups' eight waves.  (Interleaving single tiles among the splits at every length
    // cost 8 % at full length on Qwen2.5-7B: neighbouring 8 KB pieces then alternate between XCDs.)
    int wu = (n_tiles + n_splits - 1) / n_splits;
    wu = wu > kWaves ? kWaves : wu;
    const int tile_first = wave < wu ? id * wu + wave : n_tiles; // (n_tiles: none)
    const int tile_step = wu * n_splits;
    int tile = tile_first;
    float* const qs = reinterpret_cast<float*>(smem + G::kQOff);
    __shared__ __attribute__((aligned(16))) float sh_cs_all[ROPE ? kWaves : 1][D / 2][2];
    __shared__ __attribute__((aligned(16))) float sh_krow_all[STORE ? kWaves : 1][D];
    float (*const sh_cs)[2] = sh_cs_all[ROPE ? wave : 0];
    const bool rot_early = ROPE && !a.neox && a.rope_angles != nullptr; // (the query is rotated piece by piece before it is parked)
    if (id * wu < n_tiles) {
        // The query pieces meet in LDS: each wave parks the piece it fetched, then a barrier that
        // waits for LDS only.  Ahead of the tile requests, where the eight waves are still in
        // step (the position and the pieces arrive together); behind them the waves are microseconds
        // apart -- the load unit takes a CU's 128 KB of requests as fast as memory answers them --
        // and a barrier there holds every wave's products until the last has all its requests out.
        float4 q_park = q_share;
        if constexpr (ROPE) {
            // "Normal" pairs are neighbours, so the piece a wave fetched holds two whole pairs: with the caller's
            // table of angles at hand the wave rotates just those before it parks the piece, and nobody has to
            // rotate the whole query behind the barrier (eight waves each used to: sixteen table reads and as
            // many rotations a lane between the query's arrival and its conversion; 0.4 us of a Llama-3-8B
            // launch pair).  Without a table the angles are a power, a sine and a cosine away, which must not
            // sit ahead of the tile requests.  ("neox" pairs sit half a head apart, in another wave's piece:
            // fetching that piece as well and rotating early was built and gained nothing.)
            if (rot_early) {
                if (lane < a.n_rot / 2) {
                    sh_cs[lane][0] = cs_given.x;
                    sh_cs[lane][1] = cs_given.y;
                }
                __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
                __builtin_amdgcn_wave_barrier();
                __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
                const int e0 = (q_piece >> 1) * 32 + grp * 8 + (q_piece & 1) * 4, last = max(a.n_rot / 2 - 1, 0);
                const float2 c0 = *reinterpret_cast<const float2*>(sh_cs[min(e0 / 2, last)]);
                const float2 c1 = *reinterpret_cast<const float2*>(sh_cs[min(e0 / 2 + 1, last)]);
                float x0 = q_park.x, x1 = q_park.y, y0 = q_park.z, y1 = q_park.w;
                rope_rotate(x0, x1, c0.x, c0.y);
                rope_rotate(y0, y1, c1.x, c1.y);
                q_park.x = e0 < a.n_rot ? x0 : q_park.x;
                q_park.y = e0 < a.n_rot ? x1 : q_park.y;
                q_park.z = e0 + 2 < a.n_rot ? y0 : q_park.z;
                q_park.w = e0 + 2 < a.n_rot ? y1 : q_park.w;
            }
        }
        *reinterpret_cast<float4*>(qs + col * G::kQStride + (q_piece >> 1) * 32 + grp * 8 + (q_piece & 1) * 4) = q_park;
        asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
        fetch_k(tile);
        fetch_v(tile);
        asm volatile("" ::: "memory"); // (as above: ahead of the conversions that follow, not behind them)
        __builtin_amdgcn_sched_barrier(0);
    }
    if (id * wu >= n_tiles) {
        // Inactive split: it leaves "no row seen" for its heads, so that the combine kernel can tell
        // without reading the position itself (one more trip to memory on its short critical path);
        // the partial outputs are left as they are and get weight zero.
        if (threadIdx.x < 16 && hg * 16 + (int)threadIdx.x < r) {
            const size_t mi = (size_t)(kvh * r + hg * 16 + threadIdx.x) * n_splits + id; // [head][split]
            part_ml[mi * 2 + 0] = -INFINITY;
            part_ml[mi * 2 + 1] = 0.0f;
        }
        return;
    }

    FA_STAMP(1);
    if constexpr (kProbeCutOff) { // (cut-off build: wait for the tile, keep every load alive, leave)
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        unsigned acc = __float_as_uint(q_share.x) ^ __float_as_uint(q_share.w);
#pragma unroll
        for (int i = 0; i < 2 * G::kSteps; ++i) acc ^= kreg[i].x ^ kreg[i].y ^ kreg[i].z ^ kreg[i].w;
#pragma unroll
        for (int i = 0; i < G::kLoads; ++i) acc ^= vreg[i].x ^ vreg[i].y ^ vreg[i].z ^ vreg[i].w;
        if (acc == 0x9E3779B9u) part_ml[0] = 1.0f;
        if (acc != 0x9E3779BAu) return;
    }
    // (the query pieces met ahead of the tile requests; the operands are picked up while the first tile is on its way)
    float qf[G::kSteps][8]; // this lane's 8 elements of every k-step: head_dim indices kk*32 + grp*8 + 0..7
#pragma unroll
    for (int kk = 0; kk < G::kSteps; ++kk) {
        const float4 x0 = *reinterpret_cast<const float4*>(qs + col * G::kQStride + kk * 32 + grp * 8);
        const float4 x1 = *reinterpret_cast<const float4*>(qs + col * G::kQStride + kk * 32 + grp * 8 + 4);
        qf[kk][0] = x0.x; qf[kk][1] = x0.y; qf[kk][2] = x0.z; qf[kk][3] = x0.w;
        qf[kk][4] = x1.x; qf[kk][5] = x1.y; qf[kk][6] = x1.z; qf[kk][7] = x1.w;
    }
    // (rotate + store) the rotation of this lane's 8 elements of every k-step, by the wave's table
    // x0, x1: this lane's elements of k-steps kk and kk + kSteps/2 (head_dim indices kk*32 + grp*8 + e
    // and the same + head_dim/2)
    auto rotate2 = [&](float (&x0)[8], float (&x1)[8], int kk) {
        if (a.neox) { // n_rot == D (checked by the host): element e pairs with e + D/2
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const int i = kk * 32 + grp * 8 + e;
                rope_rotate(x0[e], x1[e], sh_cs[i][0], sh_cs[i][1]);
            }
        } else {      // elements 2i and 2i + 1, below n_rot
            // No branch per pair: el0 differs from lane to lane, and a branch around each pair's table
            // read makes the wave wait out sixteen LDS round trips one after the other (1.7 us of a
            // Llama-3-8B launch).  Every lane reads an entry (its own, or the table's last), all reads
            // go out together, and a pair past n_rot keeps its values by a select.
            const int last = max(a.n_rot / 2 - 1, 0); // (n_rot = 0: nothing is rotated, entry 0 is read and not used)
            float2 cs0[4], cs1[4];
#pragma unroll
            for (int e = 0; e < 8; e += 2) {
                const int el0 = kk * 32 + grp * 8 + e, el1 = el0 + D / 2;
                cs0[e / 2] = *reinterpret_cast<const float2*>(sh_cs[min(el0 / 2, last)]);
                cs1[e / 2] = *reinterpret_cast<const float2*>(sh_cs[min(el1 / 2, last)]);
            }
#pragma unroll
            for (int e = 0; e < 8; e += 2) {
                const int el0 = kk * 32 + grp * 8 + e, el1 = el0 + D / 2;
                float a0 = x0[e], a1 = x0[e + 1], b0 = x1[e], b1 = x1[e + 1];
                rope_rotate(a0, a1, cs0[e / 2].x, cs0[e / 2].y);
                rope_rotate(b0, b1, cs1[e / 2].x, cs1[e / 2].y);
                x0[e] = el0 < a.n_rot ? a0 : x0[e];
                x0[e + 1] = el0 < a.n_rot ? a1 : x0[e + 1];
                x1[e] = el1 < a.n_rot ? b0 : x1[e];
                x1[e + 1] = el1 < a.n_rot ? b1 : x1[e + 1];
            }
        }
    };
    if constexpr (ROPE) {
        // (cos, sin) of pair i at the raw position, as the rotary kernel forms them
        // A table per wave (head_dim <= 128: a wave's 64 lanes cover the pairs), so that no wave
        // waits here for the others: the waves of a workgroup get their loads out at very
        // different times when the whole chip is requesting its first tiles.  Write and reads
        // are the same wave's, and a wave's LDS operations complete in order.
        static_assert(D / 2 <= 64, "one lane per pair");
        const int half = a.n_rot / 2;
        if (!rot_early && lane < half) {
            if (!a.rope_angles) {
                float freq = rope_freq_base(lane, a.n_rot, a.theta);
                if (a.freq_factors) freq /= ff_given;
                const float ang = (float)pos * freq;
                cs_given.x = cosf(ang);
                cs_given.y = sinf(ang);
            }
            sh_cs[lane][0] = cs_given.x;
            sh_cs[lane][1] = cs_given.y;
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        if (!rot_early) {
#pragma unroll
            for (int kk = 0; kk < G::kSteps / 2; ++kk) rotate2(qf[kk], qf[kk + G::kSteps / 2], kk);
        }
    }
    // ---- query heads -> B operands, fp16 hi + lo ----
    h8 qhi[G::kSteps], qlo[G::kSteps];
#pragma unroll
    for (int kk = 0; kk < G::kSteps; ++kk) {
        const float* x = qf[kk];
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const float xe = x[e] * qmul;
            qhi[kk][e] = (_Float16)xe;
            qlo[kk][e] = (_Float16)(xe - (float)qhi[kk][e]);
        }
    }

    __builtin_amdgcn_sched_barrier(0);
    FA_STAMP(2);
    // m_ref: reference maximum of the raw scores (before the scale); l_run: this lane's share of
    // the row sum; o: O^T accumulators, lane (col, grp) holds head_dim rows db*16 + grp*4 + i.
    float m_ref = -INFINITY, l_run = 0.0f;
    f4 o[G::kDBlk];
#pragma unroll
    for (int db = 0; db < G::kDBlk; ++db) o[db] = f4{0.f, 0.f, 0.f, 0.f};
    const int v_rd = (grp * 4 + (col >> 2)) * G::kRowBV + (col & 3) * 8; // + h*16 rows, + db*32 bytes

    // (store, rotate + store) The new row is made ready here, while the tiles travel, by the one wave whose tiles
    // include the row's (the last visible tile: the wave's own last): converted -- and the K row rotated -- as the
    // store kernel and the rotary kernel would, the pieces this lane is to substitute and to write kept in
    // registers.  At that tile only the substitution and the two cache writes are left.  (Made ready at the tile
    // itself, as it used to be, the LDS round trips and the rotation sat between the arrival of the launch's last
    // tile and its products: 0.7 us of a Qwen2.5-1.5B launch pair at 32k.)  The row's loads went out ahead of the
    // tile requests, so waiting for them waits for no tile.
    const int own_tile = n_tiles - 1;
    [[maybe_unused]] bool owner = false;
    [[maybe_unused]] u32x4 k_new16[G::kSteps], v_new16 = u32x4{0u, 0u, 0u, 0u};
    if constexpr (STORE) {
#pragma unroll
        for (int kk = 0; kk < G::kSteps; ++kk) k_new16[kk] = u32x4{0u, 0u, 0u, 0u};
        owner = store && tile_first <= own_tile && (own_tile - tile_first) % tile_step == 0;
        if (owner) {
            // (Nothing below may be started ahead of this branch: the compiler would otherwise
            // convert the new row in every wave.)
            auto here = [](float x) { // a copy the compiler cannot make anywhere else
                float y;
                asm volatile("v_mov_b32 %0, %1" : "=v"(y) : "v"(x));
                return y;
            };
            const float4 k_own = float4{here(k_raw.x), here(k_raw.y), here(k_raw.z), here(k_raw.w)};
            const float4 v_own[2] = {float4{here(v_raw[0].x), here(v_raw[0].y), here(v_raw[0].z), here(v_raw[0].w)},
                                     float4{here(v_raw[1].x), here(v_raw[1].y), here(v_raw[1].z), here(v_raw[1].w)}};
            {
                // The new K row is rotated (rotate + store) and converted by the one wave
                // that needs it.  It has waited in four registers a lane; the lanes now hand
                // each other the pieces they hold of a K row through the wave's LDS row.
                float* const krow = sh_krow_all[wave];
                if (lane < D / 4) *reinterpret_cast<float4*>(krow + lane * 4) = k_own;
                __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
                __builtin_amdgcn_wave_barrier();
                __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
                for (int kk = 0; kk < G::kSteps / 2; ++kk) { // two k-steps at a time: the pair of a "neox" rotation
                    float x[2][8];
#pragma unroll
                    for (int u = 0; u < 2; ++u) {
                        const float* src = krow + (kk + u * (G::kSteps / 2)) * 32 + grp * 8;
                        const float4 lo = *reinterpret_cast<const float4*>(src), hi = *reinterpret_cast<const float4*>(src + 4);
                        x[u][0] = lo.x; x[u][1] = lo.y; x[u][2] = lo.z; x[u][3] = lo.w;
                        x[u][4] = hi.x; x[u][5] = hi.y; x[u][6] = hi.z; x[u][7] = hi.w;
                    }
                    if constexpr (ROPE) rotate2(x[0], x[1], kk);
#pragma unroll
                    for (int u = 0; u < 2; ++u) {
                        h8 h;
#pragma unroll
                        for (int e = 0; e < 8; ++e) h[e] = (_Float16)x[u][e];
                        k_new16[kk + u * (G::kSteps / 2)] = __builtin_bit_cast(u32x4, h);
                    }
                }
            }
            h8 vh;
            vh[0] = (_Float16)v_own[0].x; vh[1] = (_Float16)v_own[0].y; vh[2] = (_Float16)v_own[0].z; vh[3] = (_Float16)v_own[0].w;
            vh[4] = (_Float16)v_own[1].x; vh[5] = (_Float16)v_own[1].y; vh[6] = (_Float16)v_own[1].z; vh[7] = (_Float16)v_own[1].w;
            v_new16 = __builtin_bit_cast(u32x4, vh);
            // The cache gets the row now (one head group's wave writes it): whatever the tile request that is under
            // way brings back for this row is replaced from the registers above, and no other wave reads it, so the
            // order of the two does not matter, and stores issued here are long done when the kernel ends.
            if (hg == 0) {
                const int row = pos % kTile;
                const size_t row_off = ((size_t)kvh * n_ctx + pos) * D;
                if (col == row % 16) {
#pragma unroll
                    for (int kk = 0; kk < G::kSteps; ++kk)
                        *reinterpret_cast<u32x4*>(const_cast<uint16_t*>(kc) + row_off + (kk * 4 + grp) * 8) = k_new16[kk];
                }
                if (lane < G::kChunksPerRow) *reinterpret_cast<u32x4*>(const_cast<uint16_t*>(vc) + row_off + lane * 8) = v_new16;
            }
        }
    }

    for (; tile < n_tiles; tile += tile_step) {
        const bool more = tile + tile_step < n_tiles;
        if constexpr (STORE) {
            if (owner && tile == own_tile) { // the tile of the new row: into the operand registers
                const int row = pos % kTile;
                if (col == row % 16) {
#pragma unroll
                    for (int kk = 0; kk < G::kSteps; ++kk)
#pragma unroll
                        for (int t = 0; t < 2; ++t) // (constant register indices: a computed one sends the array to scratch memory)
                            if (row / 16 == t) kreg[t * G::kSteps + kk] = k_new16[kk];
                }
#pragma unroll
                for (int i = 0; i < G::kLoads; ++i)
                    if ((i * 64 + lane) / G::kChunksPerRow == row) vreg[i] = v_new16;
            }
        }
        // ---- S^T = K Q^T : rows = KV row (sub-tile t, row col), columns = query head ----
        f4 s[2], s2[2]; // the Q-lo product runs as its own accumulation chain
#pragma unroll
        for (int t = 0; t < 2; ++t) s[t] = s2[t] = f4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int kk = 0; kk < G::kSteps; ++kk)
#pragma unroll
            for (int t = 0; t < 2; ++t) {
                const h8 ka = __builtin_bit_cast(h8, kreg[t * G::kSteps + kk]);
                s[t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(ka, qhi[kk], s[t], 0, 0, 0);
                s2[t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(ka, qlo[kk], s2[t], 0, 0, 0);
            }
        s[0] += s2[0];
        s[1] += s2[1];
        if (more) fetch_k(tile + tile_step); // the operand registers are free again
        FA_STAMP(3);

        // ---- softmax weights; lane (col, grp) holds rows t*16 + grp*4 + i of its column ----
        float v[8];
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int i = 0; i < 4; ++i) v[t * 4 + i] = s[t][i];
        if (tile * kTile + kTile > npos) { // the last tile: rows past the position do not exist
#pragma unroll
            for (int t = 0; t < 2; ++t)
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    if (tile * kTile + t * 16 + grp * 4 + i >= npos) v[t * 4 + i] = -INFINITY;
        }
        float mx = fmaxf(fmaxf(v[0], v[1]), v[2]);
        mx = fmaxf(fmaxf(mx, v[3]), v[4]);
        mx = fmaxf(fmaxf(mx, v[5]), v[6]);
        mx = xor_max(fmaxf(mx, v[7]));
        // move the reference only when this tile's maximum is far above it (or it is unset)
        const bool move = (mx - m_ref) * c2 > kLazy || (m_ref == -INFINITY && mx > -INFINITY);
        if (__builtin_amdgcn_ballot_w64(move) != 0) {
            const float alpha = move ? fast_exp2((m_ref - mx) * c2) : 1.0f; // unset reference -> 0
            if (move) m_ref = mx;
            l_run *= alpha;
#pragma unroll
            for (int db = 0; db < G::kDBlk; ++db) o[db] *= alpha;
        }
        // exponent = s*c2 - m_ref*c2 + shift; a column that has seen no visible row keeps weight 0
        const float nb = (m_ref == -INFINITY) ? kPShift : kPShift - m_ref * c2;
        h8 ph, pl;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const float pe = fast_exp2(__builtin_fmaf(v[e], c2, nb));
            l_run += pe;
            ph[e] = (_Float16)pe;
            pl[e] = (_Float16)(pe - (float)ph[e]);
        }

        // ---- V: registers -> this wave's LDS slice (K was needed first and arrives first) ----
        const int rows_left = npos - tile * kTile; // rows of this tile below the position (>= 32: all)
#pragma unroll
        for (int i = 0; i < G::kLoads; ++i) {
            const int c = i * 64 + lane;
            // rows at or past the position may hold anything; their weights are zero, and 0 * NaN is not
            const u32x4 x = (c / G::kChunksPerRow) < rows_left ? vreg[i] : u32x4{0u, 0u, 0u, 0u};
            *reinterpret_cast<u32x4*>(vs + (c / G::kChunksPerRow) * G::kRowBV + (c % G::kChunksPerRow) * 16) = x;
        }
        if (more) fetch_v(tile + tile_step);
        wave_lds_sync();

        // ---- O^T += V^T P : rows = head_dim index, columns = query head, k = the tile's 32 KV rows
        //      in the order (grp, t, i) that matches the layout P already has ----
#pragma unroll
        for (int db = 0; db < G::kDBlk; ++db) {
            const h4 v0 = lds_read_tr(vs + v_rd + db * 32);
            const h4 v1 = lds_read_tr(vs + v_rd + 16 * G::kRowBV + db * 32);
            const h8 va = __builtin_shufflevector(v0, v1, 0, 1, 2, 3, 4, 5, 6, 7);
            o[db] = __builtin_amdgcn_mfma_f32_16x16x32_f16(va, ph, o[db], 0, 0, 0);
            o[db] = __builtin_amdgcn_mfma_f32_16x16x32_f16(va, pl, o[db], 0, 0, 0);
        }
        wave_lds_sync(); // the slice is overwritten at the top of the next iteration
    }

    FA_STAMP(4);
    // ---- merge the waves through LDS ----
    float* const ml = reinterpret_cast<float*>(smem + G::kMlOff);
    float* const obuf = reinterpret_cast<float*>(smem + wave * G::kWaveB);
    const float l_tot = xor_sum(l_run);
    if (grp == 0) {
        ml[(wave * 16 + col) * 2 + 0] = (m_ref == -INFINITY) ? -INFINITY : m_ref * c2; // log2 units
        ml[(wave * 16 + col) * 2 + 1] = l_tot;
    }
#pragma unroll
    for (int db = 0; db < G::kDBlk; ++db)
        *reinterpret_cast<f4*>(obuf + col * G::kOStride + db * 16 + grp * 4) = o[db];
    FA_STAMP(5);
    __syncthreads();
    FA_STAMP(6);

    for (int idx = threadIdx.x; idx < 16 * (D / 4); idx += kThreads) {
        const int c = idx / (D / 4);
        const int d4 = (idx % (D / 4)) * 4;
        const int h_local = hg * 16 + c;
        if (h_local >= r) continue;
        float mw[kWaves], lw[kWaves];
        float m_all = -INFINITY;
#pragma unroll
        for (int w = 0; w < kWaves; ++w) {
            mw[w] = ml[(w * 16 + c) * 2 + 0];
            lw[w] = ml[(w * 16 + c) * 2 + 1];
            m_all = fmaxf(m_all, mw[w]);
        }
        float l_all = 0.0f;
        f4 acc = f4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int w = 0; w < kWaves; ++w) {
            const float wgt = fast_exp2(mw[w] - m_all); // a wave that had no tile has m = -inf -> weight 0
            l_all += lw[w] * wgt;
            acc += *reinterpret_cast<const f4*>(smem + w * G::kWaveB + ((size_t)c * G::kOStride + d4) * 4) * wgt;
        }
        const int head = kvh * r + h_local;
        if (n_splits > 1) {
            const size_t pi = (size_t)id * n_head + head;
            *reinterpret_cast<f4*>(part_o + pi * D + d4) = acc;
            if (d4 == 0) {
                const size_t mi = (size_t)head * n_splits + id; // [head][split]: a head's pairs are one run of memory for the combine kernel
                part_ml[mi * 2 + 0] = m_all;
                part_ml[mi * 2 + 1] = l_all;
            }
        } else {
            const float inv = l_all > 0.0f ? 1.0f / l_all : 0.0f;
            *reinterpret_cast<f4*>(dst + (size_t)head * D + d4) = acc * inv; // (no splits: dst is the output)
        }
    }
    FA_STAMP(7);
}

// Log-sum-exp merge of the decode splits.  One workgroup of 8 waves per (query head, 64-wide
// slice of head_dim); wave w takes the partial outputs of splits w, w + 8, ...; lane = element
// of the slice.  The kernel is little more than a trip to memory, so everything is shaped to
// make that one trip and little else:
//   * a head's (m, l) pairs are one run of memory ([head][split]): every wave fetches all of them
//     with one coalesced load per 64 splits (lane = split) and finds the overall maximum and the
//     overall row sum itself, with lane-swap reductions, while its partial outputs are still on
//     their way -- so no wave waits for another's statistics, and the weights of a wave's own
//     splits are lane reads;
//   * a wave's split indices are uniform, so the address arithmetic of the partial outputs
//     stays in the scalar unit and every load is one coalesced 256 bytes (per-thread 64-bit
//     address arithmetic for every load cost more than the trip);
//   * every load is issued before anything is waited on, and nothing else is read (not even the
//     position: splits that were inactive for it have said so in their (m, l)).
// The 8 waves' weighted sums meet in LDS behind the kernel's only barrier.  Partial outputs of
// inactive splits hold stale data and are never multiplied.
// PER: splits per wave (n_splits <= 8 * PER; the launcher picks the smallest that fits).
template <int D, int PER>
__global__ __launch_bounds__(512) void fa_decode_combine_kernel(const float* __restrict__ part_o, const float* __restrict__ part_ml,
                                                                 float* __restrict__ out, const int n_splits, const int n_head) {
    constexpr int kSlices = D / 64;
    constexpr int kGroups = 8;
    constexpr int kRounds = (kGroups * PER + 63) / 64; // (m, l) pairs per lane
    static_assert(kGroups * PER <= kMaxSplits, "more slots than splits can be");
    __shared__ float sh_acc[kGroups][64];
    const int head = blockIdx.x / kSlices;
    const int lane = threadIdx.x & 63;
    const int d = (blockIdx.x % kSlices) * 64 + lane;
    const int sg = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);

    // (slots past n_splits read split 0 again and are voided below: a load under a branch
    // would make the compiler wait for the loads before it where the branch ends)
    float2 ml[kRounds];
    const float* const pm = part_ml + (size_t)head * n_splits * 2;
#pragma unroll
    for (int rd = 0; rd < kRounds; ++rd) {
        const int s = lane + 64 * rd;
        ml[rd] = *reinterpret_cast<const float2*>(pm + (s < n_splits ? s : 0) * 2);
    }
    float x[PER];
    const int stride = n_head * D; // (a split's partial outputs; the whole array is below 2^31 bytes)
    const float* const po = part_o + head * D + d;
#pragma unroll
    for (int j = 0; j < PER; ++j) {
        const int s = sg + j * kGroups;
        x[j] = po[(s < n_splits ? s : 0) * stride];
    }
    // ---- the head's statistics, in every wave, while the partial outputs travel ----
    float m_all = -INFINITY;
#pragma unroll
    for (int rd = 0; rd < kRounds; ++rd) {
        if (lane + 64 * rd >= n_splits) ml[rd] = float2{-INFINITY, 0.0f};
        m_all = fmaxf(m_all, ml[rd].x);
    }
    m_all = wave_max(m_all);
    float w[kRounds], l_all = 0.0f;
#pragma unroll
    for (int rd = 0; rd < kRounds; ++rd) {
        w[rd] = ml[rd].x > -INFINITY ? fast_exp2(ml[rd].x - m_all) : 0.0f; // (no split active at all: every weight 0)
        l_all = __builtin_fmaf(ml[rd].y, w[rd], l_all);
    }
    l_all = wave_sum(l_all);
    // ---- this wave's splits: split sg + 8j sits in lane (8j mod 64) + sg of round 8j / 64 ----
    float acc = 0.0f;
#pragma unroll
    for (int j = 0; j < PER; ++j) {
        const float wj = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(w[(j * kGroups) / 64]), ((j * kGroups) % 64) + sg));
        if (wj > 0.0f) acc = __builtin_fmaf(x[j], wj, acc); // (what a weightless split left behind may be anything)
    }
    sh_acc[sg][lane] = acc;
    __syncthreads();
    if (sg == 0) {
        float tot = 0.0f;
#pragma unroll
        for (int g = 0; g < kGroups; ++g) tot += sh_acc[g][lane];
        out[head * D + d] = l_all > 0.0f ? tot / l_all : 0.0f;
    }
}

template <int D>
hipError_t launch(const FaArgs& a, hipStream_t stream) {
    if (a.n_splits > 0xffff || a.r > 0xffff || a.n_hgroups > 0xffff) return hipErrorInvalidValue;
    constexpr int lds = DGeom<D>::kLdsB;
    const dim3 g(a.n_kv, a.n_hgroups, a.n_splits), b(kDecodeWaves * 64);
    const unsigned splits_r = (unsigned)a.n_splits | (unsigned)a.r << 16;
    float* const dst = a.n_splits > 1 ? a.part_o : a.out;
#define ORIN_FA_SPLIT_ARGS a.d_pos, a.q, a.kc, a.vc, a.n_ctx, splits_r, a.c * a.qsign, dst, a.n_head, a
    if (a.k_new && a.n_rot > 0) hipLaunchKernelGGL((fa_decode_split_kernel<D, 2>), g, b, lds, stream, ORIN_FA_SPLIT_ARGS);
    else if (a.k_new) hipLaunchKernelGGL((fa_decode_split_kernel<D, 1>), g, b, lds, stream, ORIN_FA_SPLIT_ARGS);
    else hipLaunchKernelGGL((fa_decode_split_kernel<D, 0>), g, b, lds, stream, ORIN_FA_SPLIT_ARGS);
#undef ORIN_FA_SPLIT_ARGS
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess || a.n_splits == 1 || kProbeNoCombine) return e;
    const dim3 cgrid(a.n_head * (D / 64));
#define ORIN_FA_COMBINE_ARGS a.part_o, a.part_ml, a.out, a.n_splits, a.n_head
    if (a.n_splits <= 32) hipLaunchKernelGGL((fa_decode_combine_kernel<D, 4>), cgrid, dim3(512), 0, stream, ORIN_FA_COMBINE_ARGS);
    else if (a.n_splits <= 64) hipLaunchKernelGGL((fa_decode_combine_kernel<D, 8>), cgrid, dim3(512), 0, stream, ORIN_FA_COMBINE_ARGS);
    else if (a.n_splits <= 128) hipLaunchKernelGGL((fa_decode_combine_kernel<D, 16>), cgrid, dim3(512), 0, stream, ORIN_FA_COMBINE_ARGS);
    else hipLaunchKernelGGL((fa_decode_combine_kernel<D, 32>), cgrid, dim3(512), 0, stream, ORIN_FA_COMBINE_ARGS);
#undef ORIN_FA_COMBINE_ARGS
    return hipGetLastError();
}

} // namespace

hipError_t decode_launch(const FaArgs& a, int head_dim, hipStream_t stream) {
    drop_stale_error();
    return head_dim == 128 ? launch<128>(a, stream) : launch<64>(a, stream);
}

// The split kernel uses more than 64 KB of dynamic LDS; the opt-in is set once at init so
// that no launch path touches function attributes (decode runs under stream capture).
namespace {
template <int D, int MODE>
hipError_t allow_lds() {
    const auto kernel = fa_decode_split_kernel<D, MODE>;
    return hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                               DGeom<D>::kLdsB);
}
} // namespace

hipError_t decode_allow_lds() {
    hipError_t e;
    if ((e = allow_lds<128, 0>()) != hipSuccess) return e;
    if ((e = allow_lds<128, 1>()) != hipSuccess) return e;
    if ((e = allow_lds<128, 2>()) != hipSuccess) return e;
    if ((e = allow_lds<64, 0>()) != hipSuccess) return e;
    if ((e = allow_lds<64, 1>()) != hipSuccess) return e;
    return allow_lds<64, 2>();
}

hipError_t decode_stamps(long long* host, size_t n) {
#ifdef ORIN_FA_STAMPS
    if (n > (size_t)kStampWgs * kDecodeWaves * kStampSlots) return hipErrorInvalidValue;
    hipError_t e = hipMemcpyFromSymbol(host, HIP_SYMBOL(g_decode_stamps), n * sizeof(long long)); // (synchronises with the device)
    void* dev = nullptr;
    if (e == hipSuccess) e = hipGetSymbolAddress(&dev, HIP_SYMBOL(g_decode_stamps));
    if (e == hipSuccess) e = hipMemset(dev, 0, sizeof(g_decode_stamps)); // the next launch starts from an empty table
    return e;
#else
    (void)host; (void)n;
    return hipErrorNotSupported;
#endif
}

} // namespace orin_fa
