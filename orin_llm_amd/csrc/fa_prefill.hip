// Causal chunked-prefill GQA attention over the fp16 KV cache for gfx950 (MI355X).
//
// Replaces the reference's flash_attention_prefill_mma_k and its launcher (reference:
// src/kernels.cu:1347-1568, 1944-1981).
//
// A workgroup is 4 wave64s that own one KV head, a block of NQB*16 query columns (TQ tokens x
// the heads of the group) and the 32-row KV tiles those columns can see; wave w takes tiles
// w, w+4, ... and keeps its own online-softmax state, so the main loop has no workgroup
// barrier.  S^T = K Q^T and O^T = V^T P run on v_mfma_f32_16x16x32_f16: the accumulator layout
// of the first product (lane = query column, 4 KV rows per lane-group) is the B-operand layout
// of the second once the 32 KV rows of a tile are numbered (lane-group, sub-tile, row), so P
// needs no shuffle and every rescale factor is a per-lane scalar.
//
// The three stages of a tile
//     A: S = K Q^T (MFMA)      B: P = 2^(S*c - m) (VALU)      C: O += V^T P (MFMA)
// run skewed -- iteration t issues A(t+1), B(t) and C(t-1), which are independent of one
// another, so the matrix pipe works while the vector pipe exponentiates.  K and V tiles are
// copied global->LDS by the load unit itself (no staging registers, two buffers each per wave)
// in an XOR-swizzled layout that both the 1 KB copy bursts and the operand reads hit
// conflict-free.  Each wave walks its tiles from the diagonal backwards, so the only tile
// that can need the causal mask is handled in the prologue and the steady state is mask-free.
#include "fa_common.hpp"

namespace orin_fa {
namespace {

// Cycle-counter stamps for profiling builds (defined by a prefix header there); nothing otherwise.
#ifndef FA_STAMP
#define FA_STAMP(i)
#endif

constexpr float kUnsetRef = -1.0e30f; // reference maximum of a column that has seen no visible key yet

__device__ __forceinline__ float max2(float x, float y);
__device__ __forceinline__ float xor_max_fast(float v) { // all-reduce over lanes l, l^16, l^32, l^48; inputs never NaN
    u32x2 s = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    float r = max2(__uint_as_float(s.x), __uint_as_float(s.y));
    s = __builtin_amdgcn_permlane16_swap(__float_as_uint(r), __float_as_uint(r), false, false);
    return max2(__uint_as_float(s.x), __uint_as_float(s.y));
}

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

    FA_STAMP(0);
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

    FA_STAMP(1);
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

        FA_STAMP(2);
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

        FA_STAMP(3);
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
        FA_STAMP(4);
        // ---- drain: C(R) ----
        wait_copies(IntC<0>{});
        settle(); // P(R) was converted just above
        if (R & 1) stage_c(IntC<1>{});
        else stage_c(IntC<0>{});
        __builtin_amdgcn_s_waitcnt(0xC07F); // every read of the tile buffers has returned: the merge reuses them
        settle();                            // and O is out of the matrix pipe
        wave_lds_sync();
    }

    FA_STAMP(5);
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
    FA_STAMP(6);
    __syncthreads();
    FA_STAMP(7);

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
    FA_STAMP(8);
}

template <int D, int NQB, int TQ>
hipError_t launch_kernel(const FaArgs& a, int grid, hipStream_t stream) {
    constexpr int lds = PGeom<D, NQB>::kLdsB;
    hipLaunchKernelGGL((fa_prefill_kernel<D, NQB, TQ>), dim3(grid), dim3(kPrefillWaves * 64), lds, stream, a);
    return hipGetLastError();
}

template <int D, int NQB, int TQ>
hipError_t allow_lds() {
    return hipFuncSetAttribute(reinterpret_cast<const void*>(fa_prefill_kernel<D, NQB, TQ>),
                               hipFuncAttributeMaxDynamicSharedMemorySize, PGeom<D, NQB>::kLdsB);
}

template <int D>
hipError_t allow_lds_all() {
    hipError_t e;
    if ((e = allow_lds<D, 1, 16>()) != hipSuccess) return e;
    if ((e = allow_lds<D, 2, 16>()) != hipSuccess) return e;
    if ((e = allow_lds<D, 3, 16>()) != hipSuccess) return e;
    if ((e = allow_lds<D, 4, 16>()) != hipSuccess) return e;
    if ((e = allow_lds<D, 3, 8>()) != hipSuccess) return e;
    return allow_lds<D, 4, 8>();
}

template <int D>
hipError_t launch(FaArgs a, hipStream_t stream) {
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
        case 116: return launch_kernel<D, 1, 16>(a, grid, stream);
        case 216: return launch_kernel<D, 2, 16>(a, grid, stream);
        case 316: return launch_kernel<D, 3, 16>(a, grid, stream);
        case 416: return launch_kernel<D, 4, 16>(a, grid, stream);
        case 308: return launch_kernel<D, 3, 8>(a, grid, stream);
        default:  return launch_kernel<D, 4, 8>(a, grid, stream);
    }
}

} // namespace

hipError_t prefill_launch(const FaArgs& a, int head_dim, hipStream_t stream) {
    return head_dim == 128 ? launch<128>(a, stream) : launch<64>(a, stream);
}

// The kernels use more than 64 KB of dynamic LDS; the opt-in is set once per kernel at init.
hipError_t prefill_allow_lds() {
    hipError_t e = allow_lds_all<128>();
    return e != hipSuccess ? e : allow_lds_all<64>();
}

} // namespace orin_fa
