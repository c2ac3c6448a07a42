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
// needs no shuffle and every per-column quantity is a per-lane scalar.
//
// The three stages of a tile
//     A: S = K Q^T (MFMA)      B: P = 2^(S*c + b) (VALU)      C: O += V^T P, l += 1^T P (MFMA)
// run skewed -- iteration t issues A(t+1), B(t) and C(t-1), which are independent of one
// another -- in one hand-ordered instruction stream, so the matrix pipe works while the vector
// pipe exponentiates.  What keeps the vector share small:
//   * B is one fused multiply-add (scale*log2(e) and the column's offset b = shift - reference
//     maximum; Q itself stays unscaled, so fp16-representable inputs enter the products exactly),
//     one v_exp_f32 per score and one v_cvt_pk_f16_f32 per pair.
//   * Row sums are one more matrix instruction per query block (a ones operand times P).
//   * The reference maximum is lazy: exponentials are computed optimistically while the largest
//     exponent of the tile is tracked; only if it exceeds the fp16-safe bound (on a handful of
//     early tiles) does a slow path move the reference, redo the tile's P and rescale O and l.
// K and V tiles are copied global->LDS by the load unit itself (no staging registers, two
// buffers each per wave, tile base in the scalar offset so the copies need no vector
// arithmetic) in an XOR-swizzled layout that both the 1 KB copy bursts and the operand reads
// hit conflict-free.  Each wave walks its tiles from the diagonal backwards, so the only tile
// that can need the causal mask is handled in the prologue and the steady state is mask-free.
#include "fa_common.hpp"

// Cycle-counter stamps for profiling builds (defined by a prefix header there); nothing otherwise.
#ifndef FA_STAMP
#define FA_STAMP(i)
#endif

namespace orin_fa {
namespace {

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
    static constexpr int kScratchOff = 4 * kTileB;    // 1 KB per wave: 16 bytes per lane for accumulator round trips
    static constexpr int kWaveB = (4 * kTileB + 1024 > kMergeB) ? 4 * kTileB + 1024 : kMergeB;
    static constexpr int kMlOff = kPrefillWaves * kWaveB;
    static constexpr int kQOff = kMlOff + kPrefillWaves * NQB * 16 * 2 * 4; // the query block as fp16, [column][head_dim]
    static constexpr int kQStride = D * 2 + 16;       // (padded: 16 columns read 16 bytes each without bank conflicts)
    static constexpr int kLdsB = kQOff + NQB * 16 * kQStride;
};

// ---------------------------------------------------------------------------------------------
// Instructions with the register file of each operand spelled out.  The kernel keeps its score
// accumulators in ordinary vector registers (the exponentials read them with no copy) and its
// output accumulators and the query operands in the accumulation-register file, and it fixes the issue order of matrix
// and vector work by hand -- neither of which the builtin forms allow.  The price: the compiler
// knows nothing about the hazards of these blocks.
//   (1) Result latency: a non-matrix instruction reads a matrix result only a pipeline stage
//       (at least two later matrix instructions) after it was issued, or behind settle().
//   (2) A matrix instruction must not read an operand in the two cycles after a vector
//       instruction wrote it.  The forms with the _n suffix start with the two wait states and
//       are used wherever compiler-generated vector code may sit right in front of the block
//       (prologue, drain); the main loop uses the bare forms, where every operand was written
//       a long way back (LDS reads, the previous iteration's conversions, loop invariants).
// ---------------------------------------------------------------------------------------------
__device__ __forceinline__ void mfma_v_n(f4& acc, h8 a_op, h8 b_acc) {
    asm volatile("s_nop 1\n\tv_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+v"(acc) : "v"(a_op), "a"(b_acc));
}
__device__ __forceinline__ void mfma_v_zero_n(f4& acc, h8 a_op, h8 b_acc) { // acc = A B
    // early clobber: the destination must not share registers with an operand that dies here
    asm volatile("s_nop 1\n\tv_mfma_f32_16x16x32_f16 %0, %1, %2, 0" : "=&v"(acc) : "v"(a_op), "a"(b_acc));
}
__device__ __forceinline__ void mfma_a_n(f4& acc, h8 a_op, h8 b_op) {
    asm volatile("s_nop 1\n\tv_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+a"(acc) : "v"(a_op), "v"(b_op));
}
__device__ __forceinline__ void mfma_a_zero_n(f4& acc, h8 a_op, h8 b_op) {
    asm volatile("s_nop 1\n\tv_mfma_f32_16x16x32_f16 %0, %1, %2, 0" : "=&a"(acc) : "v"(a_op), "v"(b_op));
}
__device__ __forceinline__ void mfma_v(f4& acc, h8 a_op, h8 b_acc) {
    asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+v"(acc) : "v"(a_op), "a"(b_acc));
}
__device__ __forceinline__ void mfma_v_zero(f4& acc, h8 a_op, h8 b_acc) { // acc = A B
    asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, 0" : "=&v"(acc) : "v"(a_op), "a"(b_acc));
}
__device__ __forceinline__ void mfma_a(f4& acc, h8 a_op, h8 b_op) {
    asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+a"(acc) : "v"(a_op), "v"(b_op));
}
// Lets the matrix pipe drain (32 wait states, more than any 16x16x32 result needs) and stops the
// compiler from moving anything across.
__device__ __forceinline__ void settle() {
    __builtin_amdgcn_sched_barrier(0);
    asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");
    __builtin_amdgcn_sched_barrier(0);
}
// 16 bytes between LDS and the accumulation-register file, without a detour through vector
// registers.  The output accumulators are only ever touched by these and by the matrix
// instructions, which keeps them in that file for the whole kernel.
__device__ __forceinline__ void lds_store_acc(unsigned lds_addr, const f4& acc) {
    asm volatile("ds_write_b128 %0, %1\n\ts_waitcnt lgkmcnt(0)" : : "v"(lds_addr), "a"(acc) : "memory");
}
template <int OFF>
__device__ __forceinline__ void lds_store_acc_nowait(unsigned lds_addr, const f4& acc) { // caller waits
    asm volatile("ds_write_b128 %0, %1 offset:%2" : : "v"(lds_addr), "a"(acc), "n"(OFF) : "memory");
}
// (The accumulator is declared read-write although its old value is dead: a tied operand keeps it in
// the same registers, where a fresh definition on a rarely taken path costs a copy of the whole set.)
__device__ __forceinline__ void lds_load_acc(f4& acc, unsigned lds_addr) {
    asm volatile("s_waitcnt lgkmcnt(0)\n\tds_read_b128 %0, %1\n\ts_waitcnt lgkmcnt(0)" : "+a"(acc) : "v"(lds_addr) : "memory");
}
// The vector side of the main loop, as volatile blocks so that it stays where it is written,
// interleaved with the matrix instructions.
__device__ __forceinline__ void v_fma(float& r, float x, float y, float z) { asm volatile("v_fma_f32 %0, %1, %2, %3" : "=v"(r) : "v"(x), "v"(y), "v"(z)); }
__device__ __forceinline__ void v_exp2(float& r) { asm volatile("v_exp_f32 %0, %0" : "+v"(r)); }
__device__ __forceinline__ void v_cvt_pk(unsigned& r, float lo, float hi) { // two fp32 -> packed fp16, round to nearest even
    asm volatile("v_cvt_pk_f16_f32 %0, %1, %2" : "=v"(r) : "v"(lo), "v"(hi));
}
__device__ __forceinline__ void v_max2(float& r, float x, float y) { asm volatile("v_max_f32 %0, %1, %2" : "=v"(r) : "v"(x), "v"(y)); }
__device__ __forceinline__ void v_max3_acc(float& r, float x, float y) { asm volatile("v_max3_f32 %0, %0, %1, %2" : "+v"(r) : "v"(x), "v"(y)); }

// maxima without the NaN-quieting moves the library fmaxf carries; the trailing wait state is
// for results that feed a lane-swap instruction, which must not read a register in the cycle
// after a vector instruction wrote it (the compiler cannot see that this block is one)
__device__ __forceinline__ float max3(float x, float y, float z) {
    float r;
    asm("v_max3_f32 %0, %1, %2, %3" : "=v"(r) : "v"(x), "v"(y), "v"(z));
    return r;
}
__device__ __forceinline__ float max2(float x, float y) {
    float r;
    asm("v_max_f32 %0, %1, %2\n\ts_nop 1" : "=v"(r) : "v"(x), "v"(y));
    return r;
}
__device__ __forceinline__ float xor_max_fast(float v) { // all-reduce over lanes l, l^16, l^32, l^48; inputs never NaN
    u32x2 s = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    float r = max2(__uint_as_float(s.x), __uint_as_float(s.y));
    s = __builtin_amdgcn_permlane16_swap(__float_as_uint(r), __float_as_uint(r), false, false);
    return max2(__uint_as_float(s.x), __uint_as_float(s.y));
}

// Buffer descriptor words for the global->LDS copies below: base address, stride 0, byte
// count, raw 32-bit format.  Vector offsets at or past the byte count are not fetched.
__device__ __forceinline__ i32x4 make_desc(const void* base, unsigned bytes) {
    const unsigned long long b = reinterpret_cast<unsigned long long>(base);
    return i32x4{(int)(unsigned)b, (int)((unsigned)(b >> 32) & 0xffffu), (int)bytes, 0x00020000};
}

// Four 1 KB global->LDS copies (buffer_load ... lds): lane l of copy i fetches 16 bytes at
// global offset soff + off_i + i*1024 and the load unit writes them to LDS byte lds_base +
// i*1024 + l*16 (the immediate offset advances both addresses).  soff is a scalar and is not
// part of the range check.  The copies count on the vector-memory counter and complete in
// issue order; callers wait with s_waitcnt vmcnt(n).  One asm block, so that M0 (the LDS base)
// cannot change between the copies.
__device__ __forceinline__ void lds_copy_4k(i32x4 desc, unsigned lds_base, int off_even, int off_odd, int soff) {
    asm volatile(
        "s_mov_b32 m0, %0\n\t"
        "buffer_load_dwordx4 %1, %3, %4 offen lds\n\t"
        "buffer_load_dwordx4 %2, %3, %4 offen offset:1024 lds\n\t"
        "buffer_load_dwordx4 %1, %3, %4 offen offset:2048 lds\n\t"
        "buffer_load_dwordx4 %2, %3, %4 offen offset:3072 lds"
        :
        : "s"(lds_base), "v"(off_even), "v"(off_odd), "s"(desc), "s"(soff)
        : "memory", "m0");
}

// 16 bytes per lane from global memory into vector registers, same addressing.  Counts on the
// vector-memory counter like the copies; the consumer waits with s_waitcnt vmcnt(n) (the
// compiler does not know that the registers are filled late).
template <int IMM>
__device__ __forceinline__ void reg_load16(u32x4& dst, i32x4 desc, int off, int soff) {
    asm volatile("buffer_load_dwordx4 %0, %1, %2, %3 offen offset:%4"
                 : "=&v"(dst)
                 : "v"(off), "s"(desc), "s"(soff), "n"(IMM)
                 : "memory");
}

// One such copy, for the main loop, which deals them out between the matrix instructions so
// that the vector-memory issue queue never backs up.
template <int IMM>
__device__ __forceinline__ void lds_copy_1k(i32x4 desc, unsigned lds_base, int off, int soff) {
    asm volatile(
        "s_mov_b32 m0, %0\n\t"
        "buffer_load_dwordx4 %1, %2, %3 offen offset:%4 lds"
        :
        : "s"(lds_base), "v"(off), "s"(desc), "s"(soff), "n"(IMM)
        : "memory", "m0");
}

template <int D, int NQB, int TQ>
__global__ __launch_bounds__(kPrefillWaves * 64) void fa_prefill_kernel(const FaArgs a) {
    using G = PGeom<D, NQB>;
    constexpr int kWaves = kPrefillWaves;
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    FA_STAMP(0);

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6); // uniform: tile indices live in scalar registers
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
    const int kv_end = n_past + tok_hi;   // the workgroup's columns see rows [0, kv_end) at most
    const int full_end = n_past + t0 + 1; // rows below this are visible to every column
    const int n_tiles = (kv_end + kTile - 1) / kTile;
    // Wave w owns tiles w, w+4, ...; step j visits them from the highest down.  Steps past the
    // end map to negative tiles, whose copies fetch nothing.
    const int n_mine = n_tiles > wave ? (n_tiles - 1 - wave) / kWaves + 1 : 0;
    auto tile_of = [&](int j) { return wave + kWaves * (n_mine - 1 - j); };

    unsigned char* const ws = smem + wave * G::kWaveB; // this wave's LDS slice
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
    // K operand read: lane (col, grp) takes row t*16 + col, logical chunk kk*4 + grp.  The
    // pointers carry every per-lane term; buffer parity and sub-tile are immediate offsets.
    const unsigned char* kp[G::kSteps];
#pragma unroll
    for (int kk = 0; kk < G::kSteps; ++kk) kp[kk] = ws + G::kKOff + col * G::kRowB + (((kk * 4 + grp) ^ (col & 7)) * 16);
    // V transposing read: lane (col, grp) addresses row grp*4 + col/4 (+16 for the second half),
    // 8-byte column db*4 + col%4.
    const unsigned char* vp[G::kDBlk];
    {
        const int r0 = grp * 4 + (col >> 2), sw = r0 & 7;
#pragma unroll
        for (int db = 0; db < G::kDBlk; ++db)
            vp[db] = ws + G::kVOff + r0 * G::kRowB + (((db * 2 + ((col & 3) >> 1)) ^ sw) * 16) + (col & 1) * 8;
    }

    // Prologue copies: the whole offset is in the (range-checked) vector operand, so rows at or
    // past kv_end of the diagonal tile, and tiles below zero, are not fetched.
    auto copy_checked = [&](const i32x4& desc, unsigned lds_dst, int tile) {
        const int base = tile * G::kTileB;
        lds_copy_4k(desc, lds_dst, base + g_off[0], base + g_off[kOdd], 0);
        if (G::kCopies > 4) lds_copy_4k(desc, lds_dst + 4096, base + 4096 + g_off[0], base + 4096 + g_off[kOdd], 0);
    };
    // Main-loop copies: every tile they name is either wholly inside the visible range, and its
    // base travels as the scalar offset, or below zero, and then the descriptor is emptied.
    auto copy_fast = [&](const i32x4& desc, unsigned lds_dst, int tile) {
        const bool live = tile >= 0;
        const i32x4 d = i32x4{desc[0], desc[1], live ? desc[2] : 0, desc[3]};
        const int soff = live ? tile * G::kTileB : 0;
        lds_copy_4k(d, lds_dst, g_off[0], g_off[kOdd], soff);
        if (G::kCopies > 4) lds_copy_4k(d, lds_dst + 4096, g_off[0], g_off[kOdd], soff + 4096);
    };
    // Copy number i (of kCopies) of a main-loop tile; desc and soff as prepared by live_desc / tile_soff.
    auto live_desc = [&](const i32x4& desc, int tile) { return i32x4{desc[0], desc[1], tile >= 0 ? desc[2] : 0, desc[3]}; };
    auto tile_soff = [&](int tile) { return tile >= 0 ? tile * G::kTileB : 0; };
    auto copy_one = [&](auto ic, const i32x4& d, unsigned lds_dst, int soff) {
        constexpr int i = decltype(ic)::value;
        constexpr int half = i / 4, sub = i % 4;
        lds_copy_1k<sub * 1024>(d, lds_dst + half * 4096, g_off[(sub & 1) ? kOdd : 0], soff + half * 4096);
    };
    auto k_buf = [&](int par) { return ws_addr + G::kKOff + par * G::kTileB; };
    auto v_buf = [&](int par) { return ws_addr + G::kVOff + par * G::kTileB; };

    // ---- state ----
    h8 q[NQB][G::kSteps]; // B operands of A: the query columns, fp16
    float nb[NQB];        // each column's exponent offset: shift - reference maximum * c (log2 units)
    f4 o[NQB][G::kDBlk];  // O^T accumulators (accumulation registers)
    f4 lacc[NQB];         // row sums: every element of a lane's four holds the column's sum
    f4 s[2][2][NQB];      // scores: [parity][sub-tile][query block]
    u32x4 pw[2][NQB];     // P as packed fp16: [parity][query block]
    h8 ones;
#pragma unroll
    for (int e = 0; e < 8; ++e) ones[e] = (_Float16)1.0f;
    asm volatile("" : "+v"(ones)); // stays in registers; never rematerialised in front of a matrix instruction

    const unsigned scratch_addr = ws_addr + G::kScratchOff + lane * 16;
    float* const scratch = reinterpret_cast<float*>(ws + G::kScratchOff) + lane * 4;

    // ---- prologue loads, most urgent first: the query block, then the first K tile; the rest of
    // the first two tiles follows once the queries are on their way into LDS.  All of them are
    // issued by hand and counted on the vector-memory counter, so that no wait has to sit out
    // the loads behind the one it needs.
    // The query block is loaded once per workgroup: wave w takes a quarter of the columns with
    // coalesced 16-byte loads (a column is D/4 lanes wide), converts to fp16 and leaves it in LDS;
    // after the barrier every wave picks up its B operands from there. ----
    constexpr int kColsPerLoad = 256 / D;              // columns one load instruction covers
    constexpr int kQLoads = NQB * 4 / kColsPerLoad;    // load instructions per wave
    u32x4 qraw[kQLoads];
    float qmul[kQLoads];
    int qcol[kQLoads];
    {
        const i32x4 qdesc = make_desc(a.q, (unsigned)batch * a.n_head * D * 4);
        static_for<0, kQLoads>([&](auto jc) {
            constexpr int j = decltype(jc)::value;
            const int c = wave * (NQB * 4) + j * kColsPerLoad + lane / (D / 4);
            const int tok = t0 + c % TQ;
            const int hl = head_lo + c / TQ;
            const bool valid = (hl < a.r) && (tok < batch);
            qcol[j] = c;
            qmul[j] = valid ? a.qsign : 0.0f; // c > 0 multiplies the scores; the sign of the scale goes here
            const int q_off = valid ? ((tok * a.n_head + kvh * a.r + hl) * D + (lane % (D / 4)) * 4) * 4 : 0;
            reg_load16<0>(qraw[j], qdesc, q_off, 0);
        });
    }
    if (n_mine > 0) copy_checked(kdesc, k_buf(0), tile_of(0));
    FA_STAMP(9);
    // O = 0, l = 0: a matrix instruction with a zero addend writes the accumulation registers
    // without touching memory.
    {
        h8 zero;
#pragma unroll
        for (int e = 0; e < 8; ++e) zero[e] = (_Float16)0.0f;
        asm volatile("" : "+v"(zero));
#pragma unroll
        for (int qb = 0; qb < NQB; ++qb) {
#pragma unroll
            for (int db = 0; db < G::kDBlk; ++db) mfma_a_zero_n(o[qb][db], zero, zero);
            mfma_a_zero_n(lacc[qb], zero, zero);
        }
    }
    if (n_mine > 0) {
        // V buffer 0 receives the diagonal tile, whose rows at or past kv_end are not fetched:
        // clear it first, so that no stale bit pattern meets a zero weight (0 * NaN is not 0).
#pragma unroll
        for (int i = 0; i < G::kCopies; ++i)
            *reinterpret_cast<u32x4*>(ws + G::kVOff + i * 1024 + lane * 16) = u32x4{0u, 0u, 0u, 0u};
    }
    FA_STAMP(10);
    // ---- query block -> LDS (fp16) ----
    if (n_mine > 0) __builtin_amdgcn_s_waitcnt(0x0F70 | (G::kCopies & 15) | ((G::kCopies >> 4) << 14)); // vmcnt: the queries are in, K(0) may be in flight
    else __builtin_amdgcn_s_waitcnt(0x0F70);
#pragma unroll
    for (int j = 0; j < kQLoads; ++j) {
        h4 hv;
#pragma unroll
        for (int e = 0; e < 4; ++e) hv[e] = (_Float16)(__uint_as_float(qraw[j][e]) * qmul[j]);
        *reinterpret_cast<h4*>(smem + G::kQOff + qcol[j] * G::kQStride + (lane % (D / 4)) * 8) = hv;
    }
    __syncthreads(); // (also orders the clearing of V buffer 0 before the copy into it)
    if (n_mine > 0) {
        copy_checked(vdesc, v_buf(0), tile_of(0));
        copy_checked(kdesc, k_buf(1), tile_of(1));
        copy_checked(vdesc, v_buf(1), tile_of(1));
    }
    int limit[NQB];
#pragma unroll
    for (int qb = 0; qb < NQB; ++qb) {
        const int c = qb * 16 + col;
        const int tok = t0 + c % TQ;
        const int hl = head_lo + c / TQ;
        limit[qb] = (hl < a.r) && (tok < batch) ? n_past + tok + 1 : 0x7fffffff;
#pragma unroll
        for (int kk = 0; kk < G::kSteps; ++kk) {
            const h8 hv = *reinterpret_cast<const h8*>(smem + G::kQOff + c * G::kQStride + (kk * 32 + grp * 8) * 2);
            asm volatile("" : "=a"(q[qb][kk]) : "0"(hv)); // parked in the accumulation-register file for good
        }
    }
    FA_STAMP(1);

    // The copies are tracked by the vector-memory counter and complete in issue order: waiting
    // until at most `newer` younger ones are outstanding guarantees a tile has landed.
    auto wait_copies = [&](auto newer) {
        constexpr int n = decltype(newer)::value;
        __builtin_amdgcn_s_waitcnt(0x0F70 | (n & 15) | ((n >> 4) << 14)); // vmcnt(n), other counters untouched
        wave_lds_sync();
    };
    constexpr int kC = G::kCopies;

    if (n_mine > 0) {
        const int R = n_mine - 1; // steps after step 0
        // Prologue form of A: S[spar] = K[kpar] Q^T with a zero addend, operands read up front.
        auto stage_a0 = [&](auto kpar, auto spar) {
            constexpr int KP = decltype(kpar)::value, SP = decltype(spar)::value;
            h8 ka[G::kSteps][2];
#pragma unroll
            for (int kk = 0; kk < G::kSteps; ++kk)
#pragma unroll
                for (int t = 0; t < 2; ++t)
                    ka[kk][t] = *reinterpret_cast<const h8*>(kp[kk] + KP * G::kTileB + t * 16 * G::kRowB);
#pragma unroll
            for (int kk = 0; kk < G::kSteps; ++kk)
#pragma unroll
                for (int t = 0; t < 2; ++t)
#pragma unroll
                    for (int qb = 0; qb < NQB; ++qb) {
                        if (kk == 0) mfma_v_zero_n(s[SP][t][qb], ka[kk][t], q[qb][kk]);
                        else mfma_v_n(s[SP][t][qb], ka[kk][t], q[qb][kk]);
                        // With few query blocks the next k-step of the same accumulator is only a
                        // couple of instructions away; give the result time to leave the pipe.
                        if (2 * NQB < 8) asm volatile("s_nop 15");
                    }
        };
        // Copy issue order: K0 V0 K1 V1 | K2 (step 0) | K3 V2 (step 1) | K4 V3 (step 2) | ...
        // (within a step, K goes out over the first tickets and V over the last)
        // ---- step 0: the diagonal tile, the only one that can need the causal mask ----
        wait_copies(IntC<3 * kC>{});        // K0 landed (V0 K1 V1 may be in flight)
        stage_a0(IntC<0>{}, IntC<0>{});     // S(0)
        __builtin_amdgcn_s_waitcnt(0xC07F); // its LDS reads have returned: K buffer 0 is free
        copy_fast(kdesc, k_buf(0), tile_of(2));
        if (R > 0) {
            wait_copies(IntC<2 * kC>{});    // K1 landed (V1 K2 may be in flight)
            stage_a0(IntC<1>{}, IntC<1>{}); // S(1)
        }
        settle();
        FA_STAMP(2);
        // Reference maximum of each column: over its visible scores of tile 0 and, when there is
        // one, tile 1 (every row of which is visible to every column).  A column with no visible
        // row in this wave keeps weight zero whatever the reference.
        {
            const int row0 = tile_of(0) * kTile + grp * 4;
            const bool masked = tile_of(0) * kTile + kTile > full_end;
#pragma unroll
            for (int qb = 0; qb < NQB; ++qb) {
                float v[8];
#pragma unroll
                for (int t = 0; t < 2; ++t)
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        v[t * 4 + i] = s[0][t][qb][i];
                        if (masked && row0 + t * 16 + i >= limit[qb]) v[t * 4 + i] = -INFINITY;
                    }
                float mx = max3(v[0], v[1], v[2]);
                mx = max3(mx, v[3], v[4]);
                mx = max3(mx, v[5], v[6]);
                mx = max2(mx, v[7]);
                if (R > 0) {
                    mx = max3(mx, s[1][0][qb][0], s[1][0][qb][1]);
                    mx = max3(mx, s[1][0][qb][2], s[1][0][qb][3]);
                    mx = max3(mx, s[1][1][qb][0], s[1][1][qb][1]);
                    mx = max3(mx, s[1][1][qb][2], s[1][1][qb][3]);
                    mx = max2(mx, mx);
                }
                mx = xor_max_fast(mx);
                nb[qb] = kPShift - (mx == -INFINITY ? 0.0f : mx) * a.c;
                h8 ph;
#pragma unroll
                for (int e = 0; e < 8; ++e) ph[e] = (_Float16)fast_exp2(__builtin_fmaf(v[e], a.c, nb[qb]));
                pw[0][qb] = __builtin_bit_cast(u32x4, ph);
            }
        }
        settle(); // (the vector writes of P are well clear of the next matrix instruction)
        FA_STAMP(3);

        // ---- steps t >= 1: A(t+1), B(t) and C(t-1) in one instruction stream.  The matrix
        // instructions are cut into groups of NQB that share an LDS operand (A: one (k-step,
        // sub-tile) of K; C: one 16-wide block of V^T; last, the row sums), ordered A0 C0 A1 C1
        // ... L; the 24 vector instructions per query block of B are dealt out evenly between
        // them.  Operands are read from LDS kAhead groups ahead of their use.
        // `newer` = copies issued after K(t+1) and before the wait: none at t == 1 (step 0 issued
        // K(2) last), V(t) afterwards. ----
        static_assert(2 * G::kSteps == G::kDBlk, "A and C groups alternate one to one");
        constexpr int kGroups = 2 * G::kSteps + G::kDBlk; // groups with an LDS operand
        constexpr int kTickets = (kGroups + 1) * NQB;     // matrix instructions per step
        constexpr int kItems = 24 * NQB;                  // vector instructions of B per step
        constexpr int kAhead = 3;
        constexpr float kBound = kLazy + kPShift;         // largest exponent P may be built from
        constexpr float kBoundP = 32768.0f;               // = 2^kBound
        // (The last step has no tile t+1: its A stage multiplies whatever the K buffer holds and
        // nobody reads the result -- cheaper than a second copy of the loop body without it.)
        float c = a.c;
        asm volatile("" : "+v"(c)); // a vector register for the whole loop, not a move per step
        auto body = [&](auto tpar, auto newer, int t) {
            constexpr int TP = decltype(tpar)::value; // t & 1
            // (Every LDS read of the previous step has been consumed by a matrix instruction that
            // was issued before this point, so the K buffer A(t) read is free.)
            // K(t+2) goes to the buffer A(t) read; its copies are dealt out over the first tickets.
            // (Issued after this step's wait, they are not among the `newer` copies any more.)
            const i32x4 kd = live_desc(kdesc, tile_of(t + 2));
            const int ksoff = tile_soff(tile_of(t + 2));
            const i32x4 vd = live_desc(vdesc, tile_of(t + 1));
            const int vsoff = tile_soff(tile_of(t + 1));
            wait_copies(newer);                          // K(t+1) landed; V(t-1) is older
            h8 gop[kGroups];
            auto issue_read = [&](auto gc) {
                constexpr int g = decltype(gc)::value;
                __builtin_amdgcn_sched_barrier(0);
                if constexpr (g % 2 == 0) {
                    constexpr int kk = (g / 2) / 2, tt = (g / 2) % 2;
                    gop[g] = *reinterpret_cast<const h8*>(kp[kk] + (TP ^ 1) * G::kTileB + tt * 16 * G::kRowB);
                } else {
                    constexpr int db = g / 2;
                    const h4 v0 = lds_read_tr(vp[db] + (TP ^ 1) * G::kTileB);
                    const h4 v1 = lds_read_tr(vp[db] + (TP ^ 1) * G::kTileB + 16 * G::kRowB);
                    gop[g] = __builtin_shufflevector(v0, v1, 0, 1, 2, 3, 4, 5, 6, 7);
                }
                __builtin_amdgcn_sched_barrier(0);
            };
            float pe[NQB][8];
            float amax;
            // Vector instruction j of B(t).  Per query block and pair of scores: two multiply-adds
            // (the exponents), two exponentials, the running maximum of the weights, the conversion;
            // no instruction reads the result of the one right before it.
            auto item = [&](auto jc) {
                constexpr int j = decltype(jc)::value;
                constexpr int qb = j / 24, r = j % 24;
                // 0 multiply-add, 1 maximum, 2 exponential, 3 conversion
                constexpr int kind[24] = {0, 0, 2, 2, 0, 0, 1, 2, 2, 3, 0, 0, 1, 2, 2, 3, 0, 0, 1, 2, 2, 3, 1, 3};
                constexpr int arg[24] = {0, 1, 0, 1, 2, 3, 0, 2, 3, 0, 4, 5, 1, 4, 5, 1, 6, 7, 2, 6, 7, 2, 3, 3};
                constexpr int x = arg[r];
                if constexpr (kind[r] == 0) {
                    v_fma(pe[qb][x], s[TP][x / 4][qb][x % 4], c, nb[qb]);
                } else if constexpr (kind[r] == 2) {
                    v_exp2(pe[qb][x]);
                } else if constexpr (kind[r] == 3) {
                    unsigned packed;
                    v_cvt_pk(packed, pe[qb][2 * x], pe[qb][2 * x + 1]);
                    pw[TP][qb][x] = packed;
                } else {
                    if constexpr (j == 6) v_max2(amax, pe[qb][2 * x], pe[qb][2 * x + 1]);
                    else v_max3_acc(amax, pe[qb][2 * x], pe[qb][2 * x + 1]);
                }
            };
            static_for<0, kAhead>(issue_read);
            static_for<0, kTickets>([&](auto ic) {
                constexpr int i = decltype(ic)::value;
                constexpr int g = i / NQB, m = i % NQB;
                if constexpr (m == 0 && g + kAhead < kGroups) issue_read(IntC<g + kAhead>{});
                if constexpr (g == kGroups) {
                    mfma_a(lacc[m], ones, __builtin_bit_cast(h8, pw[TP ^ 1][m]));
                } else if constexpr (g % 2 == 0) {
                    constexpr int kk = (g / 2) / 2, tt = (g / 2) % 2;
                    if constexpr (kk == 0) mfma_v_zero(s[TP ^ 1][tt][m], gop[g], q[m][kk]);
                    else mfma_v(s[TP ^ 1][tt][m], gop[g], q[m][kk]);
                } else {
                    mfma_a(o[m][g / 2], gop[g], __builtin_bit_cast(h8, pw[TP ^ 1][m]));
                }
                static_for<(i * kItems) / kTickets, ((i + 1) * kItems) / kTickets>(item);
                if constexpr (i % 2 == 1 && i / 2 < kC) copy_one(IntC<i / 2>{}, kd, k_buf(TP), ksoff);
                // V(t+1) goes to the buffer C(t-1) reads: its copies wait for the last of those reads
                // to be consumed, which the row-sum group (no LDS operand) marks.
                if constexpr (g == kGroups) {
                    constexpr int per = (kC + NQB - 1) / NQB;
                    static_for<m * per, (m + 1) * per < kC ? (m + 1) * per : kC>([&](auto cc) { copy_one(cc, vd, v_buf(TP ^ 1), vsoff); });
                }
            });
            // S(t+1) is alive to the end of the step even when nobody reads it (last step): its
            // registers must not be handed out while the matrix instructions that write them are in flight.
#pragma unroll
            for (int qb = 0; qb < NQB; ++qb) {
                asm volatile("" : : "v"(s[TP ^ 1][0][qb]));
                asm volatile("" : : "v"(s[TP ^ 1][1][qb]));
            }
            // ---- slow path: some exponent of this tile is above the bound.  Move the reference of
            // the columns concerned to their new maximum, redo P(t) and rescale O and l -- one
            // accumulator at a time through a 16-byte-per-lane LDS scratch, so that they never
            // become operands of a vector instruction. ----
            if (__builtin_amdgcn_ballot_w64(amax > kBoundP) != 0) {
                settle(); // C(t-1) has left the matrix pipe
                float alpha[NQB];
#pragma unroll
                for (int qb = 0; qb < NQB; ++qb) {
                    float mx = max3(s[TP][0][qb][0], s[TP][0][qb][1], s[TP][0][qb][2]);
                    mx = max3(mx, s[TP][0][qb][3], s[TP][1][qb][0]);
                    mx = max3(mx, s[TP][1][qb][1], s[TP][1][qb][2]);
                    mx = xor_max_fast(max2(mx, s[TP][1][qb][3]));
                    const float top = __builtin_fmaf(mx, c, nb[qb]); // the column's largest exponent
                    const float delta = top > kBound ? top - kPShift : 0.0f;
                    alpha[qb] = fast_exp2(-delta);
                    nb[qb] -= delta;
                    h8 ph;
#pragma unroll
                    for (int e = 0; e < 8; ++e) ph[e] = (_Float16)fast_exp2(__builtin_fmaf(s[TP][e / 4][qb][e % 4], c, nb[qb]));
                    pw[TP][qb] = __builtin_bit_cast(u32x4, ph);
                }
                auto scale_acc = [&](f4& acc, float al) {
                    lds_store_acc(scratch_addr, acc);
                    f4 x = *reinterpret_cast<f4*>(scratch);
                    x *= al;
                    *reinterpret_cast<f4*>(scratch) = x;
                    lds_load_acc(acc, scratch_addr);
                };
                static_for<0, NQB>([&](auto qbc) {
                    constexpr int qb = decltype(qbc)::value;
                    static_for<0, G::kDBlk>([&](auto dbc) { scale_acc(o[qb][decltype(dbc)::value], alpha[qb]); });
                    scale_acc(lacc[qb], alpha[qb]);
                });
                settle();
            }
        };
        if (R >= 1) body(IntC<1>{}, IntC<0>{}, 1);
        int t = 2;
        for (; t + 1 <= R; t += 2) {
            body(IntC<0>{}, IntC<kC>{}, t);
            body(IntC<1>{}, IntC<kC>{}, t + 1);
        }
        if (t == R) body(IntC<0>{}, IntC<kC>{}, t);
        FA_STAMP(4);
        // ---- drain: C(R) ----
        wait_copies(IntC<0>{});
        settle(); // P(R) was converted just above
        {   // O += V(R)^T P(R), l += 1^T P(R); both live in the buffers of parity R & 1
            const bool odd = (R & 1) != 0;
            const int v_par = odd ? G::kTileB : 0;
            h8 va[G::kDBlk], pl[NQB];
            if (odd) {
#pragma unroll
                for (int qb = 0; qb < NQB; ++qb) pw[0][qb] = pw[1][qb];
            }
#pragma unroll
            for (int db = 0; db < G::kDBlk; ++db) {
                const h4 v0 = lds_read_tr(vp[db] + v_par);
                const h4 v1 = lds_read_tr(vp[db] + v_par + 16 * G::kRowB);
                va[db] = __builtin_shufflevector(v0, v1, 0, 1, 2, 3, 4, 5, 6, 7);
            }
#pragma unroll
            for (int qb = 0; qb < NQB; ++qb) pl[qb] = __builtin_bit_cast(h8, pw[0][qb]);
#pragma unroll
            for (int db = 0; db < G::kDBlk; ++db)
#pragma unroll
                for (int qb = 0; qb < NQB; ++qb) mfma_a_n(o[qb][db], va[db], pl[qb]);
#pragma unroll
            for (int qb = 0; qb < NQB; ++qb) mfma_a_n(lacc[qb], ones, pl[qb]);
        }
        __builtin_amdgcn_s_waitcnt(0xC07F); // every read of the tile buffers has returned: the merge reuses them
    } else {
#pragma unroll
        for (int qb = 0; qb < NQB; ++qb) nb[qb] = 0.0f;
    }
    settle(); // O and l are out of the matrix pipe
    wave_lds_sync();
    FA_STAMP(5);

    // ---- merge the four waves through LDS ----
    // (m, l) per wave and column, m = the reference in log2 units (the common shift cancels);
    // a wave that saw no visible row of a column has l = 0 and is given m = -inf (weight 0).
    float* const ml = reinterpret_cast<float*>(smem + G::kMlOff);
#pragma unroll
    for (int qb = 0; qb < NQB; ++qb) {
        asm volatile("" : "+a"(lacc[qb])); // pins the read below behind the settled pipe
        const float l_tot = lacc[qb][0];
        if (grp == 0) {
            ml[(wave * NQB * 16 + qb * 16 + col) * 2 + 0] = l_tot > 0.0f ? -nb[qb] : -INFINITY;
            ml[(wave * NQB * 16 + qb * 16 + col) * 2 + 1] = l_tot;
        }
    }
    const unsigned obuf_addr = ws_addr + (col * G::kOStride + grp * 4) * 4;
    static_for<0, NQB>([&](auto qbc) {
        static_for<0, G::kDBlk>([&](auto dbc) {
            constexpr int qb = decltype(qbc)::value, db = decltype(dbc)::value;
            lds_store_acc_nowait<(qb * 16 * G::kOStride + db * 16) * 4>(obuf_addr, o[qb][db]);
        });
    });
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    FA_STAMP(6);
    __syncthreads();
    FA_STAMP(7);

    // Four threads per column: the weights are computed once, then each thread merges and stores
    // a quarter of the column's head_dim in 16-byte pieces (the four pieces of a step are one
    // contiguous 64 bytes of the output row).
    constexpr int kCols = NQB * 16;
    const int c = threadIdx.x >> 2, part = threadIdx.x & 3;
    const int tok = t0 + c % TQ;
    const int hl = head_lo + c / TQ;
    if (c < kCols && hl < a.r && tok < batch) {
        float wgt[kWaves];
        float m_all = -INFINITY, l_all = 0.0f;
#pragma unroll
        for (int w = 0; w < kWaves; ++w) {
            wgt[w] = ml[(w * kCols + c) * 2 + 0];
            m_all = fmaxf(m_all, wgt[w]);
        }
#pragma unroll
        for (int w = 0; w < kWaves; ++w) {
            wgt[w] = fast_exp2(wgt[w] - m_all); // the wave that holds the column's diagonal has a finite m
            l_all += ml[(w * kCols + c) * 2 + 1] * wgt[w];
        }
        const float inv = l_all > 0.0f ? 1.0f / l_all : 0.0f;
        float* const dst = a.out + ((size_t)tok * a.n_head + kvh * a.r + hl) * D;
#pragma unroll
        for (int j = 0; j < D / 16; ++j) {
            const int d4 = (j * 4 + part) * 4;
            f4 acc = f4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int w = 0; w < kWaves; ++w)
                acc += *reinterpret_cast<const f4*>(smem + w * G::kWaveB + ((size_t)c * G::kOStride + d4) * 4) * wgt[w];
            *reinterpret_cast<f4*>(dst + d4) = acc * inv;
        }
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
    if ((e = allow_lds<D, 2, 4>()) != hipSuccess) return e;
    return allow_lds<D, 4, 8>();
}

template <int D>
hipError_t launch(FaArgs a, int cu_count, hipStream_t stream) {
    // Column packing per GQA ratio: (16-column blocks, tokens per workgroup).
    // r <= 4: 16 tokens x r heads; r in 5..8: 8 tokens x up to 8 heads; larger ratios
    // are cut into groups of 8 heads that each re-read the KV head.
    const int r = a.r;
    int nqb, tq;
    if (r <= 4) { nqb = r; tq = 16; }
    else if (r <= 6) { nqb = 3; tq = 8; }
    else { nqb = 4; tq = 8; }
    // A workgroup occupies a whole CU and the kernel lasts as long as its longest workgroup, so
    // a grid that leaves half the CUs idle is better cut finer: 4 tokens x up to 8 heads, which
    // halves the columns (and the time) per workgroup for r = 5..8.
    if (r > 4 && 2 * a.n_kv * ((r + nqb * 16 / tq - 1) / (nqb * 16 / tq)) * ((a.batch + tq - 1) / tq) <= cu_count) {
        nqb = 2;
        tq = 4;
    }
    const int heads_per_group = nqb * 16 / tq;
    a.n_hgroups = (r + heads_per_group - 1) / heads_per_group;
    a.n_ttiles = (a.batch + tq - 1) / tq;
    const int grid = a.n_kv * a.n_hgroups * a.n_ttiles;
    switch (nqb * 100 + tq) {
        case 204: return launch_kernel<D, 2, 4>(a, grid, stream);
        case 116: return launch_kernel<D, 1, 16>(a, grid, stream);
        case 216: return launch_kernel<D, 2, 16>(a, grid, stream);
        case 316: return launch_kernel<D, 3, 16>(a, grid, stream);
        case 416: return launch_kernel<D, 4, 16>(a, grid, stream);
        case 308: return launch_kernel<D, 3, 8>(a, grid, stream);
        default:  return launch_kernel<D, 4, 8>(a, grid, stream);
    }
}

} // namespace

hipError_t prefill_launch(const FaArgs& a, int head_dim, int cu_count, hipStream_t stream) {
    return head_dim == 128 ? launch<128>(a, cu_count, stream) : launch<64>(a, cu_count, stream);
}

// The kernels use more than 64 KB of dynamic LDS; the opt-in is set once per kernel at init.
hipError_t prefill_allow_lds() {
    hipError_t e = allow_lds_all<128>();
    return e != hipSuccess ? e : allow_lds_all<64>();
}

} // namespace orin_fa
