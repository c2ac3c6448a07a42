// Causal chunked-prefill GQA attention over the fp16 KV cache for gfx950 (MI355X).
//
// Replaces the reference's flash_attention_prefill_mma_k and its launcher (reference:
// src/kernels.cu:1347-1568, 1944-1981).
//
// A workgroup is 4 wave64s that own one KV head, a block of NCB*32 query columns (tq tokens x
// the heads of the group) and the 32-row KV tiles those columns can see; wave w takes tiles
// w, w+4, ... and keeps its own online-softmax state, so the main loop has no workgroup
// barrier.  S^T = K Q^T and O^T = V^T P run on v_mfma_f32_32x32x16_f16 (a single wave reaches
// 94 % of the matrix pipe's rate with this shape against 75 % with 16x16x32, and each
// instruction leaves three times the room for vector work beside it).  The accumulator layout
// of the first product -- lane = query column, lane-half h holds KV rows 8q + 4h + 0..3 -- is
// the B-operand layout of the second once the 16 KV rows of a k-step are numbered
// (lane-half, register), so P needs no shuffle and every per-column quantity is a per-lane scalar.
//
// The three stages of a tile
//     A: S = K Q^T (MFMA)      B: P = 2^(S*c + b) (VALU)      C: O += V^T P (MFMA)
// run skewed -- iteration t issues A(t+1), B(t) and C(t-1), which are independent of one
// another -- in one instruction stream whose matrix instructions, LDS reads and copies sit at
// fixed places, with the vector work of B dealt out evenly between them, so the matrix pipe
// works while the vector pipe exponentiates.  What keeps the vector share small:
//   * B is one fused multiply-add (scale*log2(e) and the column's offset b = shift - reference
//     maximum; Q itself stays unscaled, so fp16-representable inputs enter the products exactly)
//     and one v_exp_f32 per score, and per pair of scores one v_cvt_pk_f16_f32 and one packed
//     fp16 add (the tile's share of the row sum: eight terms per half, added to the fp32 sum at
//     the end of the step).  (v_dot2_f32_f16 against packed ones would add a pair to an fp32 sum
//     directly, but it waits for the matrix instructions in flight: measured, 16 of them per
//     step cost more than everything else in B together.)
//   * The reference maximum is lazy: exponentials are computed optimistically; only if a tile's
//     fp16 partial sums show a weight above 2^12 (on a handful of early tiles; the reference sits
//     at 2^7) does a slow path move the reference, redo the tile's P and rescale O and l.
// K and V tiles are copied global->LDS by the load unit itself (no staging registers, two
// buffers each per wave, tile base in the scalar offset so the copies need no vector
// arithmetic) in an XOR-swizzled layout that both the 1 KB copy bursts and the operand reads
// hit conflict-free.  Each wave walks its tiles from the diagonal backwards, so the only tile
// that can need the causal mask is handled in the prologue and the steady state is mask-free.
//
// Few query columns on a long context (a model with few heads, or a short chunk): the launcher
// lets 2 to 16 workgroups share a token tile's KV rows (runs of four tiles go to the splits in
// turn); each writes its normalised output and log-sum-exp to the workspace and
// fa_prefill_combine_kernel merges them into `out`.
#include "fa_common.hpp"

// Stage marks: wall-clock stamps in the timeline build, nothing otherwise (fa_common.hpp).
#ifdef ORIN_FA_STAMPS
namespace orin_fa {
__device__ long long g_prefill_stamps[kStampWgs * kPrefillWaves * kStampSlots];
}
#define FA_STAMP(i) ORIN_FA_STAMP_STORE(orin_fa::g_prefill_stamps, orin_fa::kPrefillWaves, i)
#else
#define FA_STAMP(i)
#endif

// Cut-off builds (-DORIN_FA_PREFILL_PROBE=flags, liborin_fa_pprobe_<flags>.so; measurement aids whose RESULTS
// ARE WRONG by design): the kernel with parts taken out, so that bench.py's cut-off workload can say what
// each part costs.  In the main loop -- 1: no vector work (the softmax of the step), 2: no LDS operand
// reads, 4: no copies of the next tiles (7: matrix instructions only).  8: the kernel leaves behind the
// main loop (no last products, no merge, no store).  16: it leaves once the waves have handed their
// accumulators over (no barrier, no merge, no store).  32: every copy of the main loop fetches the tile at
// offset 0 (the same work for the load unit and LDS, but no trip beyond the nearest cache).  64: they fetch
// tile (t mod 32): half a megabyte per KV head, which stays in the L2 and does not fit the vector cache.  0 in the
// library proper, where none of this exists.
#ifndef ORIN_FA_PREFILL_PROBE
#define ORIN_FA_PREFILL_PROBE 0
#endif

namespace orin_fa {
namespace {
constexpr int kPProbe = ORIN_FA_PREFILL_PROBE;

typedef float f16v __attribute__((ext_vector_type(16)));

template <int D, int NCB>
struct PGeom {
    static constexpr int kSteps = D / 16;             // k-steps of A over head_dim
    static constexpr int kDBlk = D / 32;              // 32-wide output blocks over head_dim
    static constexpr int kCols = NCB * 32;            // query columns per workgroup
    static constexpr int kRowB = D * 2;               // bytes per K/V row in LDS (no padding; chunks are XOR-swizzled)
    static constexpr int kChunks = D / 8;             // 16-byte chunks per row
    static constexpr int kTileB = kTile * kRowB;      // one K or V tile
    static constexpr int kCopies = kTileB / 1024;     // one LDS copy instruction moves 64 lanes x 16 B
    static constexpr int kRowsPerCopy = 1024 / kRowB; // 4 (d=128) or 8 (d=64)
    static constexpr int kCopyVariants = 16 / kRowsPerCopy; // copies whose rows differ in what the swizzle looks at
    // The 16-byte chunks of a row sit in LDS in swizzled order: physical chunk p of row r holds
    // logical chunk p ^ swz(r).  LDS has 64 four-byte banks, i.e. 16 chunk-wide bank groups per
    // 256 bytes, and two access patterns must each spread over all 16: a K operand read
    // (ds_read_b128, 16 lanes at a time = 16 consecutive rows, one logical chunk) and a V
    // transposing read (ds_read_b64_tr_b16, 32 lanes at a time = 4 consecutive rows x 4
    // consecutive chunks).  d = 128 (a row fills all 16 groups): the row's two low bits go to
    // chunk bits 3:2, where they separate the 4 rows of a V read, and bits 3:2 of the row to chunk
    // bits 1:0, which makes 16 consecutive rows distinct.  d = 64 (two rows fill the groups, the
    // row's lowest bit picks the half): bit 1 of the row goes to chunk bit 2, bits 3:2 to bits
    // 1:0.  Either way swz(r + 16) = swz(r), and swz(r + 8) differs (second pointer set of the V reads).
    // (Measured with 4 waves reading: 25.0 instead of 32.1 clocks per K read, 16.3 instead of 32.0 per V read,
    // where an unconflicted 1 KB read takes 24.7.)
    __device__ static constexpr int swz(int r) {
        return D == 128 ? (((r & 3) << 2) | ((r >> 2) & 3)) : ((((r >> 1) & 1) << 2) | ((r >> 2) & 3));
    }
    static constexpr int kKOff = 0;                   // wave slice: K buffers 0/1, then V buffers 0/1
    static constexpr int kVOff = 2 * kTileB;
    // Merge buffer of a wave: the 16-byte pieces of its partial outputs, one 1 KB block per store
    // instruction of the hand-over.  Piece P = db*8 + 2*q + hh of column cb*32 + c32 (accumulator
    // registers 4q..4q+3 of block db in lane (c32, hh)) is chunk o_chunk(c32, hh, q) of block
    // (cb * kDBlk + db) * 4 + q.  A store instruction thus fills its own block with one chunk per
    // lane, in lane order up to an exchange of whole groups of lanes -- the form LDS takes at its
    // full write rate (53 counter ticks per instruction and wave with four waves storing, measured;
    // column-major rows, padded or permuted, take 53-64).  The exchange is there for the readers:
    // sixteen neighbouring threads of the merge, (4 columns) x (pieces hh, q & 1) or (2 columns) x
    // (hh, q), then fall on sixteen different chunk columns of the banks (19-22 ticks per load;
    // 48 with padded column-major rows, where they sat four to a bank).
    __device__ static int o_chunk(int c32, int hh, int q) {
        return (hh << 5) + (c32 ^ (hh << 3) ^ (NCB == 2 ? (q & 1) << 2 : q << 1));
    }
    __device__ static int o_byte(int col, int piece) { // where piece `piece` of column `col` sits in a wave's merge buffer
        const int hh = piece & 1, q = (piece & 7) >> 1, db = piece >> 3;
        return (((col >> 5) * kDBlk + db) * 4 + q) * 1024 + o_chunk(col & 31, hh, q) * 16;
    }
    static constexpr int kOStride = D; // floats of merge buffer per column
    static constexpr int kMergeB = kCols * kOStride * 4;
    static constexpr int kWaveB = (4 * kTileB > kMergeB) ? 4 * kTileB : kMergeB;
    static constexpr int kMlOff = kPrefillWaves * kWaveB;
    static constexpr int kQOff = kMlOff + kPrefillWaves * kCols * 2 * 4; // the query block as fp16, [column][head_dim]
    static constexpr int kQStride = D * 2 + 16;       // (padded against bank conflicts of the operand reads)
    static constexpr int kLdsB = kQOff + kCols * kQStride;
};

// ---------------------------------------------------------------------------------------------
// Instructions with the register file of each operand spelled out.  The kernel keeps its score
// accumulators in ordinary vector registers (the exponentials read them with no copy) and its
// output accumulators and the query operands in the accumulation-register file, and it fixes the
// place of every matrix instruction in the stream by hand -- neither of which the builtin forms allow.
// The price: the compiler knows nothing about the hazards of these blocks.
//   (1) Result latency: a non-matrix instruction reads a matrix result only a pipeline stage
//       (at least two later matrix instructions) after it was issued, or behind settle().
//   (2) A matrix instruction must not read an operand in the two cycles after a vector
//       instruction wrote it.  The forms with the _n suffix start with the two wait states and
//       are used wherever compiler-generated vector code may sit right in front of the block
//       (prologue, drain); the main loop uses the bare forms, where every operand was written
//       a long way back (LDS reads, the previous iteration's conversions, loop invariants).
// ---------------------------------------------------------------------------------------------
__device__ __forceinline__ void mfma_s_n(f16v& acc, h8 a_op, h8 b_acc) {
    asm volatile("s_nop 1\n\tv_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+v"(acc) : "v"(a_op), "a"(b_acc));
}
__device__ __forceinline__ void mfma_s_zero_n(f16v& acc, h8 a_op, h8 b_acc) { // acc = A B
    // early clobber: the destination must not share registers with an operand that dies here
    asm volatile("s_nop 1\n\tv_mfma_f32_32x32x16_f16 %0, %1, %2, 0" : "=&v"(acc) : "v"(a_op), "a"(b_acc));
}
__device__ __forceinline__ void mfma_o_n(f16v& acc, h8 a_op, h8 b_op) {
    asm volatile("s_nop 1\n\tv_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+a"(acc) : "v"(a_op), "v"(b_op));
}
__device__ __forceinline__ void mfma_o_zero_n(f16v& acc, h8 a_op, h8 b_op) {
    asm volatile("s_nop 1\n\tv_mfma_f32_32x32x16_f16 %0, %1, %2, 0" : "=&a"(acc) : "v"(a_op), "v"(b_op));
}
__device__ __forceinline__ void mfma_s(f16v& acc, h8 a_op, h8 b_acc) {
    asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+v"(acc) : "v"(a_op), "a"(b_acc));
}
__device__ __forceinline__ void mfma_s_zero(f16v& acc, h8 a_op, h8 b_acc) { // acc = A B
    asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, 0" : "=&v"(acc) : "v"(a_op), "a"(b_acc));
}
__device__ __forceinline__ void mfma_o(f16v& acc, h8 a_op, h8 b_op) {
    asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+a"(acc) : "v"(a_op), "v"(b_op));
}
// Lets the matrix pipe drain (48 wait states, more than any 32x32x16 result needs) and stops the
// compiler from moving anything across.
__device__ __forceinline__ void settle() {
    __builtin_amdgcn_sched_barrier(0);
    asm volatile("s_nop 15\n\ts_nop 15\n\ts_nop 15" ::: "memory");
    __builtin_amdgcn_sched_barrier(0);
}
// Empty blocks that tie a 16-register value to a register file at a point of the program: the
// compiler can neither move its reads of the value above the block nor hand out the registers
// before it (keep_v).
__device__ __forceinline__ void pin_v(f16v& x) { asm volatile("" : "+v"(x)); }
__device__ __forceinline__ void pin_a(f16v& x) { asm volatile("" : "+a"(x)); }
__device__ __forceinline__ void keep_v(const f16v& x) { asm volatile("" : : "v"(x)); }
// The two lanes that hold a column's rows are l and l ^ 32: maximum / sum over the pair.
__device__ __forceinline__ float pair_max(float v) {
    const u32x2 s = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    return fmaxf(__uint_as_float(s.x), __uint_as_float(s.y));
}
__device__ __forceinline__ float pair_sum(float v) {
    const u32x2 s = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    return __uint_as_float(s.x) + __uint_as_float(s.y);
}

// Buffer descriptor words for the global->LDS copies below: base address, stride 0, byte
// count, raw 32-bit format.  Vector offsets at or past the byte count are not fetched.
__device__ __forceinline__ i32x4 make_desc(const void* base, unsigned bytes) {
    const unsigned long long b = reinterpret_cast<unsigned long long>(base);
    // (uniform by construction; saying so keeps the words in scalar registers, where the copies need them)
    return i32x4{__builtin_amdgcn_readfirstlane((int)(unsigned)b), __builtin_amdgcn_readfirstlane((int)((unsigned)(b >> 32) & 0xffffu)),
                 __builtin_amdgcn_readfirstlane((int)bytes), 0x00020000};
}

// Four 1 KB global->LDS copies (buffer_load ... lds): lane l of copy i fetches 16 bytes at
// global offset soff + off_i + i*1024 and the load unit writes them to LDS byte lds_base +
// i*1024 + l*16 (the immediate offset advances both addresses).  soff is a scalar and is not
// part of the range check.  The copies count on the vector-memory counter and complete in
// issue order; callers wait with s_waitcnt vmcnt(n).  One asm block, so that M0 (the LDS base)
// cannot change between the copies.
__device__ __forceinline__ void lds_copy_4k(i32x4 desc, unsigned lds_base, int off0, int off1, int off2, int off3, int soff) {
    asm volatile(
        "s_mov_b32 m0, %0\n\t"
        "buffer_load_dwordx4 %1, %5, %6 offen lds\n\t"
        "buffer_load_dwordx4 %2, %5, %6 offen offset:1024 lds\n\t"
        "buffer_load_dwordx4 %3, %5, %6 offen offset:2048 lds\n\t"
        "buffer_load_dwordx4 %4, %5, %6 offen offset:3072 lds"
        :
        : "s"(lds_base), "v"(off0), "v"(off1), "v"(off2), "v"(off3), "s"(desc), "s"(soff)
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
// that the vector-memory issue queue never backs up.  The LDS base is written to M0 inside the
// same block as the copy that uses it (as lds_copy_4k does), so nothing the compiler may put
// between two copies can change the destination.
template <int IMM>
__device__ __forceinline__ void lds_copy_1k(i32x4 desc, unsigned lds_base, int off, int soff) {
    asm volatile("s_mov_b32 m0, %4\n\tbuffer_load_dwordx4 %0, %1, %2 offen offset:%3 lds"
                 :
                 : "v"(off), "s"(desc), "s"(soff), "n"(IMM), "s"(lds_base)
                 : "memory", "m0");
}

// The vector instructions of stage B for one 32x32 score block (16 scores per lane), in issue
// order.  Pair p = scores (2p, 2p+1).  Kinds: 0 multiply-add (the exponent), 1 exponential,
// 2 conversion of a pair to packed fp16, 3 addition of the converted pair to the tile's packed
// partial row sums.  The four kinds run as a software pipeline one pair apart, so that nothing
// waits for the result of the instruction right before it.
struct ItemTable {
    int kind[48];
    int arg[48];
};
constexpr ItemTable make_items() {
    ItemTable t{};
    int n = 0;
    for (int p = 0; p < 11; ++p) {
        if (p < 8) {
            t.kind[n] = 0; t.arg[n++] = 2 * p;
            t.kind[n] = 0; t.arg[n++] = 2 * p + 1;
        }
        if (p >= 1 && p <= 8) {
            t.kind[n] = 1; t.arg[n++] = 2 * p - 2;
            t.kind[n] = 1; t.arg[n++] = 2 * p - 1;
        }
        if (p >= 2 && p <= 9) {
            t.kind[n] = 2; t.arg[n++] = p - 2;
        }
        if (p >= 3) {
            t.kind[n] = 3; t.arg[n++] = p - 3;
        }
    }
    return t;
}
constexpr ItemTable kItemsOfBlock = make_items();
constexpr int kItemsPerBlock = 48;

template <int D, int NCB>
__global__ __launch_bounds__(kPrefillWaves * 64) void fa_prefill_kernel(
    // What the prologue's loads need comes first, as scalars: the leading kernel arguments are
    // handed to a wave in registers when it starts (kernel-argument preload), so the query block
    // and the first tiles are requested at once, not behind a trip to memory for their addresses.
    // packed: heads_per_group | kv_split_shift << 4 | tq << 8 | tq_magic << 16.
    const float* q_in, const uint16_t* kc, const uint16_t* vc, const int n_ctx,
    const int n_past, const int batch, const int n_head, const int r_heads, const int n_ttiles, const unsigned packed,
    const float qsign, const FaArgs a) {
    using G = PGeom<D, NCB>;
    constexpr int kWaves = kPrefillWaves;
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    FA_STAMP(0);
    const int heads_per_group = packed & 15, kv_split_shift = (packed >> 4) & 15, tq = (packed >> 8) & 255;
    const int tq_magic = packed >> 16;
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6); // uniform: tile indices live in scalar registers
    const int c32 = lane & 31; // MFMA column (query column of a block) / row (KV row or head_dim index) of the lane
    const int hh = lane >> 5;  // lane-half: 8-wide k slice of an operand, rows 8q + 4*hh + 0..3 of an accumulator

    const int kvh = __builtin_amdgcn_readfirstlane(blockIdx.x); // (the KV head varies fastest in dispatch order)
    // blockIdx.y = head group * splits + KV split (splits: a power of two, 1 unless the launcher found the grid too small)
    const int hg = __builtin_amdgcn_readfirstlane(blockIdx.y) >> kv_split_shift;
    const int split = __builtin_amdgcn_readfirstlane(blockIdx.y) & ((1 << kv_split_shift) - 1);
    const int t0 = (n_ttiles - 1 - __builtin_amdgcn_readfirstlane(blockIdx.z)) * tq; // longest rows first
    const int head_lo = hg * heads_per_group;
    const int tok_hi = (t0 + tq < batch) ? t0 + tq : batch;
    const int kv_end = n_past + tok_hi;   // the workgroup's columns see rows [0, kv_end) at most
    const int full_end = n_past + t0 + 1; // rows below this are visible to every column
    const int n_tiles = (kv_end + kTile - 1) / kTile;
    // Wave w owns tiles w, w+4, ...  Step 0 visits the highest (the only one that can need the
    // causal mask) and the steps after it walk the rest downwards.  In the 32-column shape the
    // walk starts at a tile that differs from workgroup to workgroup and wraps around: there a
    // step is about as long as a copy takes from memory, and workgroups that share a KV head on
    // an XCD and ask for the same tile at the same moment all wait for the same trip to memory,
    // on every step; staggered, one of them takes the miss and the others find the tile in L2
    // (measured on Qwen2.5-1.5B with cold caches: 27.7 us instead of 32.6).  The 64-column shape
    // keeps the common order: its steps are long enough to cover the trip, and it measured 2-4 %
    // slower with any stagger.  (The order of the tiles does not matter to the result.)
    // Steps past the end map to negative tiles, for which the copies fetch a tile nobody reads.
    // With KV splits, split s of S takes the tiles w + 4*(s + S*i): runs of four tiles (one per
    // wave) go to the splits in turn, so the tiles at the diagonal, the ones that can need the
    // mask, are still each the highest tile of the wave that owns them.
    const int t_base = wave + kWaves * split;   // this wave's lowest tile
    const int t_shift = 2 + kv_split_shift;   // log2 of the distance between its tiles
    static_assert(kWaves == 4, "tile distance as a shift");
    const int n_mine = n_tiles > t_base ? ((n_tiles - 1 - t_base) >> t_shift) + 1 : 0;
    const int n_rest = n_mine - 1;
    const int rot = (NCB == 1 && n_rest > 1)
                        ? (int)((((unsigned)__builtin_amdgcn_readfirstlane(blockIdx.z) * 0x9E3779B1u) >> 8) % (unsigned)n_rest) : 0;
    auto tile_of = [&](int j) {
        if (j == 0) return t_base + (n_rest << t_shift);
        if (j > n_rest) return -1;
        int k = j - 1 + rot;
        k = k >= n_rest ? k - n_rest : k;
        return t_base + ((n_rest - 1 - k) << t_shift);
    };
    // column c of the block -> (token, head of the group); columns past the group's heads are padding
    auto col_valid = [&](int c, int& tok, int& hl) {
        const int hq = (c * tq_magic) >> 16; // = c / tq for the c < 64 that occur (tq_magic = 65536 / tq + 1)
        tok = t0 + c - hq * tq;
        hl = head_lo + hq;
        return hq < heads_per_group && hl < r_heads && tok < batch;
    };

    unsigned char* const ws = smem + wave * G::kWaveB; // this wave's LDS slice
    const unsigned ws_addr = __builtin_amdgcn_readfirstlane(
        (unsigned)(size_t)(__attribute__((address_space(3))) unsigned char*)ws);
    const i32x4 kdesc = make_desc(kc + (size_t)kvh * n_ctx * D, (unsigned)kv_end * D * 2);
    const i32x4 vdesc = make_desc(vc + (size_t)kvh * n_ctx * D, (unsigned)kv_end * D * 2);

    // ---- per-lane offsets ----
    // Copy: lane l of copy i lands at LDS byte i*1024 + l*16 = row i*R + l/C, physical chunk l%C,
    // and physical chunk p of row r holds logical chunk p ^ swz(r); copy i is of variant i % kVar.
    constexpr int kVar = G::kCopyVariants;
    int g_off[kVar];
    {
        const int r_in = lane / G::kChunks, pc = lane % G::kChunks;
#pragma unroll
        for (int v = 0; v < kVar; ++v) {
            const int sw = G::swz(v * G::kRowsPerCopy + r_in);
            g_off[v] = r_in * G::kRowB + ((pc ^ sw) & (G::kChunks - 1)) * 16;
        }
    }
    // K operand read: lane (c32, hh) takes row c32, logical chunk ks*2 + hh.  The pointers carry
    // every per-lane term; the buffer parity is an immediate offset.
    const unsigned char* kp[G::kSteps];
#pragma unroll
    for (int ks = 0; ks < G::kSteps; ++ks) kp[ks] = ws + G::kKOff + c32 * G::kRowB + (((ks * 2 + hh) ^ G::swz(c32)) * 16);
    // V transposing read, per 16-lane group (lane i of the group): addresses row R + i/4, 8-byte
    // column (d0/4 + i%4) and receives rows R..R+3 at head_dim index d0 + i, where d0 = db*32 +
    // 16 * (lane/16 % 2) and R = 16*kh + 4*hh (+8 for the second half of the operand): the
    // operand's k index (hh, j) is KV row 16*kh + 8*(j/4) + 4*hh + j%4, the row that score
    // register 8*kh + j of lane-half hh belongs to.
    // Rows R + 8 are swizzled differently from rows R (rows R + 16 alike): two pointer sets.
    const unsigned char* vp[2][G::kDBlk];
    {
        const int i16 = lane & 15, g2 = (lane >> 4) & 1;
        const int r0 = 4 * hh + (i16 >> 2);
#pragma unroll
        for (int u = 0; u < 2; ++u)
#pragma unroll
            for (int db = 0; db < G::kDBlk; ++db)
                vp[u][db] = ws + G::kVOff + (r0 + 8 * u) * G::kRowB +
                            (((db * 4 + g2 * 2 + ((i16 & 3) >> 1)) ^ G::swz(r0 + 8 * u)) * 16) + (i16 & 1) * 8;
    }

    // Prologue copies: the whole offset is in the (range-checked) vector operand, so rows at or
    // past kv_end of the diagonal tile, and tiles below zero, are not fetched.
    auto copy_checked = [&](const i32x4& desc, unsigned lds_dst, int tile) {
        const int base = tile * G::kTileB;
        lds_copy_4k(desc, lds_dst, base + g_off[0], base + g_off[1 % kVar], base + g_off[2 % kVar], base + g_off[3 % kVar], 0);
        if (G::kCopies > 4)
            lds_copy_4k(desc, lds_dst + 4096, base + 4096 + g_off[0], base + 4096 + g_off[1 % kVar], base + 4096 + g_off[2 % kVar],
                        base + 4096 + g_off[3 % kVar], 0);
    };
    // Main-loop copies: every tile they name is either wholly inside the visible range, and its
    // base travels as the scalar offset, or below zero (steps past the wave's last tile), and then
    // tile 0 is copied instead, into a buffer nobody reads any more.
    auto tile_soff = [&](int tile) {
        if constexpr ((kPProbe & 32) != 0) return 0;
        if constexpr ((kPProbe & 64) != 0) return __builtin_amdgcn_readfirstlane(((tile > 0 ? tile : 0) & 31) * G::kTileB);
        return __builtin_amdgcn_readfirstlane((tile > 0 ? tile : 0) * G::kTileB);
    };
    auto copy_one = [&](auto ic, const i32x4& d, unsigned lds_dst, int soff) { // copy number i (of kCopies) of such a tile
        constexpr int i = decltype(ic)::value;
        constexpr int half = i / 4, sub = i % 4;
        lds_copy_1k<sub * 1024>(d, lds_dst + half * 4096, g_off[sub % kVar], soff + half * 4096);
    };
    auto k_buf = [&](int par) { return ws_addr + G::kKOff + par * G::kTileB; };
    auto v_buf = [&](int par) { return ws_addr + G::kVOff + par * G::kTileB; };

    // ---- state ----
    h8 q[NCB][G::kSteps];   // B operands of A: the query columns, fp16
    float nb[NCB];          // each column's exponent offset: shift - reference maximum * c (log2 units)
    float lsum[NCB][2];     // this lane's share (16 of a tile's 32 rows) of the column's row sum, as two partial sums
    f16v o[NCB][G::kDBlk];  // O^T accumulators (accumulation registers)
    f16v s[2][NCB];         // scores: [parity][column block]
    u32x4 pw[2][NCB][2];    // P as packed fp16: [parity][column block][k-step of C]

    // ---- prologue loads, most urgent first: the query block, then the first K tile; the rest of
    // the first two tiles follows once the queries are on their way into LDS.  All of them are
    // issued by hand and counted on the vector-memory counter, so that no wait has to sit out
    // the loads behind the one it needs.
    // The query block is loaded once per workgroup: wave w takes a quarter of the columns with
    // coalesced 16-byte loads (a column is D/4 lanes wide), converts to fp16 and leaves it in LDS;
    // after the barrier every wave picks up its B operands from there. ----
    constexpr int kColsPerLoad = 256 / D;                 // columns one load instruction covers
    constexpr int kQLoads = G::kCols / 4 / kColsPerLoad;  // load instructions per wave
    u32x4 qraw[kQLoads];
    float qmul[kQLoads];
    int qcol[kQLoads];
    {
        const i32x4 qdesc = make_desc(q_in, (unsigned)batch * n_head * D * 4);
        static_for<0, kQLoads>([&](auto jc) {
            constexpr int j = decltype(jc)::value;
            const int c = wave * (G::kCols / 4) + j * kColsPerLoad + lane / (D / 4);
            int tok, hl;
            const bool valid = col_valid(c, tok, hl);
            qcol[j] = c;
            qmul[j] = valid ? qsign : 0.0f; // c > 0 multiplies the scores; the sign of the scale goes here
            const int q_off = valid ? ((tok * n_head + kvh * r_heads + hl) * D + (lane % (D / 4)) * 4) * 4 : 0;
            reg_load16<0>(qraw[j], qdesc, q_off, 0);
        });
    }
    if (n_mine > 0) copy_checked(kdesc, k_buf(0), tile_of(0));
    FA_STAMP(9);
    // O = 0: a matrix instruction with a zero addend writes the accumulation registers without
    // touching memory.
    {
        h8 zero;
#pragma unroll
        for (int e = 0; e < 8; ++e) zero[e] = (_Float16)0.0f;
        asm volatile("" : "+v"(zero));
#pragma unroll
        for (int cb = 0; cb < NCB; ++cb) {
            lsum[cb][0] = lsum[cb][1] = 0.0f;
            nb[cb] = 0.0f;
#pragma unroll
            for (int db = 0; db < G::kDBlk; ++db) mfma_o_zero_n(o[cb][db], zero, zero);
        }
    }
    FA_STAMP(11);
    if (n_mine > 0) {
        // V buffer 0 receives the diagonal tile, whose rows at or past kv_end are not fetched:
        // clear it first, so that no stale bit pattern meets a zero weight (0 * NaN is not 0).
        // The buffer is this wave's own: once the wave's LDS writes have completed, the copy
        // into it may go out -- together with K(1), ahead of the wait for the queries, so that
        // the second tile's trip to memory runs beside the queries' instead of after it.
#pragma unroll
        for (int i = 0; i < G::kCopies; ++i)
            *reinterpret_cast<u32x4*>(ws + G::kVOff + i * 1024 + lane * 16) = u32x4{0u, 0u, 0u, 0u};
        __builtin_amdgcn_s_waitcnt(0xC07F); // lgkmcnt(0)
        FA_STAMP(12);
        copy_checked(vdesc, v_buf(0), tile_of(0));
        FA_STAMP(13);
        copy_checked(kdesc, k_buf(1), tile_of(1));
    }
    // The arguments that did not arrive in registers are fetched here, behind the prologue's loads
    // and beside their trip to memory: left alone, the compiler fetches each where it is first
    // used, one wait behind the other after the first products.
    {
        const void *p0 = a.out, *p1 = a.part_o, *p2 = a.part_ml;
        asm volatile("" ::"s"(p0), "s"(p1), "s"(p2), "s"(a.c));
    }
    FA_STAMP(10);
    // ---- query block -> LDS (fp16) ----
    constexpr int kInFlight = 3 * G::kCopies; // K(0), V(0), K(1)
    if (n_mine > 0) __builtin_amdgcn_s_waitcnt(0x0F70 | (kInFlight & 15) | ((kInFlight >> 4) << 14)); // vmcnt: the queries are in, the copies may be in flight
    else __builtin_amdgcn_s_waitcnt(0x0F70);
#pragma unroll
    for (int j = 0; j < kQLoads; ++j) {
        h4 hv;
#pragma unroll
        for (int e = 0; e < 4; ++e) hv[e] = (_Float16)(__uint_as_float(qraw[j][e]) * qmul[j]);
        *reinterpret_cast<h4*>(smem + G::kQOff + qcol[j] * G::kQStride + (lane % (D / 4)) * 8) = hv;
    }
    __syncthreads();
    int limit[NCB];
#pragma unroll
    for (int cb = 0; cb < NCB; ++cb) {
        const int c = cb * 32 + c32;
        int tok, hl;
        limit[cb] = col_valid(c, tok, hl) ? n_past + tok + 1 : 0x7fffffff;
        h8 hv[G::kSteps]; // (all reads of a block first: a read per parking block would wait out its latency alone)
#pragma unroll
        for (int ks = 0; ks < G::kSteps; ++ks)
            hv[ks] = *reinterpret_cast<const h8*>(smem + G::kQOff + c * G::kQStride + (ks * 16 + hh * 8) * 2);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int ks = 0; ks < G::kSteps; ++ks)
            asm volatile("" : "=a"(q[cb][ks]) : "0"(hv[ks])); // parked in the accumulation-register file for good
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

    // ---- the wave's hand-over to the merge of the four waves through LDS ----
    // (m, l) per wave and column, m = the reference in log2 units (the common shift cancels);
    // a wave that saw no visible row of a column has l = 0 and is given m = -inf (weight 0).
    float* const ml = reinterpret_cast<float*>(smem + G::kMlOff);
    auto write_ml = [&]() {
#pragma unroll
        for (int cb = 0; cb < NCB; ++cb) {
            const float l_tot = pair_sum(lsum[cb][0] + lsum[cb][1]);
            if (hh == 0) {
                ml[(wave * G::kCols + cb * 32 + c32) * 2 + 0] = l_tot > 0.0f ? -nb[cb] : -INFINITY;
                ml[(wave * G::kCols + cb * 32 + c32) * 2 + 1] = l_tot;
            }
        }
    };
    // O^T -> merge buffer (layout: PGeom::o_byte).  Accumulator a = cb * kDBlk + db; half h of it is
    // its pieces q = 2h and 2h + 1.  The block is an immediate offset; the chunk takes one of the
    // two (NCB = 2) or four per-lane values below.
    constexpr int kAccs = NCB * G::kDBlk;
    unsigned char* o_lane[4];
#pragma unroll
    for (int qd = 0; qd < 4; ++qd) o_lane[qd] = ws + G::o_chunk(c32, hh, qd) * 16;
    auto write_o_half = [&](auto ac, auto hc, auto pinc) {
        constexpr int acc = decltype(ac)::value, half = decltype(hc)::value;
        constexpr int cb = acc / G::kDBlk, db = acc % G::kDBlk;
        if constexpr (decltype(pinc)::value) pin_a(o[cb][db]); // (its reads stay behind this point of the instruction stream)
#pragma unroll
        for (int qd = 2 * half; qd < 2 * half + 2; ++qd)
            *reinterpret_cast<f4*>(o_lane[qd] + ((cb * G::kDBlk + db) * 4 + qd) * 1024) =
                f4{o[cb][db][4 * qd], o[cb][db][4 * qd + 1], o[cb][db][4 * qd + 2], o[cb][db][4 * qd + 3]};
    };

    if (n_mine > 0) {
        const int R = n_mine - 1; // steps after step 0
        // Prologue form of A: S[spar] = K[kpar] Q^T with a zero addend, operands read up front.
        auto stage_a0 = [&](auto kpar, auto spar) {
            constexpr int KP = decltype(kpar)::value, SP = decltype(spar)::value;
            h8 ka[G::kSteps];
#pragma unroll
            for (int ks = 0; ks < G::kSteps; ++ks) ka[ks] = *reinterpret_cast<const h8*>(kp[ks] + KP * G::kTileB);
#pragma unroll
            for (int ks = 0; ks < G::kSteps; ++ks)
#pragma unroll
                for (int cb = 0; cb < NCB; ++cb) {
                    if (ks == 0) mfma_s_zero_n(s[SP][cb], ka[ks], q[cb][ks]);
                    else mfma_s_n(s[SP][cb], ka[ks], q[cb][ks]);
                }
        };
        // Copy issue order: K0 V0 K1 | K2 V1 (step 0) | K3 V2 (step 1) | K4 V3 (step 2) | ...
        // (within a step, K goes out over the first half of the tickets and V over the second)
        // ---- step 0: the diagonal tile, the only one that can need the causal mask ----
        wait_copies(IntC<2 * kC>{});        // K0 landed (V0 K1 may be in flight)
        stage_a0(IntC<0>{}, IntC<0>{});     // S(0)
        __builtin_amdgcn_s_waitcnt(0xC07F); // its LDS reads have returned: K buffer 0 is free
        wait_copies(IntC<0>{});             // K1 and V0 landed
        // S(1), the scan of S(0) for each column's maximum and the copies of K(2) run as one
        // stream: a matrix instruction, a share of the scan, a copy.  (Sixteen copies issued in
        // one burst hold the wave for as long as the load unit takes to accept them, half a
        // microsecond with four waves at it; one at a time between other work they cost nothing.
        // When the wave has no tile 1 the products are of whatever K buffer 1 holds, and nobody
        // reads them.)
        const int ksoff0 = tile_soff(tile_of(2)), vsoff0 = tile_soff(tile_of(1));
        float v0s[NCB][16];
        float mxp[NCB][4];
        {
            h8 ka[G::kSteps];
#pragma unroll
            for (int ks = 0; ks < G::kSteps; ++ks) ka[ks] = *reinterpret_cast<const h8*>(kp[ks] + G::kTileB);
            __builtin_amdgcn_s_waitcnt(0xC07F);
            settle(); // S(0) is out of the matrix pipe
            const int row0 = tile_of(0) * kTile + 4 * hh;
            const bool masked = tile_of(0) * kTile + kTile > full_end;
#pragma unroll
            for (int cb = 0; cb < NCB; ++cb) {
                pin_v(s[0][cb]); // (the reads below stay behind the settled pipe)
                mxp[cb][0] = mxp[cb][1] = mxp[cb][2] = mxp[cb][3] = -INFINITY; // four chains instead of one long one
            }
            constexpr int kSlots = G::kSteps * NCB;     // one matrix instruction each
            constexpr int kScan = 16 * NCB / kSlots;    // scores scanned per slot
            static_assert(kScan * kSlots == 16 * NCB && kC % (kSlots / NCB) == 0, "shares");
            static_for<0, kSlots>([&](auto ic) {
                constexpr int i = decltype(ic)::value;
                constexpr int ks = i / NCB, m = i % NCB;
                if constexpr (ks == 0) mfma_s_zero_n(s[1][m], ka[ks], q[m][ks]);
                else mfma_s_n(s[1][m], ka[ks], q[m][ks]);
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int u = 0; u < kScan; ++u) {
                    constexpr int cb = (i * kScan) / 16;
                    const int r = (i * kScan) % 16 + u;
                    float x = s[0][cb][r];
                    if (masked && row0 + 8 * (r / 4) + (r % 4) >= limit[cb]) x = -INFINITY;
                    v0s[cb][r] = x;
                    mxp[cb][r % 4] = fmaxf(mxp[cb][r % 4], x);
                }
                __builtin_amdgcn_sched_barrier(0);
                if constexpr (m == NCB - 1) {
                    constexpr int per = kC / G::kSteps; // copies per k-step
                    static_for<0, per>([&](auto jc) { copy_one(IntC<ks * per + decltype(jc)::value>{}, kdesc, k_buf(0), ksoff0); });
                }
            });
        }
        settle();
        FA_STAMP(2);
        // Reference maximum of each column: over its visible scores of tile 0 and, when there is
        // one, tile 1 (every row of which is visible to every column).  A column with no visible
        // row in this wave keeps weight zero whatever the reference.  The copies of V(1) go out
        // between the pieces of this.
        {
            constexpr int kPieces = 2 * NCB;
            static_assert(kC % kPieces == 0, "copies per piece");
#pragma unroll
            for (int cb = 0; cb < NCB; ++cb) {
                if (R > 0) {
                    pin_v(s[1][cb]);
#pragma unroll
                    for (int r = 0; r < 16; ++r) mxp[cb][r % 4] = fmaxf(mxp[cb][r % 4], s[1][cb][r]);
                }
                const float mx = pair_max(fmaxf(fmaxf(mxp[cb][0], mxp[cb][1]), fmaxf(mxp[cb][2], mxp[cb][3])));
                nb[cb] = kPShift - (mx == -INFINITY ? 0.0f : mx) * a.c;
            }
            static_for<0, kPieces>([&](auto pc) {
                constexpr int piece = decltype(pc)::value, cb = piece / 2, kh = piece % 2;
                __builtin_amdgcn_sched_barrier(0);
                static_for<0, kC / kPieces>([&](auto jc) {
                    copy_one(IntC<piece * (kC / kPieces) + decltype(jc)::value>{}, vdesc, v_buf(1), vsoff0);
                });
                __builtin_amdgcn_sched_barrier(0);
                float sump[4] = {0.0f, 0.0f, 0.0f, 0.0f};
                h8 ph;
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    ph[j] = (_Float16)fast_exp2(__builtin_fmaf(v0s[cb][kh * 8 + j], a.c, nb[cb]));
                    sump[j % 4] += (float)ph[j];
                }
                pw[0][cb][kh] = __builtin_bit_cast(u32x4, ph);
                const float sum = (sump[0] + sump[1]) + (sump[2] + sump[3]);
                if constexpr (kh == 0) lsum[cb][0] = sum;
                else lsum[cb][0] += sum;
                lsum[cb][1] = 0.0f;
            });
        }
        settle(); // (the vector writes of P are well clear of the next matrix instruction)
        FA_STAMP(3);

        // ---- steps t >= 1: A(t+1), B(t) and C(t-1) in one instruction stream.  The matrix
        // instructions are cut into groups of NCB that share an LDS operand -- C: one 32-wide block
        // of V^T for one half of the tile's rows, A: one k-step of K -- with all of C first: the V
        // buffer C reads is then free for the copy of V(t+1) from the middle of the step, and
        // both copies (K(t+2) over the first half, V(t+1) over the second) have more than a step
        // to land, so neither wait in the step ever stalls.  The 48 vector instructions per
        // column block of B are dealt out evenly between the matrix instructions.  Operands are
        // read from LDS kAhead groups ahead of their use, across the end of the step too: the
        // first groups' operands arrive in `carry`, read during the previous step. ----
        constexpr int kCG = 2 * G::kDBlk;             // groups of C
        constexpr int kGroups = kCG + G::kSteps;      // groups of matrix instructions per step
        constexpr int kTickets = kGroups * NCB;       // matrix instructions per step
        constexpr int kHalf = kCG * NCB;              // tickets of C
        constexpr int kItems = kItemsPerBlock * NCB;  // vector instructions of B per step
        constexpr int kSkip = NCB == 1 ? 1 : 0;       // tickets without vector work at the start of a step: S(t) of
                                                      // column block 0 is two matrix instructions old when it is read
        constexpr int kAhead = 4;
        static_assert(kAhead <= kCG && kAhead <= G::kSteps, "the reads carried over a step boundary are reads of V");
        static_assert(kAhead % 2 == 0 && kCG % 2 == 0 && kGroups % 2 == 0, "operands are read in pairs of groups");
        static_assert(kHalf == kC * NCB && kTickets - kHalf == kC * NCB, "one copy every NCB tickets");
        constexpr float kBound = 12.0f;               // a column whose largest exponent is above this is moved ...
        constexpr float kBoundP = 32768.0f;           // ... once a half-sum (eight weights) of the tile reaches this: then some
                                                      // weight is above 2^12; below, no half-sum can leave the fp16 range
        float c = a.c;
        asm volatile("" : "+v"(c)); // a vector register for the whole loop, not a move per step
        h8 carry[kAhead];
        // The V operand of C group g (block g % kDBlk of head_dim, half g / kDBlk of the tile's rows).
        auto read_v = [&](auto gc, int par_off) {
            constexpr int g = decltype(gc)::value;
            constexpr int db = g % G::kDBlk, kh = g / G::kDBlk;
            const h4 v0 = lds_read_tr(vp[0][db] + par_off + kh * 16 * G::kRowB);
            const h4 v1 = lds_read_tr(vp[1][db] + par_off + kh * 16 * G::kRowB);
            return __builtin_shufflevector(v0, v1, 0, 1, 2, 3, 4, 5, 6, 7);
        };
        static_for<0, kAhead>([&](auto gc) { carry[kAhead - 1 - decltype(gc)::value] = read_v(IntC<kAhead - 1 - decltype(gc)::value>{}, 0); }); // for step 1: V(0)
        // (The last step has no tile t+1: its A stage multiplies whatever the K buffer holds and
        // nobody reads the result -- cheaper than a second copy of the loop body without it.)
        auto body = [&](auto tpar, int t) {
            constexpr int TP = decltype(tpar)::value; // t & 1
            // K(t+2) goes to the buffer A(t) read, V(t+1) to the buffer C(t-1) reads in the first half of this step.
            const int ksoff = tile_soff(tile_of(t + 2));
            const int vsoff = tile_soff(tile_of(t + 1));
            h8 gop[kGroups];
            static_for<0, kAhead>([&](auto gc) { gop[decltype(gc)::value] = carry[decltype(gc)::value]; });
            // Issue order of the copies is ... K(t+1) V(t) | K(t+2) V(t+1): a wait that leaves the
            // copies issued since outstanding guarantees the older tile.  T = the ticket about to issue.
            // Reads are issued for two groups at a time, the later group first: LDS returns data
            // in order, so the wait for the earlier group's operand covers the later group's too.
            auto read_group = [&](auto gc) {
                constexpr int g = decltype(gc)::value;
                if constexpr ((kPProbe & 2) != 0) { // (cut-off build: whatever the registers hold)
                    if constexpr (g < kGroups) gop[g] = carry[g % kAhead];
                }
                else if constexpr (g < kCG) gop[g] = read_v(gc, (TP ^ 1) * G::kTileB);
                else if constexpr (g < kGroups) gop[g] = *reinterpret_cast<const h8*>(kp[g - kCG] + (TP ^ 1) * G::kTileB);
                else carry[g - kGroups] = read_v(IntC<g - kGroups>{}, TP * G::kTileB);     // for C(t) of the next step
            };
            auto issue_reads = [&](auto gc, auto tc) { // groups g + 1 and g
                constexpr int g = decltype(gc)::value, T = decltype(tc)::value;
                constexpr int k_issued = T / NCB < kC ? T / NCB : kC;
                constexpr int v_issued = T < kHalf ? 0 : ((T - kHalf) / NCB < kC ? (T - kHalf) / NCB : kC);
                __builtin_amdgcn_sched_barrier(0);
                if constexpr (g == kCG) wait_copies(IntC<kC + k_issued>{});           // K(t+1) landed
                if constexpr (g == kGroups) wait_copies(IntC<k_issued + v_issued>{}); // V(t) landed
                read_group(IntC<g + 1>{});
                read_group(gc);
                __builtin_amdgcn_sched_barrier(0);
            };
            float pe[NCB][16];
            typedef _Float16 h2v __attribute__((ext_vector_type(2)));
            h2v hp[NCB][8];      // the pairs of weights, as converted
            h2v hsum[NCB];       // this tile's share of the row sums, two fp16 partial sums per column block
#pragma unroll
            for (int cb = 0; cb < NCB; ++cb) hsum[cb] = h2v{(_Float16)0.0f, (_Float16)0.0f};
            float l_before[NCB]; // the row sums without this tile, for the slow path
#pragma unroll
            for (int cb = 0; cb < NCB; ++cb) l_before[cb] = lsum[cb][0] + lsum[cb][1];
            // Vector instruction j of B(t) (see ItemTable).
            auto item = [&](auto jc) {
                constexpr int j = decltype(jc)::value;
                constexpr int cb = j / kItemsPerBlock, r = j % kItemsPerBlock;
                constexpr int kind = kItemsOfBlock.kind[r], x = kItemsOfBlock.arg[r];
                if constexpr (kind == 0) {
                    pe[cb][x] = __builtin_fmaf(s[TP][cb][x], c, nb[cb]);
                } else if constexpr (kind == 1) {
                    pe[cb][x] = __builtin_amdgcn_exp2f(pe[cb][x]);
                } else if constexpr (kind == 2) {
                    typedef float f2 __attribute__((ext_vector_type(2)));
                    typedef _Float16 h2 __attribute__((ext_vector_type(2)));
                    hp[cb][x] = __builtin_convertvector(f2{pe[cb][2 * x], pe[cb][2 * x + 1]}, h2); // round to nearest even
                    pw[TP][cb][x / 4][x % 4] = __builtin_bit_cast(unsigned, hp[cb][x]);
                } else {
                    // The tile's share of the row sum is added up in packed fp16, one instruction per
                    // pair (eight terms per half; the rounding of these short sums averages out over
                    // the tiles), and joins the fp32 sum at the end of the step.  (v_dot2_f32_f16
                    // would add a pair to an fp32 sum directly, but it stalls behind the matrix
                    // instructions in flight.)
                    // (hp, not the element of pw it was stored to: read back through a bit cast, the
                    // compiler takes element 0 of the vector for every pair)
                    hsum[cb] += hp[cb][x];
                }
            };
            static_for<0, kTickets>([&](auto ic) {
                constexpr int i = decltype(ic)::value;
                constexpr int g = i / NCB, m = i % NCB;
                if constexpr (m == 0 && g % 2 == 0) issue_reads(IntC<g + kAhead>{}, ic);
                if constexpr (g < kCG) {
                    constexpr int db = g % G::kDBlk, kh = g / G::kDBlk;
                    mfma_o(o[m][db], gop[g], __builtin_bit_cast(h8, pw[TP ^ 1][m][kh]));
                } else {
                    constexpr int ks = g - kCG;
                    if constexpr (ks == 0) mfma_s_zero(s[TP ^ 1][m], gop[g], q[m][ks]);
                    else mfma_s(s[TP ^ 1][m], gop[g], q[m][ks]);
                }
                // (the compiler orders the vector instructions within a ticket, not across tickets:
                // the scores they read were written two or more matrix instructions earlier)
                __builtin_amdgcn_sched_barrier(0);
                if constexpr (i >= kSkip && (kPProbe & 1) == 0)
                    static_for<((i - kSkip) * kItems) / (kTickets - kSkip), ((i + 1 - kSkip) * kItems) / (kTickets - kSkip)>(item);
                __builtin_amdgcn_sched_barrier(0);
                if constexpr (m == NCB - 1 && (kPProbe & 4) == 0) {
                    if constexpr (i < kHalf) copy_one(IntC<i / NCB>{}, kdesc, k_buf(TP), ksoff);
                    else copy_one(IntC<(i - kHalf) / NCB>{}, vdesc, v_buf(TP ^ 1), vsoff);
                }
            });
            // ---- slow path: a weight of this tile is at the edge of the fp16 range or beyond.  Move
            // the reference of the columns concerned to their new maximum, redo P(t) and rescale
            // O and l. ----
            float amax = 0.0f;
#pragma unroll
            for (int cb = 0; cb < NCB; ++cb) {
                const float lo = (float)hsum[cb][0], hi = (float)hsum[cb][1];
                lsum[cb][0] += lo;
                lsum[cb][1] += hi;
                amax = __builtin_fmaxf(__builtin_fmaxf(amax, lo), hi);
            }
            if (__builtin_expect(__builtin_amdgcn_ballot_w64(!(amax < kBoundP)) != 0, 0)) {
                settle(); // C(t-1) has left the matrix pipe
#pragma unroll
                for (int cb = 0; cb < NCB; ++cb) {
                    float mx = s[TP][cb][0];
#pragma unroll
                    for (int r = 1; r < 16; ++r) mx = fmaxf(mx, s[TP][cb][r]);
                    mx = pair_max(mx);
                    const float top = __builtin_fmaf(mx, c, nb[cb]); // the column's largest exponent
                    const float delta = top > kBound ? top - kPShift : 0.0f;
                    const float alpha = fast_exp2(-delta);
                    nb[cb] -= delta;
                    // l: this tile's share was added under the old offset and may have overflowed:
                    // start again from the sum before this step
                    float new_sum = 0.0f;
#pragma unroll
                    for (int kh = 0; kh < 2; ++kh) {
                        h8 ph;
#pragma unroll
                        for (int j = 0; j < 8; ++j) {
                            ph[j] = (_Float16)fast_exp2(__builtin_fmaf(s[TP][cb][kh * 8 + j], c, nb[cb]));
                            new_sum += (float)ph[j];
                        }
                        pw[TP][cb][kh] = __builtin_bit_cast(u32x4, ph);
                    }
                    lsum[cb][0] = l_before[cb] * alpha + new_sum;
                    lsum[cb][1] = 0.0f;
#pragma unroll
                    for (int db = 0; db < G::kDBlk; ++db) {
                        pin_a(o[cb][db]); // the reads below stay behind the settled pipe
                        o[cb][db] *= alpha;
                        pin_a(o[cb][db]);
                    }
                }
                settle();
            }
            // S(t+1) is alive to the very end of the step even when nobody reads it (last step): its
            // registers must not be handed out while the matrix instructions that write them are
            // in flight (the compiler is free to sink the step's last vector instructions down to here).
#pragma unroll
            for (int cb = 0; cb < NCB; ++cb) keep_v(s[TP ^ 1][cb]);
        };
        if (R >= 1) body(IntC<1>{}, 1);
        int t = 2;
        for (; t + 1 <= R; t += 2) {
            body(IntC<0>{}, t);
            body(IntC<1>{}, t + 1);
        }
        if (t == R) body(IntC<0>{}, t);
        FA_STAMP(4);
        if constexpr ((kPProbe & 8) != 0) { if (n_past >= 0) return; } // (cut-off build)
        // ---- drain: C(R), and the accumulators on their way to the merge ----
        // V(R) has landed once the two tiles of copies issued after it are all that is outstanding
        // (those, for steps past the last, land in buffers nobody reads; their latency hides
        // behind the matrix instructions below).
        wait_copies(IntC<2 * kC>{});
        settle(); // P(R) was converted just above
        write_ml();
        {   // O += V(R)^T P(R); both live in the buffers of parity R & 1
            const bool odd = (R & 1) != 0;
            const int v_par = odd ? G::kTileB : 0;
            h8 va[2 * G::kDBlk], pl[NCB][2];
            if (odd) {
#pragma unroll
                for (int cb = 0; cb < NCB; ++cb) {
                    pw[0][cb][0] = pw[1][cb][0];
                    pw[0][cb][1] = pw[1][cb][1];
                }
            }
#pragma unroll
            for (int j = 0; j < 2 * G::kDBlk; ++j) {
                const int db = j % G::kDBlk, kh = j / G::kDBlk;
                const h4 v0 = lds_read_tr(vp[0][db] + v_par + kh * 16 * G::kRowB);
                const h4 v1 = lds_read_tr(vp[1][db] + v_par + kh * 16 * G::kRowB);
                va[j] = __builtin_shufflevector(v0, v1, 0, 1, 2, 3, 4, 5, 6, 7);
            }
#pragma unroll
            for (int cb = 0; cb < NCB; ++cb) {
                pl[cb][0] = __builtin_bit_cast(h8, pw[0][cb][0]);
                pl[cb][1] = __builtin_bit_cast(h8, pw[0][cb][1]);
            }
            // The accumulators are finished two at a time (their two products each alternating,
            // so that no product follows straight on the one it adds to), and a finished pair
            // goes to the merge buffer between the products of the next pair: one 32-byte share
            // per matrix instruction, read two or more matrix instructions after the last one
            // that wrote it.  Only the last pair's way to LDS is not covered.
            static_for<0, kAccs / 2>([&](auto pc) {
                constexpr int p = decltype(pc)::value;
                if constexpr (p == 1) // the merge buffer takes the tile buffers' place: every read of those has
                    __builtin_amdgcn_s_waitcnt(0x0070); // returned and every copy into them has landed
                static_for<0, 4>([&](auto sc) {
                    constexpr int sl = decltype(sc)::value, acc = 2 * p + sl % 2, kh = sl / 2;
                    constexpr int cb = acc / G::kDBlk, db = acc % G::kDBlk;
                    mfma_o_n(o[cb][db], va[kh * G::kDBlk + db], pl[cb][kh]);
                    if constexpr (p > 0) {
                        __builtin_amdgcn_sched_barrier(0);
                        write_o_half(IntC<2 * (p - 1) + sl / 2>{}, IntC<sl % 2>{}, IntC<1>{});
                        __builtin_amdgcn_sched_barrier(0);
                    }
                });
            });
            if constexpr (kAccs == 2) __builtin_amdgcn_s_waitcnt(0x0070);
        }
        settle(); // O is out of the matrix pipe
        static_for<kAccs - 2, kAccs>([&](auto ac) {
            write_o_half(ac, IntC<0>{}, IntC<1>{});
            write_o_half(ac, IntC<1>{}, IntC<1>{});
        });
    } else {
        // no tile for this wave: its share of the merge is zero, with weight zero
        settle(); // (the matrix instructions that cleared O are long done; said once more for the reads below)
        write_ml();
        static_for<0, kAccs>([&](auto ac) { // (behind settle(): LDS writes do not move across it)
            write_o_half(ac, IntC<0>{}, IntC<0>{});
            write_o_half(ac, IntC<1>{}, IntC<0>{});
        });
    }
    FA_STAMP(5);
    if constexpr ((kPProbe & 16) != 0) { if (n_past >= 0) return; } // (cut-off build)
    FA_STAMP(6);
    __syncthreads();
    FA_STAMP(7);

    // Four threads per column (eight in the 32-column shape, so that no thread idles): the weights
    // are computed once, then each thread merges and stores its share of the column's head_dim in
    // 16-byte pieces (the pieces of a step are one contiguous 64 or 128 bytes of the output row).
    constexpr int kParts = (kWaves * 64) / G::kCols; // threads per column: 4 with 64 columns, 8 with 32
    const int cm = threadIdx.x / kParts, part = threadIdx.x % kParts;
    int tok, hl;
    if (cm < G::kCols && col_valid(cm, tok, hl)) {
        // every LDS read first (the partial outputs in two halves of 16 reads), so that their
        // latencies overlap instead of adding up
        float mw[kWaves], lw[kWaves];
#pragma unroll
        for (int w = 0; w < kWaves; ++w) {
            mw[w] = ml[(w * G::kCols + cm) * 2 + 0];
            lw[w] = ml[(w * G::kCols + cm) * 2 + 1];
        }
        constexpr int kHalfJ = D / (8 * kParts); // 16-byte pieces per thread and half
        f4 x[kHalfJ][kWaves];
        auto load_half = [&](int j0) {
#pragma unroll
            for (int j = 0; j < kHalfJ; ++j)
#pragma unroll
                for (int w = 0; w < kWaves; ++w)
                    x[j][w] = *reinterpret_cast<const f4*>(smem + w * G::kWaveB + G::o_byte(cm, (j0 + j) * kParts + part));
        };
        load_half(0);
        __builtin_amdgcn_sched_barrier(0);
        float wgt[kWaves];
        float m_all = -INFINITY, l_all = 0.0f;
#pragma unroll
        for (int w = 0; w < kWaves; ++w) m_all = fmaxf(m_all, mw[w]);
#pragma unroll
        for (int w = 0; w < kWaves; ++w) {
            // (the wave that holds the column's diagonal has a finite m; with KV splits a split may
            // hold no visible row of a column at all)
            wgt[w] = m_all > -INFINITY ? fast_exp2(mw[w] - m_all) : 0.0f;
            l_all += lw[w] * wgt[w];
        }
        const float inv = l_all > 0.0f ? 1.0f / l_all : 0.0f;
#pragma unroll
        for (int w = 0; w < kWaves; ++w) wgt[w] *= inv;
        const size_t orow = (size_t)tok * n_head + kvh * r_heads + hl;
        float* dst = a.out + orow * D;
        if (kv_split_shift > 0) { // this split's normalised share and its log-sum-exp, for the combine kernel
            const size_t prow = (size_t)split * batch * n_head + orow;
            dst = a.part_o + prow * D;
            if (part == 0) a.part_ml[prow] = l_all > 0.0f ? m_all + __builtin_amdgcn_logf(l_all) : -INFINITY;
        }
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            f4 acc[kHalfJ];
#pragma unroll
            for (int j = 0; j < kHalfJ; ++j) {
                acc[j] = x[j][0] * wgt[0];
#pragma unroll
                for (int w = 1; w < kWaves; ++w) acc[j] += x[j][w] * wgt[w];
            }
            __builtin_amdgcn_sched_barrier(0);
            if (h == 0) load_half(kHalfJ);
            __builtin_amdgcn_sched_barrier(0);
            // Output rows leave with streaming stores: they go on their way to memory as each workgroup
            // finishes, instead of sitting in L2 until the kernel's end writes megabytes of them back at
            // once (1.2 us per launch on a Llama-3-8B chunk; a KV split's partial results, which the
            // combine kernel reads next, are better left to the caches: 1.5 us the other way on 16 splits).
            if (kv_split_shift > 0) {
#pragma unroll
                for (int j = 0; j < kHalfJ; ++j) *reinterpret_cast<f4*>(dst + ((h * kHalfJ + j) * kParts + part) * 4) = acc[j];
            } else {
#pragma unroll
                for (int j = 0; j < kHalfJ; ++j) // (spelled out: as a builtin the hint is lost when the compiler merges the two branches)
                    asm volatile("global_store_dwordx4 %0, %1, off nt" ::"v"(dst + ((h * kHalfJ + j) * kParts + part) * 4), "v"(acc[j]) : "memory");
            }
        }
    }
    FA_STAMP(8);
}

// out = sum over the KV splits of their normalised outputs, weighted by 2^(lse_s - max lse) and
// divided by the weights' sum.  One thread per 16 bytes of out; rows = batch * n_head.
template <int D>
__global__ __launch_bounds__(256) void fa_prefill_combine_kernel(const float* part_o, const float* part_lse, float* out,
                                                                 int rows, int splits) {
    const int idx = blockIdx.x * 256 + threadIdx.x;
    const int row = idx / (D / 4), piece = idx % (D / 4);
    if (row >= rows) return;
    float lse[4];
    f4 x[4];
    // (the loads of four splits at a time go out together; 2 or 4 splits is the common case)
    float m = -INFINITY, wsum = 0.0f;
    f4 acc = f4{0.f, 0.f, 0.f, 0.f};
    for (int s0 = 0; s0 < splits; s0 += 4) {
#pragma unroll
        for (int u = 0; u < 4; ++u)
            if (s0 + u < splits) {
                lse[u] = part_lse[(size_t)(s0 + u) * rows + row];
                x[u] = *reinterpret_cast<const f4*>(part_o + ((size_t)(s0 + u) * rows + row) * D + piece * 4);
            }
        float m_new = m;
#pragma unroll
        for (int u = 0; u < 4; ++u)
            if (s0 + u < splits) m_new = fmaxf(m_new, lse[u]);
        if (m_new > -INFINITY) { // (else: no split so far held a visible row of this column)
            const float keep = fast_exp2(m - m_new); // 0 on the first splits that hold one
            wsum *= keep;
            acc *= keep;
#pragma unroll
            for (int u = 0; u < 4; ++u)
                if (s0 + u < splits) {
                    const float w = fast_exp2(lse[u] - m_new); // 0 for a split without a visible row
                    wsum += w;
                    acc += x[u] * w;
                }
            m = m_new;
        }
    }
    const float inv = wsum > 0.0f ? 1.0f / wsum : 0.0f;
    *reinterpret_cast<f4*>(out + (size_t)row * D + piece * 4) = acc * inv;
}

template <int D, int NCB>
hipError_t launch_kernel(const FaArgs& a, dim3 grid, hipStream_t stream) {
    constexpr int lds = PGeom<D, NCB>::kLdsB;
    const unsigned packed = (unsigned)a.heads_per_group | (unsigned)a.kv_split_shift << 4 | (unsigned)a.tq << 8 | (unsigned)a.tq_magic << 16;
    hipLaunchKernelGGL((fa_prefill_kernel<D, NCB>), grid, dim3(kPrefillWaves * 64), lds, stream, a.q, a.kc, a.vc, a.n_ctx, a.n_past,
                       a.batch, a.n_head, a.r, a.n_ttiles, packed, a.qsign, a);
    return hipGetLastError();
}

template <int D, int NCB>
hipError_t allow_lds() {
    const auto kernel = fa_prefill_kernel<D, NCB>;
    return hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                               PGeom<D, NCB>::kLdsB);
}

constexpr int kMaxPrefillSplitShift = 4; // up to 16 workgroups share a token tile's KV rows (small chunks on long contexts)

// Rows of context from which cutting a token tile's rows among several workgroups pays for the
// second launch and the partial results' trip through memory (Qwen2.5-1.5B heads, 512-token
// chunk: 35.1 -> 33.2 us at 6144 rows, 106 -> 71 us at 16896, 304 -> 121 us at 32768; slower
// below about 4600 rows).
#ifndef ORIN_FA_SPLIT_MIN_ROWS
#define ORIN_FA_SPLIT_MIN_ROWS 5120
#endif
constexpr int kSplitMinRows = ORIN_FA_SPLIT_MIN_ROWS;

template <int D>
hipError_t launch(FaArgs a, int cu_count, hipStream_t stream, void* workspace, size_t workspace_bytes) {
    // Column packing: a workgroup's columns are (heads of the group) x (tq tokens), 64 of them
    // (two 32-column blocks) or 32.  GQA ratios up to 8 are one group; larger ratios are cut
    // into groups of 8 heads that each re-read the KV head.
    const int r = a.r;
    a.heads_per_group = r < 8 ? r : 8;
    a.n_hgroups = (r + a.heads_per_group - 1) / a.heads_per_group;
    int ncb = 2;
    a.tq = 64 / a.heads_per_group;
    // A workgroup occupies a whole CU and the kernel lasts as long as its longest workgroup, so
    // a grid that would leave half the CUs idle is cut finer: 32 columns per workgroup.
    // On a long context the better cut is along the KV rows: the workgroup keeps its 64 columns
    // (a step's K and V tiles then serve twice the columns: in the 32-column shape the step is
    // bound by what the CU's vector memory path delivers, 64 bytes a clock, not by the matrix
    // pipe) and 2, 4, 8 or 16 workgroups share a token tile's rows; a second, small kernel merges
    // their results.  Needs room for the partial results in the workspace.
    a.kv_split_shift = 0;
    const int wgs64 = a.n_kv * a.n_hgroups * ((a.batch + a.tq - 1) / a.tq);
    if (2 * wgs64 <= cu_count) {
        int shift = 1;
        while (shift < kMaxPrefillSplitShift && (wgs64 << (shift + 1)) <= cu_count) ++shift;
        const size_t rows = (size_t)a.batch * a.n_head;
        const size_t need = (rows << shift) * (D + 1) * sizeof(float);
        // (with four or more workgroups per token tile the walk shortens enough to pay from about
        // 2500 rows: 19.9 -> 17.7 us at 4000 rows for a 256-token chunk)
        const int min_rows = shift >= 2 ? (kSplitMinRows * 3) / 5 : kSplitMinRows;
        if (a.n_past + a.batch >= min_rows && workspace && need <= workspace_bytes) {
            a.kv_split_shift = shift;
            a.part_o = static_cast<float*>(workspace);
            a.part_ml = a.part_o + (rows << shift) * D;
        } else {
            ncb = 1;
            a.tq = 32 / a.heads_per_group;
        }
    }
    a.n_ttiles = (a.batch + a.tq - 1) / a.tq;
    a.tq_magic = 65536 / a.tq + 1;
    if ((a.n_hgroups << a.kv_split_shift) > 65535 || a.n_ttiles > 65535) return hipErrorInvalidValue;
    const dim3 grid(a.n_kv, a.n_hgroups << a.kv_split_shift, a.n_ttiles);
    const hipError_t e = ncb == 2 ? launch_kernel<D, 2>(a, grid, stream) : launch_kernel<D, 1>(a, grid, stream);
    if (e != hipSuccess || a.kv_split_shift == 0) return e;
    const int rows = a.batch * a.n_head;
    const unsigned blocks = (unsigned)(((size_t)rows * (D / 4) + 255) / 256);
    hipLaunchKernelGGL(fa_prefill_combine_kernel<D>, dim3(blocks), dim3(256), 0, stream, a.part_o, a.part_ml, a.out, rows,
                       1 << a.kv_split_shift);
    return hipGetLastError();
}

} // namespace

hipError_t prefill_launch(const FaArgs& a, int head_dim, int cu_count, hipStream_t stream, void* workspace,
                          size_t workspace_bytes) {
    drop_stale_error();
    return head_dim == 128 ? launch<128>(a, cu_count, stream, workspace, workspace_bytes)
                           : launch<64>(a, cu_count, stream, workspace, workspace_bytes);
}

// The kernels use more than 64 KB of dynamic LDS; the opt-in is set once per kernel at init.
hipError_t prefill_allow_lds() {
    hipError_t e;
    if ((e = allow_lds<128, 1>()) != hipSuccess) return e;
    if ((e = allow_lds<128, 2>()) != hipSuccess) return e;
    if ((e = allow_lds<64, 1>()) != hipSuccess) return e;
    return allow_lds<64, 2>();
}

hipError_t prefill_stamps(long long* host, size_t n) {
#ifdef ORIN_FA_STAMPS
    if (n > (size_t)kStampWgs * kPrefillWaves * kStampSlots) return hipErrorInvalidValue;
    hipError_t e = hipMemcpyFromSymbol(host, HIP_SYMBOL(g_prefill_stamps), n * sizeof(long long)); // (synchronises with the device)
    void* dev = nullptr;
    if (e == hipSuccess) e = hipGetSymbolAddress(&dev, HIP_SYMBOL(g_prefill_stamps));
    if (e == hipSuccess) e = hipMemset(dev, 0, sizeof(g_prefill_stamps)); // the next launch starts from an empty table
    return e;
#else
    (void)host; (void)n;
    return hipErrorNotSupported;
#endif
}

} // namespace orin_fa
