// Matrix-vector products over quantised weight rows (Q4_K, Q5_K, Q6_K, Q8_0) on the matrix cores of gfx950
// (MI355X).
//
// The vector-ALU kernel of gemv.hip spends about three instructions per weight (byte to float,
// multiply-add, unpacking) and is bound by them at twice the time HBM needs for the bytes.  Here
// the multiply-adds run as integer matrix instructions and the vector ALU only assembles the
// weights' bytes and applies the blocks' scales:
//
//   * The activation is cut, per sub-block of the weight format (16 elements for Q6_K, 32 for
//     the others), into three signed 8-bit digits of a 24-bit integer, x = s (65536 d0 + 256 d1 + d2)
//     with s = max|x| / (2^23 - 2^16): what the reference does with one digit (quantize_q8_1_k,
//     reference: src/kernels.cu:136-157), carried to the precision of an fp32 mantissa.  Every
//     workgroup builds the digits once, in LDS (together with the RMS norm, when that is folded
//     in), with the sub-blocks' scales and sums beside them.
//   * v_mfma_i32_16x16x64_i8 then multiplies 16 weight rows by 64 elements at a time: the weights,
//     widened to bytes, are the B operand (lane (n, g) holds 16 elements of row n), and the A
//     operand's rows are (sub-block, digit) pairs, each row zero outside its own sub-block.  An
//     accumulator therefore holds, for a row of weights, the exact integer sums of four sub-blocks
//     against the three digits, already separated: lane (n, g) receives the three sums of
//     sub-block g.  They are recombined in fp32 and multiplied by the sub-block's scales:
//     d * scale * sum - dmin * min * sum(x) for Q4_K and Q5_K, d * scale * (sum - 32 sum(x)) for Q6_K,
//     d * sum for Q8_0 (reference CPU statements: src/model_cpu.cpp:70-152).
//   * Loads are made with four neighbouring lanes on 64 consecutive bytes of a row (lane = 4 * row +
//     piece: the vector cache then sees 16 runs per instruction; with the matrix instruction's own
//     lane order, lane = row + 16 * piece, it sees 64 separate 16-byte requests and the kernel runs
//     10 % slower) and moved to the matrix instruction's lanes by one lane permutation per register.
//   * The four waves of a workgroup take every fourth 256-element block of the same 16 rows and meet
//     in LDS at the end; blocks are requested one iteration ahead, across row tiles.
//   * Q4_K, Q5_K and Q6_K matrices made of whole 16-row tiles -- every matrix of a model -- take a second
//     kernel with the same arithmetic and another way to the bytes (gemv_rows_kernel, further down): rows
//     read in lane-linear runs of two blocks with streaming loads and laid out for the matrix instruction
//     through a wave's own LDS buffer, which this machine's memory path serves a quarter faster.  The
//     kernel described above remains for Q8_0 and for matrices with a ragged last tile.
#include "layer_common.hpp"
#include "fa_common.hpp"

// Stage marks of the kernel that reads rows in long runs: wall-clock stamps in the timeline build (waves 0-3 of a
// workgroup), nothing otherwise (fa_common.hpp).  ROWS_ITEM_STAMP marks an item's arrival in LDS and waits for the
// LDS writes first, in that build only.
#ifdef ORIN_FA_STAMPS
namespace orin_fa {
__device__ long long g_gemv_stamps[kStampWgs * 4 * kStampSlots];
}
// (its own store, all conditions in one test: wrapped around the attention kernels' macro the marks cost this kernel a
// quarter of its time)
#define ROWS_STAMP(i)                                                                                                      \
    do {                                                                                                                   \
        __builtin_amdgcn_sched_barrier(0);                                                                                 \
        const unsigned wg_ = blockIdx.x + gridDim.x * (blockIdx.y + gridDim.y * blockIdx.z);                               \
        if ((threadIdx.x & 63) == 0 && threadIdx.x < 256 && wg_ < (unsigned)orin_fa::kStampWgs && (i) < orin_fa::kStampSlots) \
            orin_fa::g_gemv_stamps[(wg_ * 4 + (threadIdx.x >> 6)) * orin_fa::kStampSlots + (i)] =                          \
                (long long)__builtin_amdgcn_s_memrealtime();                                                               \
        __builtin_amdgcn_sched_barrier(0);                                                                                 \
    } while (0)
#define ROWS_ITEM_STAMP(i)                                  \
    do {                                                    \
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); \
        ROWS_STAMP(i);                                      \
    } while (0)
#else
#define ROWS_STAMP(i)
#define ROWS_ITEM_STAMP(i)
#endif

#include <stdlib.h>

namespace orin_fa {
namespace {

constexpr int kMaxWaves = 8; // waves per workgroup: 4, or 8 where a matrix has few 16-row tiles and long rows
constexpr float kDigitRange = 8388608.0f - 65536.0f; // largest |integer| the three signed digits hold

struct XPair {
    float scale, sum; // of one sub-block of the activation
};

// LDS: digit planes [3][n_in] | XPair [n_in / G] | 16 zero bytes | partial row sums [kMaxWaves][2][16]
template <int G>
struct Lds {
    static __host__ __device__ int pairs_off(int n_in) { return 3 * n_in; }
    static __host__ __device__ int zero_off(int n_in) { return 3 * n_in + n_in / G * 8; }
    static __host__ __device__ int red_off(int n_in) { return zero_off(n_in) + 16; }
    static __host__ __device__ size_t bytes(int n_in) { return (size_t)red_off(n_in) + kMaxWaves * 2 * 16 * 4; }
};

// Eight consecutive elements (x, already multiplied by the norm's weights) of a group of G into the digit planes;
// the G / 8 threads of a group sit in one quad (n_in is a multiple of 32, so a quad is never split) and meet
// by DPP moves.
template <int G>
__device__ __forceinline__ void digits8(const float (&x)[8], int e, int n_in, unsigned char* smem, XPair* pairs, int tid) {
    float mx = 0.0f, sum = 0.0f;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        mx = fmaxf(mx, fabsf(x[i]));
        sum += x[i];
    }
    mx = fmaxf(mx, dpp_xor_step(mx, 0));
    sum += dpp_xor_step(sum, 0);
    if constexpr (G == 32) {
        mx = fmaxf(mx, dpp_xor_step(mx, 1));
        sum += dpp_xor_step(sum, 1);
    }
    // A group that holds an infinity or a NaN gets a NaN scale, so that every row sum it enters is NaN, as the
    // products of the vector-ALU kernel are (fmaxf above drops a NaN and (int)rintf would turn it into 0; the sum
    // does not lose it: a sum of floats is finite only if every term is).
    const float scale = sum - sum == 0.0f ? (mx > 0.0f ? mx / kDigitRange : 1.0f) : __builtin_nanf("");
    const float inv = 1.0f / scale;
    // X + 0x808080 carries 128 into each of the three byte positions, so its bytes are the signed
    // digits plus 128 (byte k of X + 0x808080 is ((X >> 8 k) + 128) & 255 with the lower digits'
    // carries already taken out); the exclusive-or takes the 128 off again, byte by byte.
    unsigned z[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) z[i] = ((unsigned)((int)rintf(x[i] * inv)) + 0x808080u) ^ 0x808080u;
    // byte k of four consecutive elements into one word of plane 2 - k (plane 0 holds the top digits)
    u32x2 plane[3];
#pragma unroll
    for (int k = 0; k < 3; ++k) {
        const unsigned pick = (unsigned)k | ((unsigned)(4 + k) << 8); // byte k of the second operand, then of the first
#pragma unroll
        for (int w = 0; w < 2; ++w) {
            const unsigned t01 = __builtin_amdgcn_perm(z[4 * w + 1], z[4 * w + 0], pick);
            const unsigned t23 = __builtin_amdgcn_perm(z[4 * w + 3], z[4 * w + 2], pick);
            plane[2 - k][w] = __builtin_amdgcn_perm(t23, t01, 0x05040100u);
        }
    }
    *reinterpret_cast<u32x2*>(smem + e) = plane[0];
    *reinterpret_cast<u32x2*>(smem + n_in + e) = plane[1];
    *reinterpret_cast<u32x2*>(smem + 2 * n_in + e) = plane[2];
    if ((tid & (G / 8 - 1)) == 0) pairs[e / G] = XPair{scale, sum};
}

// Digits of the (optionally normalised) activation into LDS, in groups of G elements.  Thread t takes
// elements 8 t .. 8 t + 7 of every kWaves * 512.
template <int G, int kWaves>
__device__ float stage_digits(const GemvArgs& a, int first, int n_in, unsigned char* smem, float* red) {
    // Elements [first, first + n_in) of the activation.  With the RMS norm folded in (whole rows only), the
    // digits are those of x * w; the norm's scalar 1 / sqrt(mean(x^2) + eps), which needs the whole vector,
    // multiplies the finished row sums instead (returned): one pass over x.
    const int tid = threadIdx.x;
    const float* const ax = a.x + first;
    const float* const aw = a.norm_w ? a.norm_w + first : nullptr;
    float ss = 0.0f;
    XPair* pairs = reinterpret_cast<XPair*>(smem + Lds<G>::pairs_off(n_in));
    for (int e = tid * 8; e < n_in; e += kWaves * 64 * 8) {
        float x[8];
        *reinterpret_cast<float4*>(x) = *reinterpret_cast<const float4*>(ax + e);
        *reinterpret_cast<float4*>(x + 4) = *reinterpret_cast<const float4*>(ax + e + 4);
        if (aw) {
            float g[8];
            *reinterpret_cast<float4*>(g) = *reinterpret_cast<const float4*>(aw + e);
            *reinterpret_cast<float4*>(g + 4) = *reinterpret_cast<const float4*>(aw + e + 4);
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                ss += x[i] * x[i];
                x[i] *= g[i];
            }
        }
        digits8<G>(x, e, n_in, smem, pairs, tid);
    }
    if (tid < 4) reinterpret_cast<unsigned*>(smem + Lds<G>::zero_off(n_in))[tid] = 0u;
    if (!aw) {
        __syncthreads();
        return 1.0f;
    }
    ss = wave_sum(ss);
    if ((tid & 63) == 0) red[tid >> 6] = ss;
    __syncthreads();
    ss = 0.0f;
#pragma unroll
    for (int w = 0; w < kWaves; ++w) ss += red[w];
    __syncthreads(); // (red is reused for the row sums)
    return 1.0f / sqrtf(ss / (float)n_in + a.eps);
}

// A workgroup barrier that waits for this wave's LDS traffic only: weight requests in flight stay in flight.
__device__ __forceinline__ void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

// 16-byte loads of the kernels that fetch 64 bytes of each of 16 rows per instruction: ordinary ones, because the
// neighbouring pieces of a line are fetched by other instructions and meet in the CU's cache (as streaming loads,
// which pass that cache, these kernels take half as long again).  p may be 2-byte aligned.
typedef u32x4 u32x4_a2 __attribute__((aligned(2)));
__device__ __forceinline__ u32x4 load16(const unsigned char* p) { return *reinterpret_cast<const u32x4_a2*>(p); }
__device__ __forceinline__ u32x4 load16_aligned(const unsigned char* p) { return *reinterpret_cast<const u32x4*>(p); }
__device__ __forceinline__ float half_of(unsigned bits) { return (float)__builtin_bit_cast(_Float16, (uint16_t)bits); }
__device__ __forceinline__ unsigned from_lane(int src_lane4, unsigned v) {
    return (unsigned)__builtin_amdgcn_ds_bpermute(src_lane4, (int)v);
}
// (the upper two digits' sums are put together as integers: below 2^30 for every block type, and rounded once on
// conversion where the fused multiply-add of the converted parts would round, to the same value)
__device__ __forceinline__ float digits_sum(const i32x4& acc) {
    return (float)(acc[0] * 256 + acc[1]) * 256.0f + (float)acc[2];
}
// Every byte's low nibble from a, its high nibble from b, in one instruction (spelled out, since the compiler, which
// knows which bits of b can be set, narrows the mask and then needs an AND and an AND-OR).
__device__ __forceinline__ unsigned low_nibbles_of(unsigned a, unsigned b) {
    unsigned r;
    asm("v_bfi_b32 %0, %1, %2, %3" : "=v"(r) : "v"(0x0f0f0f0fu), "v"(a), "v"(b));
    return r;
}
// LDS byte offset of a lane's A operand: base + x for a lane that holds digits (step 1), base (the zero bytes) for
// one whose rows are zero (step 0); x is the same in every lane.  One 24-bit multiply-add.
__device__ __forceinline__ int operand_at(int base, int step, int x) {
    return (int)(__umul24((unsigned)x, (unsigned)step) + (unsigned)base);
}
// (the step as a value the compiler knows nothing of: told that it is 0 or 1, it replaces the multiply-add by a
// move, a select and an add)
__device__ __forceinline__ int opaque_step(bool on) {
    int step = on ? 1 : 0;
    asm volatile("" : "+v"(step));
    return step;
}

// What a lane needs to know of itself: as a loader (row ln of the tile, 16-byte piece lg), as a lane of
// the matrix instruction (weight row / column n, element group g; the loader of its data is lane
// 4 n + g, whose piece is g as well), and as a lane of the A operand (accumulator row am = 4 p + digit).
struct LaneCtx {
    int n, g, ln, lg, src_lane4, am;
    const unsigned char* smem;
    const XPair* pairs;
    int n_in, zero_off;
};

template <int T>
struct MF;

// Q4_K and Q5_K (reference: src/quant.h:14-31): per 128-element half of a block, the lane's 16 bytes of
// nibbles are 16 elements of sub-block 2 (g / 2) (low nibbles) and of 2 (g / 2) + 1 (high nibbles); the two
// matrix instructions of a half add into one accumulator whose row group p is sub-block p of the half.
// Q5_K keeps a fifth bit per element in 32 bytes behind the header: bit p of byte e belongs to element e of
// sub-block p.
template <bool FIVE>
struct MFK45 {
    static constexpr int kGroup = 32, kBlockBytes = FIVE ? 176 : 144, kQs = FIVE ? 48 : 16;
    struct Raw {
        u32x4 hdr, q1, q2; // a block's header and this lane's 16 bytes of each half of its nibbles
        u32x4 qh;          // (Q5_K) the 16 bytes of fifth bits that cover this lane's elements
    };
    struct Addr {
        int lo_base, hi_base, lo_step, hi_step; // LDS byte offsets of this lane's A operands and whether they move with the block (1); a lane whose row is zero reads the 16 zero bytes (0)
    };
    static __device__ __forceinline__ void load(const unsigned char* blk, int lg, Raw& r) {
        r.hdr = load16_aligned(blk);
        if constexpr (FIVE) r.qh = load16_aligned(blk + 16 + 16 * (lg & 1));
        r.q1 = load16_aligned(blk + kQs + 16 * lg);
        r.q2 = load16_aligned(blk + kQs + 64 + 16 * lg);
    }
    static __device__ __forceinline__ Addr addr(const LaneCtx& c) {
        const int ap = c.am >> 2, ad = c.am & 3, g = c.g;
        const bool live = ad < 3 && (ap >> 1) == (g >> 1);
        const int elem = 64 * (g >> 1) + 16 * (g & 1);
        const bool lo = live && (ap & 1) == 0, hi = live && (ap & 1) == 1;
        return Addr{lo ? ad * c.n_in + elem : c.zero_off, hi ? ad * c.n_in + elem + 32 : c.zero_off, opaque_step(lo), opaque_step(hi)};
    }
    static __device__ __forceinline__ float block(const Raw& r, const LaneCtx& c, const Addr& ad, int b) {
        // (the loading lane holds piece lg of its row, and lane (n, g) wants piece g of row n: the bytes of
        // the packed pairs it needs are bytes lg of the loading lane's three words)
        const unsigned mine = ((r.hdr.y >> (8 * c.lg)) & 0xffu) | (((r.hdr.z >> (8 * c.lg)) & 0xffu) << 8) |
                              (((r.hdr.w >> (8 * c.lg)) & 0xffu) << 16);
        const unsigned dd = from_lane(c.src_lane4, r.hdr.x), bb = from_lane(c.src_lane4, mine);
        u32x4 fifth = {0u, 0u, 0u, 0u}, q1, q2;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            if constexpr (FIVE) fifth[i] = from_lane(c.src_lane4, r.qh[i]) >> (2 * (c.g >> 1));
            q1[i] = from_lane(c.src_lane4, r.q1[i]);
            q2[i] = from_lane(c.src_lane4, r.q2[i]);
        }
        const unsigned b0 = bb & 0xffu, b1 = (bb >> 8) & 0xffu, b2 = (bb >> 16) & 0xffu;
        // pairs g (first half of the block) and 4 + g (second half) of the twelve packed bytes
        const float sc[2] = {(float)(b0 & 63u), (float)((b2 & 0x0fu) | ((b0 >> 6) << 4))};
        const float mn[2] = {(float)(b1 & 63u), (float)((b2 >> 4) | ((b1 >> 6) << 4))};
        return math(dd, sc, mn, q1, q2, fifth, c, ad, b);
    }
    // A block laid out in LDS piece after piece (the kernel that reads rows in long runs): piece k is the block's
    // bytes 16 k ...
    static constexpr int kPieces = kBlockBytes / 16;
    static constexpr bool kAligned = true;
    static __host__ __device__ constexpr int piece_off(int k) { return 16 * k; }
    static __device__ __forceinline__ float from_lds(const unsigned char* blk, const LaneCtx& c, const Addr& ad, int b) {
        const u32x4 hdr = *reinterpret_cast<const u32x4*>(blk);
        const u32x4 q1 = *reinterpret_cast<const u32x4*>(blk + kQs + 16 * c.g);
        const u32x4 q2 = *reinterpret_cast<const u32x4*>(blk + kQs + 64 + 16 * c.g);
        u32x4 fifth = {0u, 0u, 0u, 0u};
        if constexpr (FIVE) fifth = *reinterpret_cast<const u32x4*>(blk + 16 + 16 * (c.g & 1)) >> (unsigned)(2 * (c.g >> 1));
        // the six-bit pairs straight out of the three words (bit fields at 8 g: no byte is put together first)
        const unsigned s8 = 8 * c.g;
        const float sc[2] = {(float)__builtin_amdgcn_ubfe(hdr.y, s8, 6), (float)(__builtin_amdgcn_ubfe(hdr.w, s8, 4) | ((hdr.y >> (s8 + 2)) & 0x30u))};
        const float mn[2] = {(float)__builtin_amdgcn_ubfe(hdr.z, s8, 6), (float)(__builtin_amdgcn_ubfe(hdr.w, s8 + 4, 4) | ((hdr.z >> (s8 + 2)) & 0x30u))};
        return math(hdr.x, sc, mn, q1, q2, fifth, c, ad, b);
    }
    // In lane (n, g): dd = the block's two fp16 scales, sc / mn = the six-bit scales and minima of sub-blocks g (first
    // half of the block) and 4 + g (second half), q1 / q2 = piece g of each half of the nibbles, fifth = the fifth
    // bits of this lane's elements shifted down to bit 0 (Q5_K).
    static __device__ __forceinline__ float math(unsigned dd, const float (&sc)[2], const float (&mn)[2], const u32x4& q1, const u32x4& q2,
                                                 const u32x4& fifth, const LaneCtx& c, const Addr& ad, int b) {
        const float d = half_of(dd & 0xffffu), dmin = half_of(dd >> 16);
        float scaled[2], offset[2]; // sum of sc * q * x and of mn * x over a sub-block pair; the block's two scales come last
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const i32x4 alo = *reinterpret_cast<const i32x4*>(c.smem + operand_at(ad.lo_base, ad.lo_step, 256 * b + 128 * h));
            const i32x4 ahi = *reinterpret_cast<const i32x4*>(c.smem + operand_at(ad.hi_base, ad.hi_step, 256 * b + 128 * h));
            const XPair xp = c.pairs[8 * b + 4 * h + c.g];
            const u32x4 qs = h ? q2 : q1;
            i32x4 lo, hi;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const unsigned q = qs[i];
                unsigned l = q & 0x0f0f0f0fu, u = (q >> 4) & 0x0f0f0f0fu;
                if constexpr (FIVE) { // sub-blocks 4 h + 2 (g / 2) and + 1: bits 4 h and 4 h + 1 of the shifted bytes
                    const unsigned f = fifth[i] >> (4 * h);
                    l |= (f & 0x01010101u) << 4;
                    u |= (f & 0x02020202u) << 3;
                }
                lo[i] = (int)l;
                hi[i] = (int)u;
            }
            i32x4 acc = {0, 0, 0, 0};
            acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(alo, lo, acc, 0, 0, 0);
            acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(ahi, hi, acc, 0, 0, 0);
            scaled[h] = sc[h] * (digits_sum(acc) * xp.scale);
            offset[h] = mn[h] * xp.sum;
        }
        return d * (scaled[0] + scaled[1]) - dmin * (offset[0] + offset[1]);
    }
};
template <>
struct MF<kQ4_K> : MFK45<false> {};
template <>
struct MF<kQ5_K> : MFK45<true> {};

// Q8_0 (reference: src/quant.h:42-45; blocks of 34 bytes, 2-byte aligned): eight blocks make up the 256
// elements the kernel walks at a time.  Per 128-element half, the lane's 16 bytes are half of block
// 2 run + g / 2 of the half, for run = 0, 1: one matrix instruction per run, both adding into one accumulator
// whose row group p is block p of the half.
template <>
struct MF<kQ8_0> {
    static constexpr int kGroup = 32, kBlockBytes = 272;
    struct Raw {
        u32x4 q[2][2]; // [half][run]
        unsigned d[2]; // scales of blocks lg and 4 + lg
    };
    typedef MFK45<false>::Addr Addr;
    template <typename V>
    struct __attribute__((packed, aligned(2))) Loose {
        V v;
    };
    static __device__ __forceinline__ void load(const unsigned char* blk, int lg, Raw& r) {
#pragma unroll
        for (int h = 0; h < 2; ++h) {
#pragma unroll
            for (int run = 0; run < 2; ++run)
                r.q[h][run] = load16(blk + 34 * (4 * h + 2 * run + (lg >> 1)) + 2 + 16 * (lg & 1));
            r.d[h] = *reinterpret_cast<const uint16_t*>(blk + 34 * (4 * h + lg));
        }
    }
    static __device__ __forceinline__ Addr addr(const LaneCtx& c) {
        const int ap = c.am >> 2, ad = c.am & 3, g = c.g;
        const bool live = ad < 3 && (ap & 1) == (g >> 1);
        const int elem = 32 * ap + 16 * (g & 1);
        const bool r0 = live && (ap >> 1) == 0, r1 = live && (ap >> 1) == 1;
        return Addr{r0 ? ad * c.n_in + elem : c.zero_off, r1 ? ad * c.n_in + elem : c.zero_off, opaque_step(r0), opaque_step(r1)};
    }
    static __device__ __forceinline__ float block(const Raw& r, const LaneCtx& c, const Addr& ad, int b) {
        float out[2];
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const i32x4 a0 = *reinterpret_cast<const i32x4*>(c.smem + operand_at(ad.lo_base, ad.lo_step, 256 * b + 128 * h));
            const i32x4 a1 = *reinterpret_cast<const i32x4*>(c.smem + operand_at(ad.hi_base, ad.hi_step, 256 * b + 128 * h));
            const XPair xp = c.pairs[8 * b + 4 * h + c.g];
            const float d = half_of(from_lane(c.src_lane4, r.d[h]));
            i32x4 w0, w1;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                w0[i] = (int)from_lane(c.src_lane4, r.q[h][0][i]);
                w1[i] = (int)from_lane(c.src_lane4, r.q[h][1][i]);
            }
            i32x4 acc = {0, 0, 0, 0};
            acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(a0, w0, acc, 0, 0, 0);
            acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(a1, w1, acc, 0, 0, 0);
            out[h] = d * (digits_sum(acc) * xp.scale);
        }
        return out[0] + out[1];
    }
};

// Q6_K (reference: src/quant.h:34-40; blocks of 210 bytes, 2-byte aligned): per 128-element half, piece g
// of the half's 64 low-nibble bytes holds sub-block g (elements 16 g .. 16 g + 15 of the half) in its low
// nibbles and sub-block 4 + g in its high nibbles; their high bit pairs sit in high byte 16 (g & 1) + i at
// bits 2 (g / 2) and 4 + 2 (g / 2).  One matrix instruction and one accumulator per nibble; the element
// group g of the instruction is sub-block g (or 4 + g), so the A operand's row group p is live in group p.
template <>
struct MF<kQ6_K> {
    static constexpr int kGroup = 16, kBlockBytes = 210;
    struct Raw {
        u32x4 ql[2], qh[2], sc;
        unsigned d;
    };
    struct Addr {
        int base, step;
    };
    template <typename V>
    struct __attribute__((packed, aligned(2))) Loose {
        V v;
    };
    static __device__ __forceinline__ void load(const unsigned char* blk, int lg, Raw& r) {
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            r.ql[h] = load16(blk + 64 * h + 16 * lg);
            r.qh[h] = load16(blk + 128 + 32 * h + 16 * (lg & 1));
        }
        r.sc = load16(blk + 192);
        r.d = *reinterpret_cast<const uint16_t*>(blk + 208);
    }
    static __device__ __forceinline__ Addr addr(const LaneCtx& c) {
        const int ap = c.am >> 2, ad = c.am & 3;
        const bool live = ad < 3 && ap == c.g;
        return Addr{live ? ad * c.n_in + 16 * c.g : c.zero_off, opaque_step(live)};
    }
    static __device__ __forceinline__ float block(const Raw& r, const LaneCtx& c, const Addr& ad, int b) {
        // scales 8 h + g and 8 h + 4 + g of both halves: byte lg of each of the loading lane's four words
        const unsigned mine = ((r.sc.x >> (8 * c.lg)) & 0xffu) | (((r.sc.y >> (8 * c.lg)) & 0xffu) << 8) |
                              (((r.sc.z >> (8 * c.lg)) & 0xffu) << 16) | (((r.sc.w >> (8 * c.lg)) & 0xffu) << 24);
        const unsigned ss = from_lane(c.src_lane4, mine);
        const unsigned dd = from_lane(c.src_lane4, r.d);
        u32x4 ql[2], qh[2];
#pragma unroll
        for (int h = 0; h < 2; ++h) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                ql[h][i] = from_lane(c.src_lane4, r.ql[h][i]);
                qh[h][i] = from_lane(c.src_lane4, r.qh[h][i]);
            }
        }
        return math(ss, dd, ql, qh, c, ad, b);
    }
    // A block laid out in LDS piece after piece (the kernel that reads rows in long runs): pieces 0 ... 12 are the
    // block's bytes 16 k ..., piece 13 its last 16 bytes (194 ... 209: the fp16 scale in its last two), so that no
    // piece reaches past the block.
    static constexpr int kPieces = 14;
    static constexpr bool kAligned = false;
    static __host__ __device__ constexpr int piece_off(int k) { return k < 13 ? 16 * k : 194; }
    static __device__ __forceinline__ float from_lds(const unsigned char* blk, const LaneCtx& c, const Addr& ad, int b) {
        const u32x4 sc = *reinterpret_cast<const u32x4*>(blk + 192);
        const unsigned ss = ((sc.x >> (8 * c.g)) & 0xffu) | (((sc.y >> (8 * c.g)) & 0xffu) << 8) | (((sc.z >> (8 * c.g)) & 0xffu) << 16) |
                            (((sc.w >> (8 * c.g)) & 0xffu) << 24);
        const unsigned dd = *reinterpret_cast<const unsigned*>(blk + 13 * 16 + 12) >> 16;
        u32x4 ql[2], qh[2];
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            ql[h] = *reinterpret_cast<const u32x4*>(blk + 64 * h + 16 * c.g);
            qh[h] = *reinterpret_cast<const u32x4*>(blk + 128 + 32 * h + 16 * (c.g & 1));
        }
        return math(ss, dd, ql, qh, c, ad, b);
    }
    // In lane (n, g): ss = the scales 8 h + g and 8 h + 4 + g of both halves (a byte each), dd = the block's fp16
    // scale, ql / qh = piece g of each half's low nibbles and the piece of high bit pairs that covers it.
    static __device__ __forceinline__ float math(unsigned ss, unsigned dd, const u32x4 (&ql)[2], const u32x4 (&qh)[2], const LaneCtx& c,
                                                 const Addr& ad, int b) {
        const float d = half_of(dd & 0xffffu);
        const int s1 = 2 * (c.g >> 1);
        float out[2];
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const i32x4 alo = *reinterpret_cast<const i32x4*>(c.smem + operand_at(ad.base, ad.step, 256 * b + 128 * h));
            const i32x4 ahi = *reinterpret_cast<const i32x4*>(c.smem + operand_at(ad.base, ad.step, 256 * b + 128 * h + 64));
            const XPair xlo = c.pairs[16 * b + 8 * h + c.g], xhi = c.pairs[16 * b + 8 * h + 4 + c.g];
            i32x4 lo, hi;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                // u: this lane's two bit pairs of every byte at bits 0, 1 and 4, 5, nothing else; each lands in the
                // high nibble of its element by one bit-field insert
                const unsigned l = ql[h][i], u = (qh[h][i] >> s1) & 0x33333333u;
                lo[i] = (int)low_nibbles_of(l, u << 4);
                hi[i] = (int)low_nibbles_of(l >> 4, u);
            }
            const i32x4 zero = {0, 0, 0, 0};
            const i32x4 acc_lo = __builtin_amdgcn_mfma_i32_16x16x64_i8(alo, lo, zero, 0, 0, 0);
            const i32x4 acc_hi = __builtin_amdgcn_mfma_i32_16x16x64_i8(ahi, hi, zero, 0, 0, 0);
            const float sc_lo = (float)((int)(ss << (24 - 16 * h)) >> 24), sc_hi = (float)((int)(ss << (16 - 16 * h)) >> 24);
            out[h] = sc_lo * (digits_sum(acc_lo) * xlo.scale - 32.0f * xlo.sum) + sc_hi * (digits_sum(acc_hi) * xhi.scale - 32.0f * xhi.sum);
        }
        return d * (out[0] + out[1]);
    }
};

// T: weight type.  DUAL: two matrices (gate, up) and SiLU(gate) * up.  Grid: (workgroups, matrices); a
// workgroup walks the 16-row tiles blockIdx.x, + gridDim.x, ...
template <int T, bool DUAL, int kWaves>
__device__ __forceinline__ void gemv_mfma_body(const GemvArgs& a) {
    using F = MF<T>;
    using L = Lds<F::kGroup>;
    typedef typename F::Raw Raw;
    constexpr int M = DUAL ? 2 : 1;
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    // gridDim.z workgroups share a tile's blocks (a matrix with few tiles and long rows, accumulating into y):
    // this one takes blocks [b0, b0 + nb), stages that part of the activation only, and adds its row sums to
    // y atomically.  gridDim.z = 1: the whole row, stored.
    const int nb_row = a.n_in >> 8;
    const int b0 = (int)blockIdx.z * nb_row / (int)gridDim.z, nb = ((int)blockIdx.z + 1) * nb_row / (int)gridDim.z - b0;
    const int n_in = nb << 8; // (elements this workgroup works on: LDS is laid out for them)
    float* const red = reinterpret_cast<float*>(smem + L::red_off(n_in));
    const GemvSeg seg = a.seg[blockIdx.y];
    const size_t row_bytes = a.n_seg_types ? seg.row_bytes : a.row_bytes;
    const int n_tiles = (seg.n_out + 15) >> 4;
    if ((int)blockIdx.x >= n_tiles) return; // (whole workgroup: a shorter matrix of a shared launch)
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    LaneCtx c;
    c.n = lane & 15; c.g = lane >> 4; c.ln = lane >> 2; c.lg = lane & 3;
    c.src_lane4 = 4 * (4 * c.n + c.g);
    c.am = lane & 15;
    c.smem = smem;
    c.pairs = reinterpret_cast<const XPair*>(smem + L::pairs_off(n_in));
    c.n_in = n_in;
    c.zero_off = L::zero_off(n_in);
    const unsigned char* const wbase[2] = {static_cast<const unsigned char*>(seg.w),
                                           static_cast<const unsigned char*>(DUAL ? a.w_up : seg.w)};
    // (rows past the end repeat the last one; nothing is written for them.  Blocks past a row's end: the
    // last block once more, never used.)
    auto request = [&](Raw (&r)[M], int tile, int b) {
        const int row = min(tile * 16 + c.ln, seg.n_out - 1);
        b = min(b, nb - 1);
#pragma unroll
        for (int m = 0; m < M; ++m) F::load(wbase[m] + (size_t)row * row_bytes + (size_t)(b0 + b) * F::kBlockBytes, c.lg, r[m]);
    };
    Raw raw_a[M], raw_b[M];
    request(raw_a, blockIdx.x, wave);
    __builtin_amdgcn_sched_barrier(0);

    const float rinv = stage_digits<F::kGroup, kWaves>(a, b0 << 8, n_in, smem, red);

    const typename F::Addr addr = F::addr(c);
    float rowacc[M];
    auto finish = [&](const Raw (&r)[M], int b) {
#pragma unroll
        for (int m = 0; m < M; ++m) rowacc[m] += F::block(r[m], c, addr, b);
    };
    // Row tiles blockIdx.x, + gridDim.x, ...: the digits are staged once per workgroup.  The first block of
    // the next tile is requested while the last of this one is multiplied out.
    for (int tile = blockIdx.x; tile < n_tiles; tile += gridDim.x) {
        const int next_tile = tile + (int)gridDim.x < n_tiles ? tile + (int)gridDim.x : tile;
#pragma unroll
        for (int m = 0; m < M; ++m) rowacc[m] = 0.0f;
        // (raw_a holds block `wave` of this tile)
        for (int b = wave;; b += 2 * kWaves) {
            const bool more1 = b + kWaves < nb;
            request(raw_b, more1 ? tile : next_tile, more1 ? b + kWaves : wave);
            if (b < nb) finish(raw_a, b);
            if (!more1) { // raw_b holds the next tile's first block: hand it over
#pragma unroll
                for (int m = 0; m < M; ++m) raw_a[m] = raw_b[m];
                break;
            }
            const bool more2 = b + 2 * kWaves < nb;
            request(raw_a, more2 ? tile : next_tile, more2 ? b + 2 * kWaves : wave);
            finish(raw_b, b + kWaves);
            if (!more2) break;
        }
        // ---- the four sub-block lanes of a row, then the four waves ----
        const int row0 = tile * 16;
#pragma unroll
        for (int m = 0; m < M; ++m) {
            const float t = xor_sum(rowacc[m]);
            if (c.g == 0) red[(wave * M + m) * 16 + c.n] = t;
        }
        __syncthreads();
        if (threadIdx.x < 16 && row0 + (int)threadIdx.x < seg.n_out) {
            const int r = row0 + threadIdx.x;
            float v[M];
#pragma unroll
            for (int m = 0; m < M; ++m) {
                v[m] = 0.0f;
#pragma unroll
                for (int w = 0; w < kWaves; ++w) v[m] += red[(w * M + m) * 16 + threadIdx.x];
                v[m] *= rinv;
            }
            float y = v[0];
            if constexpr (DUAL) y = y / (1.0f + expf(-y)) * v[1]; // SiLU(gate) * up
            if (gridDim.z > 1) { // (a share of the row: y already holds what is accumulated into)
                if (seg.bias && blockIdx.z == 0) y += seg.bias[r];
                atomicAdd(seg.y + r, y);
            } else {
                if (seg.bias) y += seg.bias[r];
                if (a.accumulate) y += seg.y[r];
                seg.y[r] = y;
            }
        }
        __syncthreads(); // (the partial sums are free for the next tile)
    }
}

template <int T, bool DUAL, int kWaves>
__global__ __launch_bounds__(kWaves * 64) void gemv_mfma_kernel(const GemvArgs a) {
    gemv_mfma_body<T, DUAL, kWaves>(a);
}

// Q4_K, Q5_K and Q6_K rows read in long runs.  The kernel above fetches, per load instruction, 64 bytes of each of
// 16 rows; this machine's memory path moves that pattern at 4.6-4.7 TB/s where lane-linear runs of two whole blocks
// of a row (288 bytes) move at 5.5-5.8 TB/s, as fast as a plain streaming read (the read-only stand-ins of
// bench_aids.hip over the 66 MB of a Llama-3-8B gate/up pair, `bench.py --workload weights-read-patterns`: 14.1-14.4
// us a launch against 11.5-12.0; runs of one block 13.5, of four blocks 17.9).  Here a wave's item is CB <= 2
// consecutive blocks of each of a tile's 16 rows, of one matrix, fetched as (row, 16-byte piece) slots in row-major
// order, lane after lane, with streaming loads: every line is asked for by one instruction.  The pieces pass
// through a wave-private LDS buffer (rows padded to an odd number of pieces, so that the 16 rows a
// matrix-instruction operand is read from lie in 16 different bank groups) and come back in the matrix
// instruction's lane order: no lane permutations.  Two items per wave are on their way or in use; chunks w, w +
// kWaves, ... of a tile's blocks are wave w's, and so are those chunks' digits of the activation, which the wave
// makes for itself: no wave waits for another before the first tile's end, where the norm's sum of squares is put
// together as well.  Barriers wait for LDS only, row sums leave through stores and atomic adds without a return
// value, a tile's bias values travel with its items: nothing in the loop waits for anything but the oldest item.
// Requires whole 16-row tiles.  (Deeper request queues, three and four items a wave, were slower in both kernels,
// and so were four-block items: what bounds the kernels after the loads is the vector ALU, about 74 instructions
// per block and wave for the nibbles, the six-bit pairs and the digit sums.)
constexpr int kRowsMaxCb = 2; // blocks of a row in an item, at most
constexpr int kRowsRedBytes = 2 * kMaxWaves * 2 * 16 * 4 + 64; // two sets of partial row sums (tiles alternate: one barrier a tile), the waves' sums of squares

template <int T, int CB>
struct RowsGeom {
    static constexpr int P = MF<T>::kPieces;                 // pieces of a block
    static constexpr int kRowPieces = CB * P;                // pieces of a row in an item
    static constexpr int R = kRowPieces | 1;                 // LDS row stride, pieces
    static constexpr int NL = (16 * kRowPieces + 63) / 64;   // load instructions an item
    static constexpr int kWaveBytes = (16 * R + 1) * 16;     // (one more piece: where lanes past the item's end write)
    static __host__ __device__ size_t lds_bytes(int n_in, int waves) {
        return (size_t)Lds<MF<T>::kGroup>::red_off(n_in) + kRowsRedBytes + (size_t)waves * kWaveBytes;
    }
};

template <int T, bool DUAL, int kWaves, int CB, bool kShortPrologue = false>
__device__ __forceinline__ void gemv_rows_body(const GemvArgs& a) {
    using F = MF<T>;
    using L = Lds<F::kGroup>;
    using G = RowsGeom<T, CB>;
    constexpr int M = DUAL ? 2 : 1, P = G::P, R = G::R, NL = G::NL;
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    ROWS_STAMP(0);
    const GemvSeg seg = a.seg[blockIdx.y];
    {
        // Every argument word the kernel reads, asked for here in one batch: left to the compiler the scalar loads
        // sit ahead of their uses, four dependent trips to the argument block before the first weight request.
        const int grid_x = gridDim.x;
        asm volatile("" ::"s"(seg.w), "s"(seg.bias), "s"(seg.y), "s"(seg.n_out), "s"(seg.row_bytes), "s"(a.w_up), "s"(a.x), "s"(a.norm_w),
                     "s"(a.eps), "s"(a.accumulate), "s"(a.row_bytes), "s"(a.n_seg_types), "s"(a.share_blocks), "s"(a.share_extra), "s"(grid_x));
    }
    // (this share's blocks of a row, from what the launcher divided: no division ahead of the first requests)
    const int b0 = (int)blockIdx.z * a.share_blocks + min((int)blockIdx.z, a.share_extra);
    const int nb = a.share_blocks + ((int)blockIdx.z < a.share_extra ? 1 : 0);
    const int n_in = nb << 8;
    float* const red = reinterpret_cast<float*>(smem + L::red_off(n_in));
    const unsigned row_bytes = (unsigned)(a.n_seg_types ? seg.row_bytes : a.row_bytes);
    const int n_tiles = seg.n_out >> 4;
    if ((int)blockIdx.x >= n_tiles) return; // (whole workgroup: a shorter matrix of a shared launch)
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6); // (scalar: what follows from it stays in scalar registers)
    unsigned char* const transit = smem + L::red_off(n_in) + kRowsRedBytes + wave * G::kWaveBytes;
    LaneCtx c;
    c.n = lane & 15; c.g = lane >> 4; c.ln = 0; c.lg = 0; c.src_lane4 = 0;
    c.am = lane & 15;
    c.smem = smem;
    c.pairs = reinterpret_cast<const XPair*>(smem + L::pairs_off(n_in));
    c.n_in = n_in;
    c.zero_off = L::zero_off(n_in);
    const unsigned char* const wbase[2] = {static_cast<const unsigned char*>(seg.w),
                                           static_cast<const unsigned char*>(DUAL ? a.w_up : seg.w)};
    const int n_chunks = (nb + CB - 1) / CB;
    const int my_chunks = wave < n_chunks ? (n_chunks - wave + kWaves - 1) / kWaves : 0;
    const int n_mine = n_tiles <= (int)gridDim.x ? 1 : (n_tiles - (int)blockIdx.x + (int)gridDim.x - 1) / (int)gridDim.x;
    const int total = n_mine * my_chunks * M;
    // slot 64 i + lane of an item: (row, piece), row-major
    unsigned goff[NL];
    int loff[NL];
#pragma unroll
    for (int i = 0; i < NL; ++i) {
        const int s = 64 * i + lane, row = s / G::kRowPieces, piece = s - row * G::kRowPieces, blk = piece / P;
        goff[i] = row < 16 ? (unsigned)row * row_bytes + (unsigned)(blk * F::kBlockBytes + F::piece_off(piece - blk * P)) : 0xffffffffu; // (past the end: cut to the item's last piece below)
        loff[i] = row < 16 ? (row * R + piece) * 16 : 16 * R * 16;
    }

    // ---- requests ----
    int rq_tile = blockIdx.x, rq_c = wave;
    constexpr int kRing = 2; // items on their way or in use (M divides it: an item's matrix is its slot's)
    u32x4 buf[kRing][NL];
    float bias_v[kRing];
    auto request = [&](u32x4 (&r)[NL], float& bias, int m) {
        const int cb = min(CB, nb - rq_c * CB);
        // pieces past the chunk's end in rows above the last are the row's next blocks or the next row's first (fetched,
        // never used); in the last row they are cut to the last piece
        const unsigned limit = 15u * row_bytes + (unsigned)((cb - 1) * F::kBlockBytes + F::piece_off(P - 1));
        const unsigned char* const base = wbase[m] + (size_t)rq_tile * 16 * row_bytes + (size_t)(b0 + rq_c * CB) * F::kBlockBytes;
#pragma unroll
        for (int i = 0; i < NL; ++i) {
            // whole runs, read once: streaming loads
            if constexpr (F::kAligned) r[i] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(base + min(goff[i], limit)));
            else r[i] = __builtin_nontemporal_load(reinterpret_cast<const u32x4_a2*>(base + min(goff[i], limit)));
        }
        bias = *(seg.bias ? seg.bias + rq_tile * 16 + c.n : a.x); // (always a load: the same count on every path)
        if (m == M - 1) {
            rq_c += kWaves;
            if (rq_c >= n_chunks) {
                rq_c = wave;
                rq_tile += (int)gridDim.x;
            }
        }
    };
    // ---- the activation's digits: every wave makes those of its own chunks (it multiplies no others), so
    // nothing waits for another wave before the first tile's end; the norm's sum of squares is put together
    // there.  The first chunk's loads go out ahead of the weight requests (loads return in order). ----
    float* const wave_ss = red + 2 * kMaxWaves * 2 * 16;
    {
        const float* const ax = a.x + (b0 << 8);
        const float* const aw = a.norm_w ? a.norm_w + (b0 << 8) : nullptr;
        XPair* const pairs = reinterpret_cast<XPair*>(smem + L::pairs_off(n_in));
        float ss = 0.0f;
        auto fetch = [&](const float* p, int e, float (&v)[8]) {
            *reinterpret_cast<float4*>(v) = *reinterpret_cast<const float4*>(p + e);
            *reinterpret_cast<float4*>(v + 4) = *reinterpret_cast<const float4*>(p + e + 4);
        };
        auto digits = [&](float (&x)[8], const float (&g)[8], int e) {
            if (aw) {
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    ss += x[i] * x[i];
                    x[i] *= g[i];
                }
            }
            digits8<F::kGroup>(x, e, n_in, smem, pairs, lane);
        };
        constexpr int kPasses = (CB * 256 + 511) / 512; // 512 elements a pass
        // The wave's first kPre chunks are fetched ahead of the weight requests: loads return in order, so fetched
        // behind them a chunk's few floats wait for two items of weights, and the wave's first item for all its
        // digits (the stage marks below, read in the timeline build: first digits 1.4 us after the requests, the second chunk's 2.1 us
        // later, the first item 0.5 us after that).
        constexpr int kPre = kWaves == 8 ? 2 : 4; // (eight-wave workgroups: fewer chunks a wave, and registers for four waves a SIMD)
        float xs[kPre][kPasses][8], gs[kPre][kPasses][8]; // (read under the conditions they are loaded under)
        if (kShortPrologue && kPasses == 1 && total >= kRing && my_chunks <= 2) {
            // One or two chunks and at least two items: nothing between the loads and their uses is under a
            // condition (a second chunk the wave does not have is fetched from the row's end and dropped), so the
            // compiler's waits are exact: the digits wait for the activation, not for the weights behind it, and
            // the first item is used as soon as it is there.  Only in the kernel for launches that leave resident places empty
            // (Qwen2.5-1.5B's gate/up 8.1 -> 7.4 us, its down projection 7.25 -> 6.9): a launch that fills the chip
            // runs 1.5 us longer this way, its second round of requests getting in the way of the first.  Not in
            // the kernels of eight waves and of mixed types either.
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                const int e = min((wave + i * kWaves) * CB * 256 + lane * 8, n_in - 8);
                fetch(ax, e, xs[i][0]);
                fetch(aw ? aw : ax, e, gs[i][0]);
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int j = 0; j < kRing; ++j) request(buf[j], bias_v[j], j % M);
            __builtin_amdgcn_sched_barrier(0);
            {
                const int e = wave * CB * 256 + lane * 8;
                if (e < min((wave + 1) * CB * 256, n_in)) digits(xs[0][0], gs[0][0], e);
            }
            if (my_chunks == 2) {
                const int e = (wave + kWaves) * CB * 256 + lane * 8;
                if (e < min((wave + kWaves + 1) * CB * 256, n_in)) digits(xs[1][0], gs[1][0], e);
            }
        } else {
#pragma unroll
        for (int i = 0; i < kPre; ++i) {
            const int ch = wave + i * kWaves, end = min((ch + 1) * CB * 256, n_in);
#pragma unroll
            for (int ps = 0; ps < kPasses; ++ps) {
                const int e = ch * CB * 256 + ps * 512 + lane * 8;
                if (e < end) { // (a chunk past the row's end starts past it)
                    fetch(ax, e, xs[i][ps]);
                    if (aw) fetch(aw, e, gs[i][ps]);
                }
            }
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int j = 0; j < kRing; ++j)
            if (j < total) request(buf[j], bias_v[j], j % M);
        __builtin_amdgcn_sched_barrier(0);
        ROWS_STAMP(1);
#pragma unroll
        for (int i = 0; i < kPre; ++i) {
            const int ch = wave + i * kWaves, end = min((ch + 1) * CB * 256, n_in);
#pragma unroll
            for (int ps = 0; ps < kPasses; ++ps) {
                const int e = ch * CB * 256 + ps * 512 + lane * 8;
                if (e < end) digits(xs[i][ps], gs[i][ps], e);
            }
        }
        for (int ch = wave + kPre * kWaves; ch < n_chunks; ch += kWaves) { // (rows longer still: these loads queue behind the weights)
            const int end = min((ch + 1) * CB * 256, n_in);
            for (int e = ch * CB * 256 + lane * 8; e < end; e += 512) {
                float x[8], g[8] = {};
                fetch(ax, e, x);
                if (aw) fetch(aw, e, g);
                digits(x, g, e);
            }
        }
        }
        if (lane < 4) reinterpret_cast<unsigned*>(smem + L::zero_off(n_in))[lane] = 0u; // (every wave writes the same zeros)
        ss = wave_sum(ss);
        if (lane == 0) wave_ss[wave] = ss;
    }
    ROWS_STAMP(2);
    [[maybe_unused]] int n_consumed = 0;
    const bool has_norm = a.norm_w != nullptr;
    const float norm_n = (float)n_in, norm_eps = a.eps;

    const typename F::Addr addr = F::addr(c);
    int set = 0;
    auto tile_end = [&](int tile, const float (&rowacc)[M], float bias) {
        float* const mine = red + set * (kMaxWaves * 2 * 16);
        set ^= 1;
#pragma unroll
        for (int m = 0; m < M; ++m) {
            const float t = xor_sum(rowacc[m]);
            if (c.g == 0) mine[(wave * M + m) * 16 + c.n] = t;
        }
        lds_barrier();
        if (threadIdx.x < 16) {
            const int r = tile * 16 + (int)threadIdx.x;
            float rinv = 1.0f;
            if (has_norm) { // (every wave has left its sum of squares before its first barrier here)
                float ss = 0.0f;
#pragma unroll
                for (int w = 0; w < kWaves; ++w) ss += wave_ss[w];
                rinv = 1.0f / sqrtf(ss / norm_n + norm_eps);
            }
            float v[M];
#pragma unroll
            for (int m = 0; m < M; ++m) {
                v[m] = 0.0f;
#pragma unroll
                for (int w = 0; w < kWaves; ++w) v[m] += mine[(w * M + m) * 16 + threadIdx.x];
                v[m] *= rinv;
            }
            float y = v[0];
            if constexpr (DUAL) y = y / (1.0f + expf(-y)) * v[1]; // SiLU(gate) * up
            if (seg.bias && blockIdx.z == 0) y += bias;
            if (gridDim.z > 1 || a.accumulate) atomicAdd(seg.y + r, y); // (one writer a row and share: with one share the sum is the plain one)
            else seg.y[r] = y;
        }
        ROWS_STAMP(13);
    };
    if (my_chunks == 0) { // (fewer chunks than waves: this wave only keeps the barriers' count)
        const float zero[M] = {};
        for (int t = 0; t < n_mine; ++t) tile_end((int)blockIdx.x + t * (int)gridDim.x, zero, 0.0f);
        return;
    }
    int cs_tile = blockIdx.x, cs_c = wave;
    float rowacc[M] = {};
    auto consume = [&](const u32x4 (&r)[NL], float bias, int m) {
#pragma unroll
        for (int i = 0; i < NL; ++i) *reinterpret_cast<u32x4*>(transit + loff[i]) = r[i];
        ROWS_ITEM_STAMP(3 + n_consumed);
        ++n_consumed;
        const int cb = min(CB, nb - cs_c * CB);
        // (unrolled over CB with a test per block, not a loop over cb: every LDS offset is a constant of its instruction)
        float v = F::from_lds(transit + c.n * R * 16, c, addr, cs_c * CB);
#pragma unroll
        for (int j = 1; j < CB; ++j)
            if (j < cb) v += F::from_lds(transit + (c.n * R + j * P) * 16, c, addr, cs_c * CB + j);
        rowacc[m] += v;
        if (m == M - 1) {
            cs_c += kWaves;
            if (cs_c >= n_chunks) {
                tile_end(cs_tile, rowacc, bias);
                cs_c = wave;
                cs_tile += (int)gridDim.x;
#pragma unroll
                for (int mm = 0; mm < M; ++mm) rowacc[mm] = 0.0f;
            }
        }
    };
    // Steady state: every item consumed is followed by the request kRing items on, which exists: no branch around
    // a load, so the compiler's wait counts are exact.
    int k = 0;
    for (; k + 2 * kRing <= total; k += kRing) {
#pragma unroll
        for (int j = 0; j < kRing; ++j) {
            consume(buf[j], bias_v[j], j % M);
            request(buf[j], bias_v[j], j % M);
        }
    }
    // the last two or three items (or the only one)
    if (k < total) consume(buf[0], bias_v[0], 0);
    if (k + 2 < total) request(buf[0], bias_v[0], 0);
    if (k + 1 < total) consume(buf[1], bias_v[1], M - 1);
    if (k + 2 < total) consume(buf[0], bias_v[0], 0);
    ROWS_STAMP(14);
}

// kShortPrologue: the kernel for launches that leave resident places empty (see the body's prologue): a kernel of
// its own, because the second path's code alone costs the launches that do not take it a microsecond.
template <int T, bool DUAL, int kWaves, int CB, bool kShortPrologue = false>
__global__ __launch_bounds__(kWaves * 64) void gemv_rows_kernel(const GemvArgs a) {
    gemv_rows_body<T, DUAL, kWaves, CB, kShortPrologue>(a);
}

// Matrices of different block types in one launch (the q, k, v projections of a file that keeps attn_v in
// Q6_K): a workgroup belongs to one matrix and runs that matrix's code.
template <int kWaves>
__global__ __launch_bounds__(kWaves * 64) void gemv_mfma_mixed_kernel(const GemvArgs a) {
    switch (a.seg[blockIdx.y].type) {
    case kQ4_K: gemv_mfma_body<kQ4_K, false, kWaves>(a); break;
    case kQ5_K: gemv_mfma_body<kQ5_K, false, kWaves>(a); break;
    case kQ6_K: gemv_mfma_body<kQ6_K, false, kWaves>(a); break;
    default: gemv_mfma_body<kQ8_0, false, kWaves>(a); break;
    }
}

// The same for the kernel that reads rows in long runs (no Q8_0 there).
template <int kWaves, int CB>
__global__ __launch_bounds__(kWaves * 64) void gemv_rows_mixed_kernel(const GemvArgs a) {
    switch (a.seg[blockIdx.y].type) {
    case kQ4_K: gemv_rows_body<kQ4_K, false, kWaves, CB>(a); break;
    case kQ5_K: gemv_rows_body<kQ5_K, false, kWaves, CB>(a); break;
    default: gemv_rows_body<kQ6_K, false, kWaves, CB>(a); break;
    }
}

constexpr size_t kMfmaLdsMax = 96u * 1024u;

template <int T>
size_t lds_bytes(int n_in) { return Lds<MF<T>::kGroup>::bytes(n_in); }

// The long-run kernel where it applies: Q4_K / Q5_K / Q6_K, whole 16-row tiles, LDS within the limit.
bool rows_enabled() {
    static const bool on = getenv("ORIN_GEMV_NO_ROWS") == nullptr;
    return on;
}
// Its workgroups per CU: three (staging is each wave's own business there, so a workgroup more costs little and
// hides more of the others' waits); ORIN_GEMV_MFMA_WGS_PER_CU overrides as for the other kernel.
int rows_wgs_per_cu(int given) {
    static const bool env = getenv("ORIN_GEMV_MFMA_WGS_PER_CU") != nullptr;
    return env ? given : 3;
}

int g_rows_resident = 768; // workgroups of four waves the chip holds at once (three a CU; set by the launcher)

template <int T, bool DUAL, int kWaves, int CB>
bool launch_rows_as(const GemvArgs& a, dim3 grid, int n_in_wg, hipStream_t stream) {
    const size_t lds = RowsGeom<T, CB>::lds_bytes(n_in_wg, kWaves);
    if (lds > kMfmaLdsMax) return false;
    GemvArgs b = a;
    b.share_blocks = (a.n_in / 256) / (int)grid.z;
    b.share_extra = (a.n_in / 256) % (int)grid.z;
    // (... and gives a wave one or two chunks: the other kernel's prologue serves more)
    b.few_workgroups = kWaves == 4 && (int)(grid.x * grid.y * grid.z) <= g_rows_resident * 3 / 4 && (n_in_wg / 256 + CB - 1) / CB <= 2 * kWaves;
    if constexpr (kWaves == 4) {
        if (b.few_workgroups) {
            hipLaunchKernelGGL((gemv_rows_kernel<T, DUAL, kWaves, CB, true>), grid, dim3(kWaves * 64), lds, stream, b);
            return true;
        }
    }
    hipLaunchKernelGGL((gemv_rows_kernel<T, DUAL, kWaves, CB>), grid, dim3(kWaves * 64), lds, stream, b);
    return true;
}

template <int T>
bool launch_rows(const GemvArgs& a, dim3 grid, bool wide, int nb_wg, hipStream_t stream) {
    if (!rows_enabled()) return false;
    for (int i = 0; i < a.n_seg; ++i)
        if (a.seg[i].n_out % 16 != 0) return false;
    const int n_in_wg = nb_wg * 256;
    if (wide) { // (eight waves: never two matrices)
        return (nb_wg + 7) / 8 <= 1 ? launch_rows_as<T, false, 8, 1>(a, grid, n_in_wg, stream)
                                    : launch_rows_as<T, false, 8, 2>(a, grid, n_in_wg, stream);
    }
    // runs of 288 (352) bytes read within a few percent of longer ones, and the wave's last item, which nothing
    // overlaps, is half as long as with four blocks
    const int cb = min(kRowsMaxCb, (nb_wg + 3) / 4);
    if (a.w_up) {
        return cb == 1 ? launch_rows_as<T, true, 4, 1>(a, grid, n_in_wg, stream) : launch_rows_as<T, true, 4, 2>(a, grid, n_in_wg, stream);
    }
    return cb == 1 ? launch_rows_as<T, false, 4, 1>(a, grid, n_in_wg, stream) : launch_rows_as<T, false, 4, 2>(a, grid, n_in_wg, stream);
}

template <int T>
hipError_t launch(const GemvArgs& a, int cu_count, hipStream_t stream) {
    int max_out = 0;
    for (int i = 0; i < a.n_seg; ++i) max_out = max(max_out, a.seg[i].n_out);
    const int cap = a.mfma_wgs_per_cu > 0 ? cu_count * a.mfma_wgs_per_cu : (max_out + 15) / 16;
    const dim3 grid(min((max_out + 15) / 16, cap), a.n_seg);
    dim3 g3 = grid;
    // A matrix with too few tiles to fill the chip whose rows are long, accumulating into y without a norm (output
    // and down projections): 2 or 4 workgroups share a tile's blocks, each staging its own part of the activation.
    const int nb_row = a.n_in / 256;
    int ks = 1;
    if (a.accumulate && !a.w_up && !a.norm_w && (int)(grid.x * grid.y) <= cu_count) ks = nb_row >= 32 ? 4 : nb_row >= 12 ? 2 : 1;
    if (a.k_split_override > 0) ks = a.accumulate && !a.w_up && !a.norm_w ? min(a.k_split_override, nb_row) : 1;
    g3.z = ks;
    // Eight waves a workgroup where a row has the blocks to share out and a workgroup has one tile only (a
    // second tile would have amortised the staging instead).
    const bool wide = ks == 1 && nb_row >= 16 && !a.w_up && (int)grid.x == (max_out + 15) / 16;
    if constexpr (T == kQ4_K || T == kQ5_K || T == kQ6_K) {
        const int per_cu = rows_wgs_per_cu(a.mfma_wgs_per_cu);
        g_rows_resident = cu_count * 3;
        dim3 gr = g3;
        gr.x = min((max_out + 15) / 16, per_cu > 0 ? cu_count * per_cu : (max_out + 15) / 16);
        // (its LDS buffers let three workgroups of four waves share a CU: no more shares of a row than are resident at once)
        int ks_r = ks;
        if (a.k_split_override <= 0) {
            if (ks == 1 && nb_row >= 6 && a.accumulate && !a.w_up && !a.norm_w && (int)(grid.x * grid.y) <= cu_count) ks_r = 2; // (shorter rows too: a share is cheap here)
            while (ks_r > 1 && (int)(gr.x * gr.y) * ks_r > cu_count * 3) ks_r /= 2;
        }
        gr.z = ks_r;
        const bool wide_r = ks_r == 1 && nb_row >= 16 && !a.w_up && (int)gr.x == (max_out + 15) / 16;
        if (launch_rows<T>(a, gr, wide_r, (nb_row + ks_r - 1) / ks_r, stream)) return hipGetLastError();
    }
    const size_t lds = lds_bytes<T>((nb_row + ks - 1) / ks * 256);
    if (a.w_up) {
        if (wide) hipLaunchKernelGGL((gemv_mfma_kernel<T, true, 8>), g3, dim3(512), lds, stream, a);
        else hipLaunchKernelGGL((gemv_mfma_kernel<T, true, 4>), g3, dim3(256), lds, stream, a);
    } else {
        if (wide) hipLaunchKernelGGL((gemv_mfma_kernel<T, false, 8>), g3, dim3(512), lds, stream, a);
        else hipLaunchKernelGGL((gemv_mfma_kernel<T, false, 4>), g3, dim3(256), lds, stream, a);
    }
    return hipGetLastError();
}

template <int T, bool DUAL>
hipError_t allow() {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&gemv_mfma_kernel<T, DUAL, 4>),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)kMfmaLdsMax);
    if (e != hipSuccess) return e;
    return hipFuncSetAttribute(reinterpret_cast<const void*>(&gemv_mfma_kernel<T, DUAL, 8>),
                               hipFuncAttributeMaxDynamicSharedMemorySize, (int)kMfmaLdsMax);
}

template <int T, bool DUAL, int kWaves, int CB>
hipError_t allow_rows() {
    if constexpr (kWaves == 4) {
        const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&gemv_rows_kernel<T, DUAL, kWaves, CB, true>),
                                                 hipFuncAttributeMaxDynamicSharedMemorySize, (int)kMfmaLdsMax);
        if (e != hipSuccess) return e;
    }
    return hipFuncSetAttribute(reinterpret_cast<const void*>(&gemv_rows_kernel<T, DUAL, kWaves, CB>),
                               hipFuncAttributeMaxDynamicSharedMemorySize, (int)kMfmaLdsMax);
}

template <int T>
hipError_t allow_rows_all() {
    hipError_t e;
    if ((e = allow_rows<T, false, 8, 1>()) != hipSuccess) return e;
    if ((e = allow_rows<T, false, 8, 2>()) != hipSuccess) return e;
    if ((e = allow_rows<T, false, 4, 1>()) != hipSuccess) return e;
    if ((e = allow_rows<T, false, 4, 2>()) != hipSuccess) return e;
    if ((e = allow_rows<T, true, 4, 1>()) != hipSuccess) return e;
    return allow_rows<T, true, 4, 2>();
}

} // namespace

// Every matrix of a block type (Q4_K, Q5_K, Q6_K, Q8_0), each its own type (GemvSeg::type, row_bytes filled in by the caller).
hipError_t gemv_mfma_mixed_launch(GemvArgs a, int cu_count, hipStream_t stream) {
    drop_stale_error();
    int max_out = 0;
    for (int i = 0; i < a.n_seg; ++i) max_out = max(max_out, a.seg[i].n_out);
    const int cap = a.mfma_wgs_per_cu > 0 ? cu_count * a.mfma_wgs_per_cu : (max_out + 15) / 16;
    const dim3 grid(min((max_out + 15) / 16, cap), a.n_seg);
    a.n_seg_types = 1;
    bool rows = rows_enabled();
    for (int i = 0; i < a.n_seg; ++i) rows = rows && a.seg[i].n_out % 16 == 0 && a.seg[i].type != kQ8_0;
    a.share_blocks = a.n_in / 256; // (one share: whole rows)
    a.share_extra = 0;
    a.few_workgroups = 0;
    if (rows) {
        const int per_cu = rows_wgs_per_cu(a.mfma_wgs_per_cu), nb = a.n_in / 256;
        const dim3 gr(min((max_out + 15) / 16, per_cu > 0 ? cu_count * per_cu : (max_out + 15) / 16), a.n_seg);
        const bool wide_r = nb >= 16 && (int)gr.x == (max_out + 15) / 16;
        // (the largest of the types' layouts: Q6_K's digits in groups of 16, Q5_K's 11 pieces a block are within Q6_K's 14)
        if (wide_r) {
            const size_t lds = RowsGeom<kQ6_K, 2>::lds_bytes(a.n_in, 8);
            if (lds <= kMfmaLdsMax) {
                if ((nb + 7) / 8 <= 1) hipLaunchKernelGGL((gemv_rows_mixed_kernel<8, 1>), gr, dim3(512), lds, stream, a);
                else hipLaunchKernelGGL((gemv_rows_mixed_kernel<8, 2>), gr, dim3(512), lds, stream, a);
                return hipGetLastError();
            }
        } else {
            const size_t lds = RowsGeom<kQ6_K, 2>::lds_bytes(a.n_in, 4);
            if (lds <= kMfmaLdsMax) {
                if ((nb + 3) / 4 <= 1) hipLaunchKernelGGL((gemv_rows_mixed_kernel<4, 1>), gr, dim3(256), lds, stream, a);
                else hipLaunchKernelGGL((gemv_rows_mixed_kernel<4, 2>), gr, dim3(256), lds, stream, a);
                return hipGetLastError();
            }
        }
    }
    const size_t lds = max(lds_bytes<kQ4_K>(a.n_in), lds_bytes<kQ6_K>(a.n_in));
    const bool wide = a.n_in / 256 >= 16 && (int)grid.x == (max_out + 15) / 16; // (as in launch() above)
    if (wide) hipLaunchKernelGGL((gemv_mfma_mixed_kernel<8>), grid, dim3(512), lds, stream, a);
    else hipLaunchKernelGGL((gemv_mfma_mixed_kernel<4>), grid, dim3(256), lds, stream, a);
    return hipGetLastError();
}

bool gemv_mfma_ok(int type, const GemvArgs& a) {
    if (a.n_in % 256 != 0) return false;
    if (type == kQ4_K || type == kQ5_K || type == kQ8_0) return lds_bytes<kQ4_K>(a.n_in) <= kMfmaLdsMax;
    if (type == kQ6_K) return lds_bytes<kQ6_K>(a.n_in) <= kMfmaLdsMax;
    return false;
}

hipError_t gemv_mfma_launch(int type, const GemvArgs& a, int cu_count, hipStream_t stream) {
    drop_stale_error();
    switch (type) {
    case kQ4_K: return launch<kQ4_K>(a, cu_count, stream);
    case kQ5_K: return launch<kQ5_K>(a, cu_count, stream);
    case kQ6_K: return launch<kQ6_K>(a, cu_count, stream);
    case kQ8_0: return launch<kQ8_0>(a, cu_count, stream);
    default: return hipErrorInvalidValue;
    }
}

// More than 64 KB of LDS per workgroup (rows longer than about 16k elements) needs to be allowed once.
hipError_t gemv_mfma_allow_lds() {
    hipError_t e;
    if ((e = allow<kQ4_K, false>()) != hipSuccess) return e;
    if ((e = allow<kQ4_K, true>()) != hipSuccess) return e;
    if ((e = allow<kQ6_K, false>()) != hipSuccess) return e;
    if ((e = allow<kQ6_K, true>()) != hipSuccess) return e;
    if ((e = allow<kQ5_K, false>()) != hipSuccess) return e;
    if ((e = allow<kQ5_K, true>()) != hipSuccess) return e;
    if ((e = allow<kQ8_0, false>()) != hipSuccess) return e;
    if ((e = allow<kQ8_0, true>()) != hipSuccess) return e;
    if ((e = allow_rows_all<kQ4_K>()) != hipSuccess) return e;
    if ((e = allow_rows_all<kQ5_K>()) != hipSuccess) return e;
    if ((e = allow_rows_all<kQ6_K>()) != hipSuccess) return e;
    if ((e = hipFuncSetAttribute(reinterpret_cast<const void*>(&gemv_rows_mixed_kernel<8, 1>), hipFuncAttributeMaxDynamicSharedMemorySize, (int)kMfmaLdsMax)) != hipSuccess) return e;
    if ((e = hipFuncSetAttribute(reinterpret_cast<const void*>(&gemv_rows_mixed_kernel<8, 2>), hipFuncAttributeMaxDynamicSharedMemorySize, (int)kMfmaLdsMax)) != hipSuccess) return e;
    if ((e = hipFuncSetAttribute(reinterpret_cast<const void*>(&gemv_rows_mixed_kernel<4, 1>), hipFuncAttributeMaxDynamicSharedMemorySize, (int)kMfmaLdsMax)) != hipSuccess) return e;
    if ((e = hipFuncSetAttribute(reinterpret_cast<const void*>(&gemv_rows_mixed_kernel<4, 2>), hipFuncAttributeMaxDynamicSharedMemorySize, (int)kMfmaLdsMax)) != hipSuccess) return e;
    if ((e = hipFuncSetAttribute(reinterpret_cast<const void*>(&gemv_mfma_mixed_kernel<8>),
                                 hipFuncAttributeMaxDynamicSharedMemorySize, (int)kMfmaLdsMax)) != hipSuccess) return e;
    return hipFuncSetAttribute(reinterpret_cast<const void*>(&gemv_mfma_mixed_kernel<4>),
                               hipFuncAttributeMaxDynamicSharedMemorySize, (int)kMfmaLdsMax);
}

hipError_t gemv_stamps(long long* host, size_t n) {
#ifdef ORIN_FA_STAMPS
    if (n > (size_t)kStampWgs * 4 * kStampSlots) return hipErrorInvalidValue;
    hipError_t e = hipMemcpyFromSymbol(host, HIP_SYMBOL(g_gemv_stamps), n * sizeof(long long)); // (synchronises with the device)
    void* dev = nullptr;
    if (e == hipSuccess) e = hipGetSymbolAddress(&dev, HIP_SYMBOL(g_gemv_stamps));
    if (e == hipSuccess) e = hipMemset(dev, 0, sizeof(g_gemv_stamps)); // the next launch starts from an empty table
    return e;
#else
    (void)host; (void)n;
    return hipErrorNotSupported;
#endif
}

} // namespace orin_fa
