// Shared pieces of the gfx950 flash-attention kernels: vector types, launch arguments,
// wave-level helpers.  Included by fa_prefill.hip, fa_decode.hip and fa_api.hip only.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace orin_fa {

typedef _Float16 h8 __attribute__((ext_vector_type(8)));
typedef _Float16 h4 __attribute__((ext_vector_type(4)));
typedef __fp16 fp16x4 __attribute__((ext_vector_type(4)));
typedef float f4 __attribute__((ext_vector_type(4)));
typedef unsigned u32x2 __attribute__((ext_vector_type(2)));
typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
typedef int i32x4 __attribute__((ext_vector_type(4)));

constexpr int kPrefillWaves = 4; // waves per prefill workgroup (one per SIMD: the kernel fills the register file)
constexpr int kDecodeWaves = 8;  // waves per decode workgroup (two per SIMD, one workgroup per CU)
constexpr int kTile = 32;        // KV rows per wave tile
constexpr float kLog2e = 1.4426950408889634f;
// Softmax weights are computed against a reference maximum that is only moved when a score
// exceeds it by more than kLazy (log2 units), so the O accumulators are rescaled on a handful
// of early tiles instead of every tile.  P = 2^(s - m_ref + kPShift) therefore lies in
// (0, 2^(kLazy + kPShift)] = (0, 2^15], inside fp16 range and far enough above its subnormals
// that small weights keep their 11 bits; the common factor cancels in O / l.
constexpr float kLazy = 8.0f;
constexpr float kPShift = 7.0f;
constexpr int kMaxSplits = 256;                 // decode KV splits per KV head, at most
constexpr size_t kWorkspaceBytes = 8u << 20;    // split-KV partial results

struct FaArgs {
    const float* q;
    const uint16_t* kc;
    const uint16_t* vc;
    float* out;
    float* part_o;    // decode: [split][n_head][D]
    float* part_ml;   // decode: [n_head][split][2] = (reference maximum in log2 units, row sum)
    const int* d_pos; // decode only
    const float* k_new; // decode with store: the current token's K and V rows, fp32 [n_kv][head_dim];
    const float* v_new; // null for plain decode (the cache pointers are then never written through)
    const float* freq_factors; // decode with rotary embedding of q and k_new (n_rot > 0), as rope_launch takes them
    const float* rope_angles;  // optional: (cos, sin) of every pair at this token's position, [n_rot/2][2], from rope_angles_launch
    int n_rot, neox;
    float theta;
    int n_head, n_kv, n_ctx;
    int n_past, batch; // prefill only
    int r;             // query heads per KV head
    int n_hgroups;     // head groups per KV head
    int n_ttiles;      // prefill: token tiles
    int tq;            // prefill: tokens per token tile
    int tq_magic;      // prefill: 65536 / tq + 1 (division of a column index by tq as multiply and shift)
    int heads_per_group; // prefill: query heads per head group
    int n_splits;      // decode: KV splits
    int kv_split_shift; // prefill: log2 of the number of KV splits a token tile's rows are shared among (0: none);
                        // with splits, part_o [split][batch][n_head][D] and part_ml [split][batch][n_head] (log-sum-exp, log2
                        // units) receive what the combine kernel turns into out
    float c;           // |scale| * log2(e), clamped away from zero
    float qsign;       // sign of scale, folded into Q
};

// hipGetLastError() returns, and clears, the last error of any HIP call this host thread has made, the host
// application's own included.  Every launcher below starts by dropping what is pending, so that the code it
// returns after its launch is the launch's own and an unrelated stale error is not blamed on (and, through the
// llm::cuda shim, does not abort) an operator that worked.
inline void drop_stale_error() { (void)hipGetLastError(); }

// Launchers (defined next to their kernels).  All return hipError_t of the launch.
hipError_t prefill_launch(const FaArgs& args, int head_dim, int cu_count, hipStream_t stream, void* workspace,
                          size_t workspace_bytes);
hipError_t prefill_allow_lds();
hipError_t decode_launch(const FaArgs& args, int head_dim, hipStream_t stream);
hipError_t decode_allow_lds();

// KV-cache mutators (kv_cache.hip).  d_pos not null selects the single-token form that reads
// the position on the device.
hipError_t kv_store_launch(uint16_t* kc, uint16_t* vc, const float* k, const float* v, int heads, int head_dim,
                           int n_ctx, int pos_base, int batch, const int* d_pos, hipStream_t stream);
hipError_t kv_shift_launch(uint16_t* kc, uint16_t* vc, int n_layer, int n_kv, int head_dim, int n_ctx, int n_keep,
                           int shift, hipStream_t stream);

// Rotary embedding (rope.hip).  d_pos not null selects the single-token form.
hipError_t rope_launch(float* x, int rows, int head_dim, int n_rot, float theta, int n_past, int heads,
                       const int* d_pos, const float* freq_factors, bool neox, hipStream_t stream);
bool rope_store_fused_ok(const float* q, const float* k, const float* v, const uint16_t* kc, const uint16_t* vc,
                         int head_dim, int n_rot);
hipError_t rope_store_launch(float* q, float* k, const float* v, uint16_t* kc, uint16_t* vc, int tokens, int n_head,
                             int n_kv, int head_dim, int n_ctx, int n_past, float theta, const float* freq_factors,
                             bool neox, hipStream_t stream);
hipError_t rope_angles_launch(float* angles, int n_rot, float theta, const int* d_pos, const float* freq_factors,
                              hipStream_t stream);

// ---- timeline build (-DORIN_FA_STAMPS, liborin_fa_stamps.so; a measurement aid) ----
// The attention kernels carry FA_STAMP(i) marks at the ends of their stages.  In the ordinary
// library they are nothing.  In the timeline build lane 0 of every wave stores the 100 MHz
// wall clock there, into [workgroup][wave][kStampSlots] of a table that the bench reads back:
// medians over the waves of one launch say where a kernel's microseconds go.  The stores cost
// a little time themselves, so this library is never the one that is timed.
constexpr int kStampWgs = 1024, kStampSlots = 16;
#ifdef ORIN_FA_STAMPS
#define ORIN_FA_STAMP_STORE(table, waves, i)                                                                   \
    do {                                                                                                       \
        __builtin_amdgcn_sched_barrier(0);                                                                     \
        const unsigned fa_wg_ = blockIdx.x + gridDim.x * (blockIdx.y + gridDim.y * blockIdx.z);                \
        if ((threadIdx.x & 63) == 0 && fa_wg_ < (unsigned)orin_fa::kStampWgs)                                  \
            table[(fa_wg_ * (waves) + (threadIdx.x >> 6)) * orin_fa::kStampSlots + (i)] = wall_clock64();        \
        __builtin_amdgcn_sched_barrier(0);                                                                     \
    } while (0)
#endif
// Copies a kernel's table to the host (which: 0 prefill, 4 waves a workgroup; 1 decode split, 8 waves; 2 the
// matrix-vector kernel, 4 waves);
// hipErrorNotSupported in the ordinary library.
hipError_t prefill_stamps(long long* host, size_t n);
hipError_t decode_stamps(long long* host, size_t n);
hipError_t gemv_stamps(long long* host, size_t n); // the matrix-vector kernel that reads rows in long runs: waves 0-3 of a workgroup

template <int N>
struct IntC {
    static constexpr int value = N;
};
template <int I, int N, class F>
__device__ __forceinline__ void static_for(F&& f) {
    if constexpr (I < N) {
        f(IntC<I>{});
        static_for<I + 1, N>(f);
    }
}

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// All-reduce over the four 16-lane groups of a wave (lanes l, l^16, l^32, l^48) with the
// gfx950 lane-swap instructions: v_permlane32_swap exchanges the upper half of one register
// with the lower half of the other, v_permlane16_swap does the same for odd/even 16-lane rows.
__device__ __forceinline__ float xor_max(float v) {
    u32x2 s = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    v = fmaxf(__uint_as_float(s.x), __uint_as_float(s.y));
    s = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    return fmaxf(__uint_as_float(s.x), __uint_as_float(s.y));
}
__device__ __forceinline__ float xor_sum(float v) {
    u32x2 s = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    v = __uint_as_float(s.x) + __uint_as_float(s.y);
    s = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    return __uint_as_float(s.x) + __uint_as_float(s.y);
}

// Sums and maxima over the 64 lanes of a wave: inside rows of 16 by DPP moves, across the four rows by
// the lane-swap instructions; every lane ends up with the result.
__device__ __forceinline__ float dpp_xor_step(float v, int which) {
    // lane i <-> the lane whose index differs within its row of 16: 1, 2 (quad permutes), 7 - i within 8, 15 - i within 16
    const int x = __float_as_int(v);
    int y;
    if (which == 0) y = __builtin_amdgcn_update_dpp(x, x, 0xB1, 0xF, 0xF, false);       // quad_perm [1,0,3,2]
    else if (which == 1) y = __builtin_amdgcn_update_dpp(x, x, 0x4E, 0xF, 0xF, false);  // quad_perm [2,3,0,1]
    else if (which == 2) y = __builtin_amdgcn_update_dpp(x, x, 0x141, 0xF, 0xF, false); // row_half_mirror
    else y = __builtin_amdgcn_update_dpp(x, x, 0x140, 0xF, 0xF, false);                 // row_mirror
    return __int_as_float(y);
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int i = 0; i < 4; ++i) v = fmaxf(v, dpp_xor_step(v, i));
    return xor_max(v); // across the four rows of 16
}
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int i = 0; i < 4; ++i) v += dpp_xor_step(v, i);
    return xor_sum(v);
}

// 16-byte load through a buffer descriptor: the hardware returns zeros for offsets at or
// past the descriptor's byte count, so rows beyond the bound are never fetched and need no
// branch.
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
    const fp16x4 t = __builtin_amdgcn_ds_read_tr16_b64_v4f16((__attribute__((address_space(3))) fp16x4*)(p));
    return __builtin_bit_cast(h4, t);
}

// Orders this wave's LDS writes before its later LDS reads (lanes of one wave exchange
// data through the wave-private LDS slice).
__device__ __forceinline__ void wave_lds_sync() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// The rotary embedding's arithmetic, in one place for the kernels that apply it (rope.hip and the
// decode kernel that rotates its own q and k).  It follows the CPU statement (reference:
// src/model_cpu.cpp:179-203) operation by operation in fp32, without contraction into fused
// multiply-adds; the frequency is the double-precision power rounded to fp32, which is what a
// correctly rounded powf returns (at position 32768 one ulp of the frequency moves the angle by
// 2e-3 rad).
__device__ __forceinline__ float rope_freq_base(int i, int n_rot, float theta) {
#pragma clang fp contract(off)
    const float expo = -2.0f * (float)i / (float)n_rot;
    return (float)pow((double)theta, (double)expo);
}
__device__ __forceinline__ float rope_freq(int i, int n_rot, float theta, const float* freq_factors) {
    float f = rope_freq_base(i, n_rot, theta);
    if (freq_factors) f /= freq_factors[i];
    return f;
}
__device__ __forceinline__ void rope_rotate(float& x0, float& x1, float c, float s) {
#pragma clang fp contract(off)
    const float r0 = x0 * c - x1 * s;
    const float r1 = x0 * s + x1 * c;
    x0 = r0;
    x1 = r1;
}

} // namespace orin_fa
