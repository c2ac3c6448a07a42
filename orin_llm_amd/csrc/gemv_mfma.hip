// Matrix-vector products over Q4_K weight rows on the matrix cores of gfx950 (MI355X).
//
// The vector-ALU kernel of gemv.hip spends about three instructions per weight (byte to float,
// multiply-add, unpacking) and is bound by them at twice the time HBM needs for the bytes.  Here
// the multiply-adds run as integer matrix instructions and the vector ALU only splits nibbles and
// applies the blocks' scales:
//
//   * The activation is cut, per 32-element sub-block, into three signed 8-bit digits of a 24-bit
//     integer, x = s (65536 d0 + 256 d1 + d2) with s = max|x| / (2^23 - 2^16): what the reference
//     does with one digit (quantize_q8_1_k, reference: src/kernels.cu:136-157), carried to the
//     precision of an fp32 mantissa.  Every workgroup builds the digits once, in LDS (together
//     with the RMS norm, when that is folded in), with the sub-blocks' scales and sums beside them.
//   * v_mfma_i32_16x16x64_i8 then multiplies 16 weight rows by 64 elements at a time: the weights'
//     nibbles, widened to bytes, are the B operand exactly as a lane loaded them (lane (n, g) holds
//     16 bytes of row n), and the A operand's rows are (sub-block, digit) pairs, each row zero
//     outside its own sub-block.  One accumulator therefore holds, for a row of weights, the exact
//     integer sums of four sub-blocks against the three digits, already separated: lane (n, g)
//     receives the three sums of sub-block g.  They are recombined in fp32 and multiplied by the
//     sub-block's scales, d * scale * sum - dmin * min * sum(x) (reference CPU statement:
//     src/model_cpu.cpp:70-89).
//   * The four waves of a workgroup take every fourth 256-element block of the same 16 rows and meet
//     in LDS at the end; blocks are requested one iteration ahead.
#include "layer_common.hpp"

namespace orin_fa {
namespace {

constexpr int kWaves = 4;
constexpr float kDigitRange = 8388608.0f - 65536.0f; // largest |integer| the three signed digits hold

struct XPair {
    float scale, sum; // of one 32-element sub-block of the activation
};

// LDS: digit planes [3][n_in] | XPair [n_in / 32] | 16 zero bytes | partial row sums [waves][M][16]
__device__ __forceinline__ int lds_pairs_off(int n_in) { return 3 * n_in; }
__device__ __forceinline__ int lds_zero_off(int n_in) { return 3 * n_in + (n_in >> 5) * 8; }
__device__ __forceinline__ int lds_red_off(int n_in) { return lds_zero_off(n_in) + 16; }

// Digits of the (optionally normalised) activation into LDS.  Thread t takes elements 8 t .. 8 t + 7
// of every 2048; the four threads of a sub-block meet by DPP moves inside their quad.
__device__ void stage_digits(const GemvArgs& a, unsigned char* smem, float* red) {
    const int n_in = a.n_in, tid = threadIdx.x;
    float rinv = 1.0f;
    if (a.norm_w) {
        float ss = 0.0f;
        for (int e = tid * 8; e < n_in; e += kWaves * 64 * 8) {
            const float4 u = *reinterpret_cast<const float4*>(a.x + e), v = *reinterpret_cast<const float4*>(a.x + e + 4);
            ss += u.x * u.x + u.y * u.y + u.z * u.z + u.w * u.w + v.x * v.x + v.y * v.y + v.z * v.z + v.w * v.w;
        }
        ss = wave_sum(ss);
        if ((tid & 63) == 0) red[tid >> 6] = ss;
        __syncthreads();
        ss = red[0] + red[1] + red[2] + red[3];
        __syncthreads();
        rinv = 1.0f / sqrtf(ss / (float)n_in + a.eps);
    }
    XPair* pairs = reinterpret_cast<XPair*>(smem + lds_pairs_off(n_in));
    for (int e = tid * 8; e < n_in; e += kWaves * 64 * 8) {
        float x[8];
        *reinterpret_cast<float4*>(x) = *reinterpret_cast<const float4*>(a.x + e);
        *reinterpret_cast<float4*>(x + 4) = *reinterpret_cast<const float4*>(a.x + e + 4);
        if (a.norm_w) {
            float g[8];
            *reinterpret_cast<float4*>(g) = *reinterpret_cast<const float4*>(a.norm_w + e);
            *reinterpret_cast<float4*>(g + 4) = *reinterpret_cast<const float4*>(a.norm_w + e + 4);
#pragma unroll
            for (int i = 0; i < 8; ++i) x[i] = x[i] * rinv * g[i];
        }
        float mx = 0.0f, sum = 0.0f;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            mx = fmaxf(mx, fabsf(x[i]));
            sum += x[i];
        }
        // the sub-block's four threads are one quad (n_in is a multiple of 32, so a quad is never split)
        mx = fmaxf(mx, dpp_xor_step(mx, 0));
        mx = fmaxf(mx, dpp_xor_step(mx, 1));
        sum += dpp_xor_step(sum, 0);
        sum += dpp_xor_step(sum, 1);
        const float scale = mx > 0.0f ? mx / kDigitRange : 1.0f;
        const float inv = 1.0f / scale;
        unsigned d0[2] = {0, 0}, d1[2] = {0, 0}, d2[2] = {0, 0};
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const int X = (int)rintf(x[i] * inv);
            const int lo = ((X + 128) & 255) - 128;
            const int X1 = (X - lo) >> 8;
            const int mid = ((X1 + 128) & 255) - 128;
            const int hi = (X1 - mid) >> 8;
            d0[i >> 2] |= (unsigned)(hi & 255) << (8 * (i & 3));
            d1[i >> 2] |= (unsigned)(mid & 255) << (8 * (i & 3));
            d2[i >> 2] |= (unsigned)(lo & 255) << (8 * (i & 3));
        }
        *reinterpret_cast<u32x2*>(smem + e) = u32x2{d0[0], d0[1]};
        *reinterpret_cast<u32x2*>(smem + n_in + e) = u32x2{d1[0], d1[1]};
        *reinterpret_cast<u32x2*>(smem + 2 * n_in + e) = u32x2{d2[0], d2[1]};
        if ((tid & 3) == 0) pairs[e >> 5] = XPair{scale, sum};
    }
    if (tid < 4) reinterpret_cast<unsigned*>(smem + lds_zero_off(n_in))[tid] = 0u;
    __syncthreads();
}

struct Q4Raw {
    u32x4 hdr, q1, q2; // a block's header and this lane's 16 bytes of each half of its nibbles
};

// DUAL: two matrices (gate, up) and SiLU(gate) * up.  Grid: (workgroups, matrices); a workgroup walks the
// 16-row tiles blockIdx.x, + gridDim.x, ...
template <bool DUAL>
__global__ __launch_bounds__(kWaves * 64) void gemv_q4k_mfma_kernel(const GemvArgs a) {
    constexpr int M = DUAL ? 2 : 1;
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    const int n_in = a.n_in, nb = n_in >> 8;
    float* const red = reinterpret_cast<float*>(smem + lds_red_off(n_in));
    const GemvSeg seg = a.seg[blockIdx.y];
    const int n_tiles = (seg.n_out + 15) >> 4;
    if ((int)blockIdx.x >= n_tiles) return; // (whole workgroup: a shorter matrix of a shared launch)
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int n = lane & 15, g = lane >> 4;
    const unsigned char* const wbase[2] = {static_cast<const unsigned char*>(seg.w),
                                           static_cast<const unsigned char*>(DUAL ? a.w_up : seg.w)};
    // (rows past the end repeat the last one; nothing is written for them.  Blocks past a row's end: the
    // last block once more, never used.)
    // Loads are made with four neighbouring lanes on 64 consecutive bytes of a row (lane = 4 * row + piece:
    // the vector cache then sees 16 runs per instruction; with the matrix instruction's own lane order,
    // lane = row + 16 * piece, it sees 64 separate 16-byte requests and the kernel runs 10 % slower) and
    // moved to the matrix instruction's lanes by one lane permutation per register afterwards.
    const int ln = lane >> 2, lg = lane & 3;
    const int src_lane4 = 4 * (4 * n + g); // (byte address of the lane that loaded what lane (n, g) multiplies)
    auto request = [&](Q4Raw (&r)[M], int tile, int b) {
        const int row = min(tile * 16 + ln, seg.n_out - 1);
        b = min(b, nb - 1);
#pragma unroll
        for (int m = 0; m < M; ++m) {
            const unsigned char* blk = wbase[m] + (size_t)row * a.row_bytes + (size_t)b * 144;
            r[m].hdr = *reinterpret_cast<const u32x4*>(blk);
            r[m].q1 = *reinterpret_cast<const u32x4*>(blk + 16 + 16 * lg);
            r[m].q2 = *reinterpret_cast<const u32x4*>(blk + 80 + 16 * lg);
        }
    };
    Q4Raw raw_a[M], raw_b[M];
    request(raw_a, blockIdx.x, wave);
    __builtin_amdgcn_sched_barrier(0);

    stage_digits(a, smem, red);

    // As a lane of the A operand: row m = 4 p + digit of an accumulator covers sub-block p of the four
    // that a 128-element half of a block holds; this lane's 16 elements belong to sub-block
    // 2 (g / 2) (their low nibbles) and 2 (g / 2) + 1 (their high nibbles).
    const int am = lane & 15, ap = am >> 2, ad = am & 3;
    const bool a_live = ad < 3 && (ap >> 1) == (g >> 1);
    const int zero_off = lds_zero_off(n_in);
    // (byte offsets into LDS; lanes whose row is zero here read the 16 zero bytes, with stride 0)
    const int a_elem = 64 * (g >> 1) + 16 * (g & 1);
    const int a_lo_base = a_live && (ap & 1) == 0 ? ad * n_in + a_elem : zero_off;
    const int a_hi_base = a_live && (ap & 1) == 1 ? ad * n_in + a_elem + 32 : zero_off;
    const int a_lo_step = a_live && (ap & 1) == 0 ? 256 : 0, a_hi_step = a_live && (ap & 1) == 1 ? 256 : 0;
    const XPair* const pairs = reinterpret_cast<const XPair*>(smem + lds_pairs_off(n_in));

    float rowacc[M];
    auto finish = [&](const Q4Raw (&r)[M], int b) {
        i32x4 alo[2], ahi[2];
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            alo[h] = *reinterpret_cast<const i32x4*>(smem + a_lo_base + b * a_lo_step + (a_lo_step ? 128 * h : 0));
            ahi[h] = *reinterpret_cast<const i32x4*>(smem + a_hi_base + b * a_hi_step + (a_hi_step ? 128 * h : 0));
        }
        const XPair xp[2] = {pairs[8 * b + g], pairs[8 * b + 4 + g]};
#pragma unroll
        for (int m = 0; m < M; ++m) {
            // (the loading lane holds piece lg of row ln, and lane (n, g) wants piece g of row n: the bytes
            // of the packed pairs it needs are bytes lg of the loading lane's three words)
            const unsigned mine = ((r[m].hdr.y >> (8 * lg)) & 0xffu) | (((r[m].hdr.z >> (8 * lg)) & 0xffu) << 8) |
                                  (((r[m].hdr.w >> (8 * lg)) & 0xffu) << 16);
            const unsigned dd = (unsigned)__builtin_amdgcn_ds_bpermute(src_lane4, (int)r[m].hdr.x);
            const unsigned bb = (unsigned)__builtin_amdgcn_ds_bpermute(src_lane4, (int)mine);
            const float d = (float)__builtin_bit_cast(_Float16, (uint16_t)(dd & 0xffffu));
            const float dmin = (float)__builtin_bit_cast(_Float16, (uint16_t)(dd >> 16));
            const unsigned b0 = bb & 0xffu, b1 = (bb >> 8) & 0xffu, b2 = (bb >> 16) & 0xffu;
            // pairs g (first half of the block) and 4 + g (second half) of the twelve packed bytes
            const float sc[2] = {(float)(b0 & 63u), (float)((b2 & 0x0fu) | ((b0 >> 6) << 4))};
            const float mn[2] = {(float)(b1 & 63u), (float)((b2 >> 4) | ((b1 >> 6) << 4))};
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                const u32x4 qs = h ? r[m].q2 : r[m].q1;
                i32x4 lo, hi;
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const unsigned q = (unsigned)__builtin_amdgcn_ds_bpermute(src_lane4, (int)qs[i]);
                    lo[i] = (int)(q & 0x0f0f0f0fu);
                    hi[i] = (int)((q >> 4) & 0x0f0f0f0fu);
                }
                i32x4 acc = {0, 0, 0, 0};
                acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(alo[h], lo, acc, 0, 0, 0);
                acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(ahi[h], hi, acc, 0, 0, 0);
                const float t = ((float)acc[0] * 256.0f + (float)acc[1]) * 256.0f + (float)acc[2];
                rowacc[m] += (d * sc[h]) * (t * xp[h].scale) - (dmin * mn[h]) * xp[h].sum;
            }
        }
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
            if (g == 0) red[(wave * M + m) * 16 + n] = t;
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
            }
            float y = v[0];
            if constexpr (DUAL) y = y / (1.0f + expf(-y)) * v[1]; // SiLU(gate) * up
            if (seg.bias) y += seg.bias[r];
            if (a.accumulate) y += seg.y[r];
            seg.y[r] = y;
        }
        __syncthreads(); // (the partial sums are free for the next tile)
    }
}

} // namespace

bool gemv_q4k_mfma_ok(const GemvArgs& a) {
    const size_t lds = 3u * a.n_in + (a.n_in / 32) * 8u + 16u + kWaves * 2 * 16 * 4u;
    return a.n_in % 256 == 0 && lds <= 64u * 1024u;
}

hipError_t gemv_q4k_mfma_launch(const GemvArgs& a, int cu_count, hipStream_t stream) {
    int max_out = 0;
    for (int i = 0; i < a.n_seg; ++i) max_out = max(max_out, a.seg[i].n_out);
    const int cap = a.mfma_wgs_per_cu > 0 ? cu_count * a.mfma_wgs_per_cu : (max_out + 15) / 16;
    const dim3 grid(min((max_out + 15) / 16, cap), a.n_seg);
    const size_t lds = 3u * a.n_in + (a.n_in / 32) * 8u + 16u + kWaves * 2 * 16 * 4u;
    if (a.w_up)
        hipLaunchKernelGGL((gemv_q4k_mfma_kernel<true>), grid, dim3(kWaves * 64), lds, stream, a);
    else
        hipLaunchKernelGGL((gemv_q4k_mfma_kernel<false>), grid, dim3(kWaves * 64), lds, stream, a);
    return hipGetLastError();
}

} // namespace orin_fa
