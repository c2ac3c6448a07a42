// The two mutators of the fp16 KV cache for gfx950 (MI355X): the fp32 -> fp16 row store that
// runs right before attention, and the rolling-window shift.
//
// Replaces the reference's kv_store_k / kv_shift_k and their wrappers (reference:
// src/kernels.cu:1659-1700, 2079-2093; CPU statement of the same operations:
// src/model_cpu.cpp:276-279, 321-338).  Cache layout as everywhere: element (head, pos, i) of
// one layer at (head * n_ctx + pos) * head_dim + i, fp16 bit patterns in uint16_t; the whole
// cache is n_layer such blocks for K, and the same again for V.
//
// Both are pure byte movers, bound by HBM:
//   * store: one thread converts 8 consecutive fp32 values (two 16-byte loads) with
//     round-to-nearest-even and writes one 16-byte piece of a cache row; K and V are handled
//     by the two halves of the grid.  The reference launches one 256-thread block per row with
//     2-byte stores.  The "ind" form reads the position on the device, so the launch can be
//     captured in a graph.
//   * shift: rows [n_keep + shift, n_ctx) move down by `shift` rows and the last `shift` rows are
//     cleared, in place.  Row p only ever takes the value of row p + shift, so the rows of one
//     residue class (p - n_keep) mod shift form a chain that one thread walks front to back
//     (load p + shift, store p), and different chains never touch the same bytes: the grid is
//     one thread per 16-byte piece of every chain head -- (layers x {K,V} x heads x shift rows x
//     head_dim/8) threads, every access a full coalesced row -- where the reference walks each
//     column of a head with a single thread.
#include "fa_common.hpp"

namespace orin_fa {
namespace {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));

// VEC = 8: head_dim is a multiple of 8 (16-byte cache pieces); VEC = 1: any head_dim.
template <int VEC, bool IND>
__global__ __launch_bounds__(256) void kv_store_kernel(uint16_t* kc, uint16_t* vc, const float* k, const float* v,
                                                       int heads, int head_dim, int n_ctx, int pos_base, int batch,
                                                       const int* d_pos) {
    const int per_row = head_dim / VEC;                       // threads per (token, head) row
    const long long rows = (long long)batch * heads;
    const long long idx = (long long)blockIdx.x * 256 + threadIdx.x;
    const bool is_v = idx >= rows * per_row;                  // second half of the grid stores V
    const long long j = is_v ? idx - rows * per_row : idx;
    if (j >= rows * per_row) return;
    const long long row = j / per_row;                        // = token * heads + head
    const int piece = (int)(j % per_row);
    const int head = (int)(row % heads);
    const int pos = IND ? *d_pos : pos_base + (int)(row / heads);
    if (pos < 0 || pos >= n_ctx) return;                      // (the reference would write out of bounds)
    const float* src = (is_v ? v : k) + row * head_dim + piece * VEC;
    uint16_t* dst = (is_v ? vc : kc) + ((size_t)head * n_ctx + pos) * head_dim + piece * VEC;
    if constexpr (VEC == 8) {
        const float4 x0 = *reinterpret_cast<const float4*>(src);
        const float4 x1 = *reinterpret_cast<const float4*>(src + 4);
        half8 h;
        h[0] = (_Float16)x0.x; h[1] = (_Float16)x0.y; h[2] = (_Float16)x0.z; h[3] = (_Float16)x0.w;
        h[4] = (_Float16)x1.x; h[5] = (_Float16)x1.y; h[6] = (_Float16)x1.z; h[7] = (_Float16)x1.w;
        // (streaming store: the row is read next by another kernel, from other compute units)
        __builtin_nontemporal_store(h, reinterpret_cast<half8*>(dst));
    } else {
        const _Float16 h = (_Float16)src[0];
        dst[0] = __builtin_bit_cast(uint16_t, h);
    }
}

// One thread per 16-byte piece of a chain head.  PIECE = bytes per thread (16, or 2 when
// head_dim is not a multiple of 8).
template <int PIECE>
__global__ __launch_bounds__(256) void kv_shift_kernel(uint16_t* kc, uint16_t* vc, long long strips, int row_bytes,
                                                       int n_ctx, int n_keep, int shift) {
    typedef unsigned piece_t __attribute__((ext_vector_type(PIECE == 16 ? 4 : 1)));
    const int per_row = row_bytes / PIECE;
    const long long per_strip = (long long)shift * per_row;   // chain heads of one (layer, head) strip, times pieces
    const long long idx = (long long)blockIdx.x * 256 + threadIdx.x;
    const bool is_v = idx >= strips * per_strip;
    const long long j = is_v ? idx - strips * per_strip : idx;
    if (j >= strips * per_strip) return;
    const long long strip = j / per_strip;                    // = layer * n_kv + head
    const int rem = (int)(j % per_strip);
    const int residue = rem / per_row, piece = rem % per_row;
    unsigned char* base = reinterpret_cast<unsigned char*>(is_v ? vc : kc) + (size_t)strip * n_ctx * row_bytes +
                          (size_t)piece * PIECE;
    int p = n_keep + residue;
    if (p >= n_ctx) return;
    for (; p + shift < n_ctx; p += shift) {
        if constexpr (PIECE == 16) {
            const piece_t x = *reinterpret_cast<const piece_t*>(base + (size_t)(p + shift) * row_bytes);
            __builtin_nontemporal_store(x, reinterpret_cast<piece_t*>(base + (size_t)p * row_bytes));
        } else {
            const uint16_t x = *reinterpret_cast<const uint16_t*>(base + (size_t)(p + shift) * row_bytes);
            *reinterpret_cast<uint16_t*>(base + (size_t)p * row_bytes) = x;
        }
    }
    // p is now the chain's row in the last `shift` rows: cleared
    if constexpr (PIECE == 16) *reinterpret_cast<piece_t*>(base + (size_t)p * row_bytes) = piece_t{0u, 0u, 0u, 0u};
    else *reinterpret_cast<uint16_t*>(base + (size_t)p * row_bytes) = 0;
}

} // namespace

hipError_t kv_store_launch(uint16_t* kc, uint16_t* vc, const float* k, const float* v, int heads, int head_dim,
                           int n_ctx, int pos_base, int batch, const int* d_pos, hipStream_t stream) {
    drop_stale_error();
    const bool vec = head_dim % 8 == 0 &&
                     ((reinterpret_cast<uintptr_t>(kc) | reinterpret_cast<uintptr_t>(vc) |
                       reinterpret_cast<uintptr_t>(k) | reinterpret_cast<uintptr_t>(v)) & 15u) == 0;
    const long long threads = 2ll * batch * heads * (head_dim / (vec ? 8 : 1));
    const unsigned grid = (unsigned)((threads + 255) / 256);
    if (grid == 0) return hipSuccess;
    if (vec) {
        if (d_pos) hipLaunchKernelGGL((kv_store_kernel<8, true>), dim3(grid), dim3(256), 0, stream, kc, vc, k, v, heads, head_dim, n_ctx, 0, 1, d_pos);
        else hipLaunchKernelGGL((kv_store_kernel<8, false>), dim3(grid), dim3(256), 0, stream, kc, vc, k, v, heads, head_dim, n_ctx, pos_base, batch, nullptr);
    } else {
        if (d_pos) hipLaunchKernelGGL((kv_store_kernel<1, true>), dim3(grid), dim3(256), 0, stream, kc, vc, k, v, heads, head_dim, n_ctx, 0, 1, d_pos);
        else hipLaunchKernelGGL((kv_store_kernel<1, false>), dim3(grid), dim3(256), 0, stream, kc, vc, k, v, heads, head_dim, n_ctx, pos_base, batch, nullptr);
    }
    return hipGetLastError();
}

hipError_t kv_shift_launch(uint16_t* kc, uint16_t* vc, int n_layer, int n_kv, int head_dim, int n_ctx, int n_keep,
                           int shift, hipStream_t stream) {
    drop_stale_error();
    const int row_bytes = head_dim * 2;
    const bool vec = row_bytes % 16 == 0 &&
                     ((reinterpret_cast<uintptr_t>(kc) | reinterpret_cast<uintptr_t>(vc)) & 15u) == 0;
    const long long strips = (long long)n_layer * n_kv;
    const long long threads = 2ll * strips * shift * (row_bytes / (vec ? 16 : 2));
    const long long blocks = (threads + 255) / 256;
    if (blocks == 0) return hipSuccess;
    if (blocks > 0x7fffffffll) return hipErrorInvalidValue;
    if (vec) hipLaunchKernelGGL((kv_shift_kernel<16>), dim3((unsigned)blocks), dim3(256), 0, stream, kc, vc, strips, row_bytes, n_ctx, n_keep, shift);
    else hipLaunchKernelGGL((kv_shift_kernel<2>), dim3((unsigned)blocks), dim3(256), 0, stream, kc, vc, strips, row_bytes, n_ctx, n_keep, shift);
    return hipGetLastError();
}

} // namespace orin_fa
