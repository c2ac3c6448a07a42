// Measurement aids of liborin_fa.so: kernels that are not part of the attention path but give
// the yardsticks its figures are read against.  Declared in include/orin_fa_bench.h.
#include "fa_common.hpp"

namespace orin_fa {
namespace {

// Plain streaming read: every thread issues PER 16-byte loads with the streaming hint (the
// decode kernel's kind of load), a grid stride apart, and folds them into a word that is
// stored only if it takes a value the data never produces, so the loads cannot be dropped.
template <int PER>
__global__ __launch_bounds__(512) void hbm_read_kernel(const u32x4* __restrict__ src, unsigned* sink, size_t n16) {
    const size_t stride = (size_t)gridDim.x * 512;
    const size_t i = (size_t)blockIdx.x * 512 + threadIdx.x;
    u32x4 r[PER];
#pragma unroll
    for (int k = 0; k < PER; ++k)
        r[k] = (i + k * stride < n16) ? __builtin_nontemporal_load(src + i + k * stride) : u32x4{0u, 0u, 0u, 0u};
    unsigned acc = 0;
#pragma unroll
    for (int k = 0; k < PER; ++k) acc ^= r[k].x ^ r[k].y ^ r[k].z ^ r[k].w;
    if (acc == 0x9E3779B9u) *sink = acc;
}

// The smallest launch there is: one wave that reads one word.
__global__ void tiny_kernel(const unsigned* src, unsigned* sink) {
    if (src[threadIdx.x & 1] == 0x9E3779B9u) *sink = 1;
}

} // namespace

hipError_t hbm_read_launch(const void* src, size_t bytes, int loads_per_thread, unsigned* sink, hipStream_t stream) {
    const size_t n16 = bytes / 16;
    const int per = loads_per_thread <= 2 ? 2 : loads_per_thread <= 4 ? 4 : loads_per_thread <= 8 ? 8 : 16;
    const size_t per_block = (size_t)512 * per;
    const unsigned grid = (unsigned)((n16 + per_block - 1) / per_block);
    if (grid == 0) return hipSuccess;
    const u32x4* p = static_cast<const u32x4*>(src);
    if (per == 2) hipLaunchKernelGGL(hbm_read_kernel<2>, dim3(grid), dim3(512), 0, stream, p, sink, n16);
    else if (per == 4) hipLaunchKernelGGL(hbm_read_kernel<4>, dim3(grid), dim3(512), 0, stream, p, sink, n16);
    else if (per == 8) hipLaunchKernelGGL(hbm_read_kernel<8>, dim3(grid), dim3(512), 0, stream, p, sink, n16);
    else hipLaunchKernelGGL(hbm_read_kernel<16>, dim3(grid), dim3(512), 0, stream, p, sink, n16);
    return hipGetLastError();
}

hipError_t tiny_launch(const unsigned* src, unsigned* sink, hipStream_t stream) {
    hipLaunchKernelGGL(tiny_kernel, dim3(1), dim3(64), 0, stream, src, sink);
    return hipGetLastError();
}

} // namespace orin_fa
