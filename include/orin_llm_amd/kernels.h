// The decode layer's slice of the orin_llm operator API -- attention, KV cache, rotary embedding, and the norms
// and quantised matrix-vector products around them -- with the reference's own signatures (reference:
// src/kernels.h:8-12, :15-47, :55-62, :66-73 and :77-81), implemented for MI355X by liborin_fa.so.  An engine
// built against the reference header links these symbols unchanged; each forwards to the C ABI in
// include/orin_fa.h and include/orin_layer.h and, like the reference's CUDA_CHECK (src/common.h:14-22), prints
// and abort()s on failure.
//
// Pointers are device pointers; kc / vc hold fp16 bit patterns laid out
// [kv_head][n_ctx][head_dim] for one layer; q / out are fp32 [batch][n_head][head_dim].
#pragma once

#include <stddef.h>
#include <stdint.h>

#ifndef ORIN_FA_SHIM_HAVE_DTYPE
// The weight types, numbered as ggml numbers them (reference: src/common.h:47-54).  An engine that includes
// its own common.h first defines ORIN_FA_SHIM_HAVE_DTYPE.
namespace llm {
enum class DType : uint32_t {
    F32  = 0,
    F16  = 1,
    Q8_0 = 8,
    Q4_K = 12,
    Q5_K = 13,
    Q6_K = 14,
};
} // namespace llm
#endif

namespace llm::cuda {

#ifndef ORIN_FA_SHIM_NO_PLUMBING
// Provided unless the engine's own operator layer already defines them; in that case
// build the shim with -DORIN_FA_SHIM_NO_PLUMBING and call orin_fa_init /
// orin_fa_set_stream from the engine's init / set_stream.
int init();
void device_info();
void set_stream(void* stream);
// The engine carves one block of device memory for the operator layer out of its activation allocation
// (reference: src/model_gpu.cu:175, 208).  Here that block holds the partial results of the attention
// kernels' KV splits (orin_fa_workspace_bytes(), whatever max_in and max_batch are); the staged activation
// of quantize_activation lives in the library's own device data.
size_t scratch_size(int max_in, int max_batch);
void scratch_assign(void* base, int max_in, int max_batch);
#endif

void quantize_activation(const float* x, int n_in);

void gemv(DType type, const void* W, const float* x, float* y, int n_in, int n_out);

void gemv_q8(DType type, const void* W, float* y, int n_in, int n_out);

void gemv_q8_bias(DType type, const void* W, const float* bias, float* y, int n_in, int n_out);

void gemv_q8_add(DType type, const void* W, float* y, int n_in, int n_out);

void gemv_fused_gate_up_swiglu(DType type, const void* Wg, const void* Wu,
                                float* out, int n_in, int n_out);

void dequant_row(DType type, const void* src, float* y, int n);

void rms_norm(const float* x, const float* w, int n, float eps, float* y);
void rms_norm_rows(const float* x, const float* w, int rows, int cols, float eps, float* y);

void swiglu(float* act, const float* gate, const float* up, int n);

void rope_neox_batch(float* x, int rows, int head_dim, int n_rot, float theta, int n_past, int heads, const float* freq_factors = nullptr);

void rope_normal_batch(float* x, int rows, int head_dim, int n_rot, float theta, int n_past, int heads, const float* freq_factors = nullptr);

void rope_neox_ind(float* x, int rows, int head_dim, int n_rot, float theta, const int* d_pos, const float* freq_factors = nullptr);

void rope_normal_ind(float* x, int rows, int head_dim, int n_rot, float theta, const int* d_pos, const float* freq_factors = nullptr);

void kv_store_batch(uint16_t* kc, uint16_t* vc, const float* k, const float* v,
                    int heads, int head_dim, int n_ctx, int pos_base, int batch);

void kv_store_ind(uint16_t* kc, uint16_t* vc, const float* k, const float* v,
                  int heads, int head_dim, int n_ctx, const int* d_pos);

void kv_shift(uint16_t* kc, uint16_t* vc, int n_layer, int n_kv, int head_dim, int n_ctx, int n_keep, int shift);

void flash_attention(const float* q, const uint16_t* kc, const uint16_t* vc, float* out,
                    int n_head, int n_kv, int head_dim, int n_ctx, int n_past, int batch, float scale);

void flash_attention_decode_ind(const float* q, const uint16_t* kc, const uint16_t* vc, float* out,
                                int n_head, int n_kv, int head_dim, int n_ctx, const int* d_pos, float scale);

} // namespace llm::cuda
