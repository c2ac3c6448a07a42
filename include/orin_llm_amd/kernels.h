// The attention, KV-cache and rotary-embedding slice of the orin_llm operator API, with the reference's own
// signatures (reference: src/kernels.h:8-10, :55-62, :66-73 and :77-81), implemented for MI355X by
// liborin_fa.so.  An engine built against the reference header links these symbols
// unchanged; each forwards to the C ABI in include/orin_fa.h and, like the
// reference's CUDA_CHECK (src/common.h:14-22), prints and abort()s on failure.
//
// Pointers are device pointers; kc / vc hold fp16 bit patterns laid out
// [kv_head][n_ctx][head_dim] for one layer; q / out are fp32 [batch][n_head][head_dim].
#pragma once

#include <stddef.h>
#include <stdint.h>

namespace llm::cuda {

#ifndef ORIN_FA_SHIM_NO_PLUMBING
// Provided unless the engine's own operator layer already defines them; in that case
// build the shim with -DORIN_FA_SHIM_NO_PLUMBING and call orin_fa_init /
// orin_fa_set_stream from the engine's init / set_stream.
int init();
void set_stream(void* stream);
#endif

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
