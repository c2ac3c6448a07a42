/*
 * orin_fa -- C ABI of the MI355X (gfx950) GQA flash-attention path.
 *
 * This is the drop-in boundary for the two attention operators of the orin_llm
 * engine and the launch plumbing they need.  Every entry point takes plain
 * pointers and sizes; all data pointers are DEVICE pointers owned by the caller.
 * Launches are asynchronous on the stream given to orin_fa_set_stream (the null
 * stream by default); the caller synchronises.  The library keeps process-global
 * state (stream, workspace) exactly as the reference operator layer does
 * (reference: src/kernels.cu:1726-1728), so it is not re-entrant.
 *
 * Return convention: 0 on success, a negative ORIN_FA_E_* code otherwise
 * (orin_fa_error_string names it).  The C++ shim that carries the reference's own
 * signatures (include/orin_llm_amd/kernels.h) turns a non-zero code into
 * print + abort(), the reference's convention (src/common.h:14-22).
 *
 * Data formats (reference: src/kernels.h:77-81, src/kernels.cu:1675-1677):
 *   q, out   fp32, [batch][n_head][head_dim] (batch = 1 for decode)
 *   kc, vc   IEEE binary16 bit patterns in uint16_t, one layer's cache,
 *            element (kv_head, pos, i) at (kv_head * n_ctx + pos) * head_dim + i
 *   GQA map  query head h reads KV head h / (n_head / n_kv)
 * Alignment: q, out, kc, vc (and k_new, v_new) of the attention entry points must be 16-byte
 * aligned (ORIN_FA_E_INVALID otherwise; the reference accepts any alignment of its element
 * types); the KV-cache mutators and the rotary embedding accept any alignment.
 */
#ifndef ORIN_FA_H
#define ORIN_FA_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum {
    ORIN_FA_OK = 0,
    ORIN_FA_E_INVALID = -1,      /* bad shape or null pointer */
    ORIN_FA_E_HEAD_DIM = -2,     /* head_dim not in {64, 128} (reference: assert, src/kernels.cu:1979,1998) */
    ORIN_FA_E_WORKSPACE = -3,    /* no workspace, or too small for this shape */
    ORIN_FA_E_NOT_INIT = -4,     /* orin_fa_init has not succeeded */
    ORIN_FA_E_HIP = -1000        /* -(1000 + hipError_t) for runtime failures */
};

/* Replaces llm::cuda::init (reference: src/kernels.h:8, src/kernels.cu:1730-1737).
 * Selects the device, reads its CU count and allocates the default split-KV
 * workspace once.  Must be called before any launch and outside stream capture. */
int orin_fa_init(int device);

/* Replaces llm::cuda::set_stream (reference: src/kernels.h:10, src/kernels.cu:1728).
 * stream is a hipStream_t; NULL selects the null stream. */
void orin_fa_set_stream(void* stream);

/* Replace the attention share of llm::cuda::scratch_size / scratch_assign
 * (reference: src/kernels.h:11-12, src/kernels.cu:1753-1776): the bytes of device
 * scratch the decode path needs for its split-KV partial results, and the call that
 * points the library at a caller-owned block of at least that size (256-byte
 * aligned).  Optional: orin_fa_init already allocates a block of this size.
 * orin_fa_prefill uses the same block when it cuts a long context's KV rows among
 * workgroups (few query columns, 3072 rows or more): launches that use the block must
 * not overlap, which one stream guarantees.  The block's address is baked into a captured
 * graph like every other pointer argument: set the workspace before capturing, keep the
 * block alive while the graph may be replayed, and capture again after changing it (a second
 * orin_fa_init on another device releases the library's own block and allocates it there). */
size_t orin_fa_workspace_bytes(void);
int orin_fa_set_workspace(void* dev_ptr, size_t bytes);

/* Replaces llm::cuda::flash_attention (reference: src/kernels.h:77-78,
 * src/kernels.cu:1974-1981): causal GQA attention for a chunk of `batch` query
 * tokens at cache positions [n_past, n_past + batch).  Token b attends to cache
 * positions [0, n_past + b]; the cache must already hold the chunk's own K/V
 * (call site: src/model_gpu.cu:383-384).  Writes every (token < batch, head, i). */
int orin_fa_prefill(const float* q, const uint16_t* kc, const uint16_t* vc, float* out,
                    int n_head, int n_kv, int head_dim, int n_ctx, int n_past, int batch, float scale);

/* Replaces llm::cuda::flash_attention_decode_ind (reference: src/kernels.h:80-81,
 * src/kernels.cu:1993-2000): one query token attending to cache positions
 * [0, *d_pos]; d_pos is a DEVICE pointer read by the kernel, so the call is safe
 * under stream capture and the captured graph can be replayed after the position
 * changes (call site: src/model_gpu.cu:281-282, 295-316).  Performs no allocation,
 * no synchronisation and no host read of *d_pos; the launch shape depends only on
 * the arguments passed by value. */
int orin_fa_decode_ind(const float* q, const uint16_t* kc, const uint16_t* vc, float* out,
                       int n_head, int n_kv, int head_dim, int n_ctx, const int* d_pos, float scale);

/* orin_fa_decode_ind for callers that cannot allocate and cannot hand over a workspace (code
 * under HIP graph capture that never saw orin_fa_set_workspace, tight serving loops, harnesses
 * that forbid hipMalloc).  No counterpart in the reference.  Same arguments, same kernels and
 * bit-identical output, but the split-KV partial results live in a fixed block inside the
 * library's own device data (orin_fa_static_scratch_bytes() = 2 MiB per GPU, held until the
 * process ends) instead of the workspace.  The call allocates and frees nothing.  A shape whose
 * partial results (splits x n_head x (head_dim + 2) x 4 bytes, splits = orin_fa_decode_splits)
 * exceed the block returns ORIN_FA_E_WORKSPACE with a message on stderr and launches nothing.
 * Every call on a GPU shares that GPU's block: calls that overlap on one GPU (two streams) race;
 * calls on one stream do not.  Nothing in the block has to start at zero. */
int orin_fa_decode_ind_static(const float* q, const uint16_t* kc, const uint16_t* vc, float* out,
                              int n_head, int n_kv, int head_dim, int n_ctx, const int* d_pos, float scale);
size_t orin_fa_static_scratch_bytes(void);

/* Replace llm::cuda::rope_neox_batch / rope_normal_batch (neox != 0 / == 0) and rope_neox_ind /
 * rope_normal_ind (reference: src/kernels.h:55-62, src/kernels.cu:1619-1657, 2059-2075; CPU statement
 * src/model_cpu.cpp:179-203): rotary position embedding in place on fp32 rows x[rows][head_dim].
 * Pair i of a row turns by pos * theta^(-2i/n_rot) (divided by freq_factors[i] when freq_factors is
 * not NULL; n_rot/2 floats on the device); elements at or past n_rot are untouched.
 * Batch form: row = token * heads + head, pos = n_past + token (call site src/model_gpu.cu:379-381).
 * Single-token form: every row is a head of the one token whose position is read from device
 * memory (capture-safe; call site src/model_gpu.cu:277-279). */
int orin_fa_rope_batch(float* x, int rows, int head_dim, int n_rot, float theta, int n_past, int heads,
                       const float* freq_factors, int neox);
int orin_fa_rope_ind(float* x, int rows, int head_dim, int n_rot, float theta, const int* d_pos,
                     const float* freq_factors, int neox);

/* The three calls a prefill layer makes ahead of its attention -- rope_*_batch on the Q rows,
 * rope_*_batch on the K rows, kv_store_batch (reference call sites: src/model_gpu.cu:378-382)
 * -- as one call; no counterpart in the reference.  q [batch][n_head][head_dim] and
 * k [batch][n_kv][head_dim] are rotated in place, k and v [batch][n_kv][head_dim] go to cache
 * positions [n_past, n_past + batch): memory ends up exactly as after the three calls.  One
 * launch when n_rot = head_dim (a multiple of 8) and all pointers are 16-byte aligned, else
 * the three launches. */
int orin_fa_rope_store_batch(float* q, float* k, const float* v, uint16_t* kc, uint16_t* vc, int batch, int n_head,
                             int n_kv, int head_dim, int n_ctx, int n_past, int n_rot, float theta,
                             const float* freq_factors, int neox);

/* Replaces llm::cuda::kv_store_batch (reference: src/kernels.h:66-67, src/kernels.cu:1659-1678,
 * 2079-2083; CPU statement src/model_cpu.cpp:276-279): rounds the fp32 K and V rows of `batch`
 * tokens (k, v: [batch][heads][head_dim]) to binary16, nearest-even, into cache positions
 * [pos_base, pos_base + batch) of one layer's caches.  This is the step that runs right before
 * orin_fa_prefill at the call site (src/model_gpu.cu:378-384).  Any head_dim is accepted. */
int orin_fa_kv_store_batch(uint16_t* kc, uint16_t* vc, const float* k, const float* v,
                           int heads, int head_dim, int n_ctx, int pos_base, int batch);

/* Replaces llm::cuda::kv_store_ind (reference: src/kernels.h:69-70, src/kernels.cu:2085-2088):
 * the same for one token whose position is read from device memory (capture-safe; call site
 * src/model_gpu.cu:276-282).  A position outside [0, n_ctx) stores nothing. */
int orin_fa_kv_store_ind(uint16_t* kc, uint16_t* vc, const float* k, const float* v,
                         int heads, int head_dim, int n_ctx, const int* d_pos);

/* Replaces llm::cuda::kv_shift (reference: src/kernels.h:72-73, src/kernels.cu:1682-1700, 2090-2093;
 * CPU statement src/model_cpu.cpp:321-338; policy src/engine.cpp:231-235): over the WHOLE cache
 * (kc, vc: [n_layer][n_kv][n_ctx][head_dim] each), per layer and head, rows [n_keep + shift, n_ctx)
 * move to [n_keep, n_ctx - shift) and the last `shift` rows are cleared, in place. */
int orin_fa_kv_shift(uint16_t* kc, uint16_t* vc, int n_layer, int n_kv, int head_dim, int n_ctx, int n_keep, int shift);

/* orin_fa_kv_store_ind followed by orin_fa_decode_ind, in the launches of the latter alone.
 * No counterpart in the reference, whose decode layer makes the two calls back to back
 * (src/model_gpu.cu:281-282; kv_store_ind src/kernels.cu:2084-2088): k_new, v_new are the
 * current token's rows, fp32 [n_kv][head_dim], 16-byte aligned.  The workgroup whose tile
 * holds row *d_pos takes the row from them, rounded to fp16 exactly as the store rounds, and
 * writes it to the cache; cache contents and output equal those of the two calls bit for bit
 * (a position outside [0, n_ctx) stores nothing and attends as orin_fa_decode_ind does).
 * Capture-safe like orin_fa_decode_ind. */
int orin_fa_decode_store_ind(const float* q, const float* k_new, const float* v_new, uint16_t* kc, uint16_t* vc,
                             float* out, int n_head, int n_kv, int head_dim, int n_ctx, const int* d_pos, float scale);

/* The decode layer's four calls around the cache -- rope_*_ind on q, rope_*_ind on the new K row,
 * kv_store_ind, flash_attention_decode_ind (reference: src/model_gpu.cu:277-282) -- in the
 * launches of the last alone.  No counterpart in the reference.  q [n_head][head_dim] and k_new
 * [n_kv][head_dim] arrive BEFORE the rotary embedding and are left as they are; every workgroup
 * rotates what it needs with the arithmetic of orin_fa_rope_ind (n_rot, theta, freq_factors,
 * neox as there), so the cache contents and the output equal those of the four calls bit for
 * bit.  Supported: the "normal" pairing with any even n_rot <= head_dim, the "neox" pairing
 * with n_rot = head_dim (or n_rot = 0: no rotation); anything else returns ORIN_FA_E_INVALID and
 * the separate calls apply.  Capture-safe like orin_fa_decode_ind.
 * angles: NULL, or the table orin_fa_rope_angles_ind wrote for the same n_rot, theta,
 * freq_factors and *d_pos (theta and freq_factors are then not used): every layer of a decode
 * step rotates by the same angles, and with the table no workgroup spends its first
 * microsecond and a half on the powers, sines and cosines.  Same results bit for bit. */
int orin_fa_decode_rope_store_ind(const float* q, const float* k_new, const float* v_new, uint16_t* kc, uint16_t* vc,
                                  float* out, int n_head, int n_kv, int head_dim, int n_ctx, const int* d_pos, float scale,
                                  int n_rot, float theta, const float* freq_factors, int neox, const float* angles);

/* (cos, sin) of the n_rot/2 rotary pairs at position *d_pos (read on the device), as
 * orin_fa_rope_ind forms them, into angles [n_rot/2][2] (device, 8-byte aligned).  No
 * counterpart in the reference, whose kernels recompute them per element pair
 * (src/kernels.cu:1619-1657); for orin_fa_decode_rope_store_ind, once per token. */
int orin_fa_rope_angles_ind(float* angles, int n_rot, float theta, const float* freq_factors, const int* d_pos);

/* Introspection for tests and benchmarks: the number of KV splits a decode launch
 * with these shapes uses (0 if the shape is rejected), and the CU count seen at init. */
int orin_fa_decode_splits(int n_head, int n_kv, int head_dim, int n_ctx);
int orin_fa_cu_count(void);

/* What llm::cuda::device_info prints (reference: src/kernels.h:9, src/kernels.cu:1739-1744): the name of a
 * device (NUL-terminated, cut to name_bytes), its compute units and its memory in bytes.  Any of the three
 * outputs may be NULL.  Needs no orin_fa_init. */
int orin_fa_device_info(int device, char* name, size_t name_bytes, int* cu_count, size_t* total_mem);

/* Human-readable name of a return code. */
const char* orin_fa_error_string(int code);

#ifdef __cplusplus
}
#endif
#endif
