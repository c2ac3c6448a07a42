// Host side of liborin_fa.so: library state, argument checks, launch-shape choice and the
// C ABI declared in include/orin_fa.h.  The kernels live in fa_prefill.hip and fa_decode.hip.
//
// Boundary: the reference's llm::cuda::flash_attention and flash_attention_decode_ind
// (reference: src/kernels.h:77-81, launchers at src/kernels.cu:1944-2000) and its KV-cache
// mutators kv_store_batch / kv_store_ind / kv_shift (src/kernels.h:66-73, src/kernels.cu:2079-2093) and the
// rotary embedding rope_{neox,normal}_{batch,ind} (src/kernels.h:55-62, src/kernels.cu:2059-2075).
#include "layer_common.hpp"

#include <stdio.h>

#include "../../include/orin_fa.h"
#ifdef ORIN_FA_STAMPS
#include "../../include/orin_fa_bench.h"
#endif

namespace orin_fa {
namespace {

// Split-KV partial results for orin_fa_decode_ind_static, the entry point that allocates nothing:
// a fixed block in the library's own device data.  Every GPU the library runs on holds its own
// copy at its own address until the process ends; that address is looked up once per device in
// orin_fa_init (the array's name is only a host-side handle: it is never passed to a kernel).
constexpr size_t kStaticScratchBytes = 2u << 20;
constexpr int kMaxDevices = 16;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];
// The activation that orin_quantize_activation stages for the *_q8 products (include/orin_layer.h),
// held the same way.
static __device__ __align__(256) float stage[kStageFloats];

struct State {
    bool ready = false;
    int device = 0;
    int cu_count = 0;
    hipStream_t stream = nullptr;
    void* own_ws = nullptr; // allocated by init, on device own_ws_device
    int own_ws_device = -1;
    void* ws = nullptr;     // active workspace
    size_t ws_bytes = 0;
    bool ws_is_own = false;
    void* static_ws[kMaxDevices] = {}; // device address of `scratch`, per device
    float* stage[kMaxDevices] = {};    // device address of `stage`, per device
};
State g_state;

inline int hip_code(hipError_t e) { return e == hipSuccess ? ORIN_FA_OK : ORIN_FA_E_HIP - (int)e; }

// The kernels take maxima over raw scores and scale afterwards, which needs a positive
// multiplier: the sign of `scale` moves into Q and a zero scale becomes a vanishing one.
inline void set_scale(FaArgs& a, float scale) {
    const float c = scale * kLog2e;
    a.qsign = c < 0.0f ? -1.0f : 1.0f;
    a.c = c < 0.0f ? -c : c;
    if (!(a.c >= 1e-30f)) a.c = 1e-30f;
}

size_t decode_bytes_per_split(int n_head, int head_dim) { return (size_t)n_head * (head_dim + 2) * sizeof(float); }

int decode_splits(int n_head, int n_kv, int head_dim, int n_ctx) {
    const int r = n_head / n_kv;
    const int n_hgroups = (r + 15) / 16;
    const int cus = g_state.cu_count > 0 ? g_state.cu_count : 256;
    int s = cus / (n_kv * n_hgroups); // one 8-wave workgroup per CU
    const int by_ctx = (n_ctx + kDecodeWaves * kTile - 1) / (kDecodeWaves * kTile);
    if (s > by_ctx) s = by_ctx;
    if (s > kMaxSplits) s = kMaxSplits;
    const size_t per_split = decode_bytes_per_split(n_head, head_dim);
    const size_t ws = g_state.ws ? g_state.ws_bytes : kWorkspaceBytes;
    if ((size_t)s * per_split > ws) s = (int)(ws / per_split);
    return s < 1 ? 1 : s;
}

int check_common(const void* q, const void* kc, const void* vc, const void* out,
                 int n_head, int n_kv, int head_dim, int n_ctx) {
    if (!g_state.ready) return ORIN_FA_E_NOT_INIT;
    if (!q || !kc || !vc || !out) return ORIN_FA_E_INVALID;
    if (n_head <= 0 || n_kv <= 0 || n_ctx <= 0 || n_head % n_kv != 0) return ORIN_FA_E_INVALID;
    if (head_dim != 64 && head_dim != 128) return ORIN_FA_E_HEAD_DIM;
    if ((long long)n_ctx * head_dim * 2 >= (1ll << 31)) return ORIN_FA_E_INVALID; // 32-bit byte offsets per KV head
    if ((reinterpret_cast<uintptr_t>(q) | reinterpret_cast<uintptr_t>(kc) | reinterpret_cast<uintptr_t>(vc) |
         reinterpret_cast<uintptr_t>(out)) & 15u)
        return ORIN_FA_E_INVALID; // 128-bit loads and stores
    return ORIN_FA_OK;
}

} // namespace

bool lib_ready() { return g_state.ready; }
int lib_cu_count() { return g_state.cu_count; }
hipStream_t lib_stream() { return g_state.stream; }
float* lib_stage() { return g_state.ready ? g_state.stage[g_state.device] : nullptr; }

} // namespace orin_fa

using namespace orin_fa;

extern "C" {

int orin_fa_init(int device) {
    hipError_t e = hipSetDevice(device);
    if (e != hipSuccess) {
        fprintf(stderr, "[orin_fa] hipSetDevice(%d) failed: %s\n", device, hipGetErrorString(e));
        return hip_code(e);
    }
    hipDeviceProp_t prop;
    e = hipGetDeviceProperties(&prop, device);
    if (e != hipSuccess) return hip_code(e);
    if (device < 0 || device >= kMaxDevices) return ORIN_FA_E_INVALID;
    g_state.ready = false;
    g_state.device = device;
    g_state.cu_count = prop.multiProcessorCount;
    if ((e = prefill_allow_lds()) != hipSuccess) return hip_code(e);
    if ((e = decode_allow_lds()) != hipSuccess) return hip_code(e);
    if ((e = gemv_mfma_allow_lds()) != hipSuccess) return hip_code(e);
    // The library's own workspace lives on the device it was last initialised for: a second init
    // on another device moves it there (the old block is released; graphs captured with it must
    // not be replayed any more, as after any change of workspace).
    if (g_state.own_ws && g_state.own_ws_device != device) {
        const bool active = g_state.ws_is_own;
        if (hipSetDevice(g_state.own_ws_device) == hipSuccess) (void)hipFree(g_state.own_ws);
        if ((e = hipSetDevice(device)) != hipSuccess) return hip_code(e);
        g_state.own_ws = nullptr;
        if (active) {
            g_state.ws = nullptr;
            g_state.ws_bytes = 0;
        }
    }
    if (!g_state.own_ws) {
        e = hipMalloc(&g_state.own_ws, kWorkspaceBytes);
        if (e != hipSuccess) return hip_code(e);
        g_state.own_ws_device = device;
    }
    if (!g_state.ws) {
        g_state.ws = g_state.own_ws;
        g_state.ws_bytes = kWorkspaceBytes;
        g_state.ws_is_own = true;
    }
    // This device's copy of the static scratch block: its address, once per device, with the
    // device current (each GPU holds the array at an address of its own).
    if (!g_state.static_ws[device]) {
        void* ptr = nullptr;
        e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
        if (e != hipSuccess) {
            fprintf(stderr, "[orin_fa] hipGetSymbolAddress(scratch) failed on device %d: %s\n", device, hipGetErrorString(e));
            return hip_code(e);
        }
        g_state.static_ws[device] = ptr;
    }
    if (!g_state.stage[device]) {
        void* ptr = nullptr;
        e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(stage));
        if (e != hipSuccess) {
            fprintf(stderr, "[orin_fa] hipGetSymbolAddress(stage) failed on device %d: %s\n", device, hipGetErrorString(e));
            return hip_code(e);
        }
        g_state.stage[device] = static_cast<float*>(ptr);
    }
    g_state.ready = true;
    return ORIN_FA_OK;
}

void orin_fa_set_stream(void* stream) { g_state.stream = static_cast<hipStream_t>(stream); }

size_t orin_fa_workspace_bytes(void) { return kWorkspaceBytes; }

int orin_fa_set_workspace(void* dev_ptr, size_t bytes) {
    if (!dev_ptr) { // back to the library's own block
        g_state.ws = g_state.own_ws;
        g_state.ws_bytes = g_state.own_ws ? kWorkspaceBytes : 0;
        g_state.ws_is_own = true;
        return ORIN_FA_OK;
    }
    if ((reinterpret_cast<uintptr_t>(dev_ptr) & 255u) != 0) return ORIN_FA_E_INVALID;
    if (bytes < kWorkspaceBytes) return ORIN_FA_E_WORKSPACE;
    g_state.ws = dev_ptr;
    g_state.ws_bytes = bytes;
    g_state.ws_is_own = false;
    return ORIN_FA_OK;
}

int orin_fa_prefill(const float* q, const uint16_t* kc, const uint16_t* vc, float* out,
                    int n_head, int n_kv, int head_dim, int n_ctx, int n_past, int batch, float scale) {
    int rc = check_common(q, kc, vc, out, n_head, n_kv, head_dim, n_ctx);
    if (rc != ORIN_FA_OK) return rc;
    if (batch < 0 || n_past < 0 || (long long)n_past + batch > n_ctx) return ORIN_FA_E_INVALID;
    if (batch == 0) return ORIN_FA_OK;
    if ((long long)batch * n_head * head_dim * 4 >= (1ll << 31)) return ORIN_FA_E_INVALID; // 32-bit byte offsets into q
    FaArgs a{};
    a.q = q; a.kc = kc; a.vc = vc; a.out = out;
    a.n_head = n_head; a.n_kv = n_kv; a.n_ctx = n_ctx; a.n_past = n_past; a.batch = batch;
    a.r = n_head / n_kv;
    a.n_splits = 1;
    set_scale(a, scale);
    return hip_code(prefill_launch(a, head_dim, g_state.cu_count, g_state.stream, g_state.ws, g_state.ws_bytes));
}

namespace {
struct RopeArgs {
    int n_rot;
    float theta;
    const float* freq_factors;
    int neox;
    const float* angles;
};
// partials: null = the active workspace; else a block of kStaticScratchBytes (the static scratch)
int decode_impl(const float* q, const uint16_t* kc, const uint16_t* vc, float* out, int n_head, int n_kv,
                int head_dim, int n_ctx, const int* d_pos, float scale,
                const float* k_new, const float* v_new, const RopeArgs* rope = nullptr, void* partials = nullptr);
}

int orin_fa_decode_ind(const float* q, const uint16_t* kc, const uint16_t* vc, float* out,
                       int n_head, int n_kv, int head_dim, int n_ctx, const int* d_pos, float scale) {
    return decode_impl(q, kc, vc, out, n_head, n_kv, head_dim, n_ctx, d_pos, scale, nullptr, nullptr);
}

int orin_fa_decode_ind_static(const float* q, const uint16_t* kc, const uint16_t* vc, float* out,
                              int n_head, int n_kv, int head_dim, int n_ctx, const int* d_pos, float scale) {
    if (!g_state.ready) return ORIN_FA_E_NOT_INIT;
    void* const block = g_state.static_ws[g_state.device]; // looked up in orin_fa_init; never the array's name
    if (!block) return ORIN_FA_E_NOT_INIT;
    return decode_impl(q, kc, vc, out, n_head, n_kv, head_dim, n_ctx, d_pos, scale, nullptr, nullptr, nullptr, block);
}

size_t orin_fa_static_scratch_bytes(void) { return kStaticScratchBytes; }

int orin_fa_decode_store_ind(const float* q, const float* k_new, const float* v_new, uint16_t* kc, uint16_t* vc,
                             float* out, int n_head, int n_kv, int head_dim, int n_ctx, const int* d_pos, float scale) {
    if (!k_new || !v_new) return ORIN_FA_E_INVALID;
    if (((reinterpret_cast<uintptr_t>(k_new) | reinterpret_cast<uintptr_t>(v_new)) & 15u) != 0) return ORIN_FA_E_INVALID;
    return decode_impl(q, kc, vc, out, n_head, n_kv, head_dim, n_ctx, d_pos, scale, k_new, v_new);
}

int orin_fa_rope_angles_ind(float* angles, int n_rot, float theta, const float* freq_factors, const int* d_pos) {
    if (!g_state.ready) return ORIN_FA_E_NOT_INIT;
    if (!angles || !d_pos || n_rot <= 0 || (n_rot & 1) || n_rot > 128) return ORIN_FA_E_INVALID; // (head_dim <= 128)
    if (reinterpret_cast<uintptr_t>(angles) & 7u) return ORIN_FA_E_INVALID;
    return hip_code(rope_angles_launch(angles, n_rot, theta, d_pos, freq_factors, g_state.stream));
}

int orin_fa_decode_rope_store_ind(const float* q, const float* k_new, const float* v_new, uint16_t* kc, uint16_t* vc,
                                  float* out, int n_head, int n_kv, int head_dim, int n_ctx, const int* d_pos, float scale,
                                  int n_rot, float theta, const float* freq_factors, int neox, const float* angles) {
    if (!k_new || !v_new) return ORIN_FA_E_INVALID;
    if (reinterpret_cast<uintptr_t>(angles) & 7u) return ORIN_FA_E_INVALID;
    if (((reinterpret_cast<uintptr_t>(k_new) | reinterpret_cast<uintptr_t>(v_new)) & 15u) != 0) return ORIN_FA_E_INVALID;
    if (n_rot < 0 || n_rot > head_dim || (n_rot & 1)) return ORIN_FA_E_INVALID;
    // the pairs must lie inside one lane's share of a row: always so for the "normal" pairing, and for
    // "neox" when the rotation spans the whole head
    if (neox && n_rot != 0 && n_rot != head_dim) return ORIN_FA_E_INVALID;
    const RopeArgs rope{n_rot, theta, freq_factors, neox != 0, angles};
    return decode_impl(q, kc, vc, out, n_head, n_kv, head_dim, n_ctx, d_pos, scale, k_new, v_new,
                       n_rot > 0 ? &rope : nullptr);
}

namespace {
int decode_impl(const float* q, const uint16_t* kc, const uint16_t* vc, float* out, int n_head, int n_kv,
                int head_dim, int n_ctx, const int* d_pos, float scale,
                const float* k_new, const float* v_new, const RopeArgs* rope, void* partials) {
    int rc = check_common(q, kc, vc, out, n_head, n_kv, head_dim, n_ctx);
    if (rc != ORIN_FA_OK) return rc;
    if (!d_pos) return ORIN_FA_E_INVALID;
    FaArgs a{};
    a.q = q; a.kc = kc; a.vc = vc; a.out = out; a.d_pos = d_pos;
    a.k_new = k_new; a.v_new = v_new;
    if (rope) {
        a.n_rot = rope->n_rot; a.theta = rope->theta; a.freq_factors = rope->freq_factors; a.neox = rope->neox;
        a.rope_angles = rope->angles;
    }
    a.n_head = n_head; a.n_kv = n_kv; a.n_ctx = n_ctx; a.batch = 1;
    a.r = n_head / n_kv;
    a.n_hgroups = (a.r + 15) / 16;
    a.n_splits = decode_splits(n_head, n_kv, head_dim, n_ctx);
    if (a.n_splits > 1) {
        if (partials) {
            // the fixed block takes the shape's usual number of splits or nothing: no quiet change of the launch
            if ((size_t)a.n_splits * decode_bytes_per_split(n_head, head_dim) > kStaticScratchBytes) {
                fprintf(stderr, "[orin_fa] orin_fa_decode_ind_static: %d splits x %d heads x head_dim %d need %zu bytes of "
                                "partial results, the static block holds %zu\n", a.n_splits, n_head, head_dim,
                        (size_t)a.n_splits * decode_bytes_per_split(n_head, head_dim), kStaticScratchBytes);
                return ORIN_FA_E_WORKSPACE;
            }
        } else if (!g_state.ws) {
            return ORIN_FA_E_WORKSPACE;
        }
        a.part_o = static_cast<float*>(partials ? partials : g_state.ws);
        a.part_ml = a.part_o + (size_t)a.n_splits * n_head * head_dim;
    }
    set_scale(a, scale);
    return hip_code(decode_launch(a, head_dim, g_state.stream));
}
} // namespace

int orin_fa_kv_store_batch(uint16_t* kc, uint16_t* vc, const float* k, const float* v,
                           int heads, int head_dim, int n_ctx, int pos_base, int batch) {
    if (!g_state.ready) return ORIN_FA_E_NOT_INIT;
    if (!kc || !vc || !k || !v) return ORIN_FA_E_INVALID;
    if (heads <= 0 || head_dim <= 0 || n_ctx <= 0 || batch < 0 || pos_base < 0) return ORIN_FA_E_INVALID;
    if ((long long)pos_base + batch > n_ctx) return ORIN_FA_E_INVALID;
    if (batch == 0) return ORIN_FA_OK;
    return hip_code(kv_store_launch(kc, vc, k, v, heads, head_dim, n_ctx, pos_base, batch, nullptr, g_state.stream));
}

int orin_fa_kv_store_ind(uint16_t* kc, uint16_t* vc, const float* k, const float* v,
                         int heads, int head_dim, int n_ctx, const int* d_pos) {
    if (!g_state.ready) return ORIN_FA_E_NOT_INIT;
    if (!kc || !vc || !k || !v || !d_pos) return ORIN_FA_E_INVALID;
    if (heads <= 0 || head_dim <= 0 || n_ctx <= 0) return ORIN_FA_E_INVALID;
    return hip_code(kv_store_launch(kc, vc, k, v, heads, head_dim, n_ctx, 0, 1, d_pos, g_state.stream));
}

int orin_fa_kv_shift(uint16_t* kc, uint16_t* vc, int n_layer, int n_kv, int head_dim, int n_ctx, int n_keep, int shift) {
    if (!g_state.ready) return ORIN_FA_E_NOT_INIT;
    if (!kc || !vc) return ORIN_FA_E_INVALID;
    if (n_layer <= 0 || n_kv <= 0 || head_dim <= 0 || n_ctx <= 0) return ORIN_FA_E_INVALID;
    if (n_keep < 0 || shift < 0 || (long long)n_keep + shift > n_ctx) return ORIN_FA_E_INVALID;
    if (shift == 0) return ORIN_FA_OK;
    return hip_code(kv_shift_launch(kc, vc, n_layer, n_kv, head_dim, n_ctx, n_keep, shift, g_state.stream));
}

int orin_fa_rope_batch(float* x, int rows, int head_dim, int n_rot, float theta, int n_past, int heads,
                       const float* freq_factors, int neox) {
    if (!g_state.ready) return ORIN_FA_E_NOT_INIT;
    if (!x) return ORIN_FA_E_INVALID;
    if (rows < 0 || head_dim <= 0 || heads <= 0 || n_past < 0 || rows % heads != 0) return ORIN_FA_E_INVALID;
    if (n_rot < 0 || n_rot > head_dim || (n_rot & 1)) return ORIN_FA_E_INVALID;
    if (rows == 0 || n_rot == 0) return ORIN_FA_OK;
    return hip_code(rope_launch(x, rows, head_dim, n_rot, theta, n_past, heads, nullptr, freq_factors, neox != 0, g_state.stream));
}

int orin_fa_rope_ind(float* x, int rows, int head_dim, int n_rot, float theta, const int* d_pos,
                     const float* freq_factors, int neox) {
    if (!g_state.ready) return ORIN_FA_E_NOT_INIT;
    if (!x || !d_pos) return ORIN_FA_E_INVALID;
    if (rows < 0 || head_dim <= 0) return ORIN_FA_E_INVALID;
    if (n_rot < 0 || n_rot > head_dim || (n_rot & 1)) return ORIN_FA_E_INVALID;
    if (rows == 0 || n_rot == 0) return ORIN_FA_OK;
    return hip_code(rope_launch(x, rows, head_dim, n_rot, theta, 0, rows, d_pos, freq_factors, neox != 0, g_state.stream));
}

int orin_fa_rope_store_batch(float* q, float* k, const float* v, uint16_t* kc, uint16_t* vc, int batch, int n_head,
                             int n_kv, int head_dim, int n_ctx, int n_past, int n_rot, float theta,
                             const float* freq_factors, int neox) {
    if (!g_state.ready) return ORIN_FA_E_NOT_INIT;
    if (!q || !k || !v || !kc || !vc) return ORIN_FA_E_INVALID;
    if (batch < 0 || n_head <= 0 || n_kv <= 0 || head_dim <= 0 || n_ctx <= 0 || n_past < 0) return ORIN_FA_E_INVALID;
    if (n_rot < 0 || n_rot > head_dim || (n_rot & 1)) return ORIN_FA_E_INVALID;
    if ((long long)n_past + batch > n_ctx) return ORIN_FA_E_INVALID;
    if (batch == 0) return ORIN_FA_OK;
    if (rope_store_fused_ok(q, k, v, kc, vc, head_dim, n_rot))
        return hip_code(rope_store_launch(q, k, v, kc, vc, batch, n_head, n_kv, head_dim, n_ctx, n_past, theta,
                                          freq_factors, neox != 0, g_state.stream));
    // any other shape: the three launches this call stands for
    if (n_rot > 0) {
        hipError_t e = rope_launch(q, batch * n_head, head_dim, n_rot, theta, n_past, n_head, nullptr, freq_factors,
                                   neox != 0, g_state.stream);
        if (e != hipSuccess) return hip_code(e);
        e = rope_launch(k, batch * n_kv, head_dim, n_rot, theta, n_past, n_kv, nullptr, freq_factors, neox != 0,
                        g_state.stream);
        if (e != hipSuccess) return hip_code(e);
    }
    return hip_code(kv_store_launch(kc, vc, k, v, n_kv, head_dim, n_ctx, n_past, batch, nullptr, g_state.stream));
}

#ifdef ORIN_FA_STAMPS
// Timeline build only (include/orin_fa_bench.h): the stage-mark tables of the kernels' last launches.
int orin_fa_bench_stamps(int which, long long* host, size_t n) {
    if (!g_state.ready) return ORIN_FA_E_NOT_INIT;
    if (!host || n == 0 || which < 0 || which > 2) return ORIN_FA_E_INVALID;
    return hip_code(which == 0 ? prefill_stamps(host, n) : which == 1 ? decode_stamps(host, n) : gemv_stamps(host, n));
}
#endif

int orin_fa_decode_splits(int n_head, int n_kv, int head_dim, int n_ctx) {
    if (n_head <= 0 || n_kv <= 0 || n_ctx <= 0 || n_head % n_kv != 0) return 0;
    if (head_dim != 64 && head_dim != 128) return 0;
    return decode_splits(n_head, n_kv, head_dim, n_ctx);
}

int orin_fa_cu_count(void) { return g_state.cu_count; }

int orin_fa_device_info(int device, char* name, size_t name_bytes, int* cu_count, size_t* total_mem) {
    hipDeviceProp_t prop;
    const hipError_t e = hipGetDeviceProperties(&prop, device);
    if (e != hipSuccess) return hip_code(e);
    if (name && name_bytes > 0) snprintf(name, name_bytes, "%s", prop.name);
    if (cu_count) *cu_count = prop.multiProcessorCount;
    if (total_mem) *total_mem = prop.totalGlobalMem;
    return ORIN_FA_OK;
}

const char* orin_fa_error_string(int code) {
    switch (code) {
        case ORIN_FA_OK: return "ok";
        case ORIN_FA_E_INVALID: return "invalid argument (shape, alignment or null pointer)";
        case ORIN_FA_E_HEAD_DIM: return "unsupported head_dim (64 and 128 only)";
        case ORIN_FA_E_WORKSPACE: return "split-KV workspace missing or too small";
        case ORIN_FA_E_NOT_INIT: return "orin_fa_init has not been called";
        default: break;
    }
    if (code <= ORIN_FA_E_HIP) return hipGetErrorString(static_cast<hipError_t>(ORIN_FA_E_HIP - code));
    return "unknown error";
}

} // extern "C"
