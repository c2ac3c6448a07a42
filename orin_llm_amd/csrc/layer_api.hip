// Host side of the decode-layer operators declared in include/orin_layer.h: argument checks,
// the staged activation, and the launch sequence of a whole layer.
//
// Boundary: the reference's llm::cuda operators that its decode_layer calls around attention
// (reference: src/kernels.h:15-47, launchers src/kernels.cu:1778-1836, 1944-1954, 2004-2044;
// call sequence src/model_gpu.cu:251-293).
#include "layer_common.hpp"

#include <stdio.h>

#include "../../include/orin_fa.h"
#include "../../include/orin_layer.h"

namespace orin_fa {
namespace {

int g_staged_n = -1; // elements of the last staged activation

inline int hip_rc(hipError_t e) { return e == hipSuccess ? ORIN_FA_OK : ORIN_FA_E_HIP - (int)e; }
inline bool aligned(const void* p, unsigned a) { return (reinterpret_cast<uintptr_t>(p) & (a - 1)) == 0; }

int check_matrix(int type, const void* w, int n_in, int n_out) {
    if (!w || n_in <= 0 || n_out <= 0 || n_in > kMaxGemvIn || n_in % 32 != 0) return ORIN_FA_E_INVALID;
    if (weight_row_bytes(type, n_in) == 0) return ORIN_FA_E_INVALID;
    if (!aligned(w, (unsigned)weight_align(type))) return ORIN_FA_E_INVALID;
    return ORIN_FA_OK;
}

// One launch: n_mat matrices of one type over x.
int gemv_call(int type, int n_mat, const void* const* w, const float* const* bias, float* const* y, const int* n_out,
              const void* w_up, const float* x, const float* norm_w, float eps, int n_in, int accumulate) {
    if (!lib_ready()) return ORIN_FA_E_NOT_INIT;
    if (n_mat < 1 || n_mat > 3 || !x || !aligned(x, 16) || (norm_w && !aligned(norm_w, 16))) return ORIN_FA_E_INVALID;
    GemvArgs a{};
    for (int i = 0; i < n_mat; ++i) {
        const int rc = check_matrix(type, w[i], n_in, n_out[i]);
        if (rc != ORIN_FA_OK) return rc;
        if (!y[i] || !aligned(y[i], 4) || (bias && bias[i] && !aligned(bias[i], 4))) return ORIN_FA_E_INVALID;
        a.seg[i] = GemvSeg{w[i], bias ? bias[i] : nullptr, y[i], n_out[i], type, 0};
    }
    if (w_up) {
        if (n_mat != 1) return ORIN_FA_E_INVALID;
        const int rc = check_matrix(type, w_up, n_in, n_out[0]);
        if (rc != ORIN_FA_OK) return rc;
    }
    a.n_seg = n_mat;
    a.w_up = w_up;
    a.x = x;
    a.norm_w = norm_w;
    a.eps = eps;
    a.n_in = n_in;
    a.accumulate = accumulate;
    return hip_rc(gemv_launch(type, a, lib_cu_count() > 0 ? lib_cu_count() : 256, lib_stream()));
}

// One launch over matrices of different types, where the matrix-core kernel takes them all; otherwise
// ORIN_FA_E_INVALID + 1 (not an error: the caller launches them type by type).
constexpr int kNotMixed = 1;
int gemv_call_mixed(const int* types, int n_mat, const void* const* w, const float* const* bias, float* const* y,
                    const int* n_out, const float* x, const float* norm_w, float eps, int n_in) {
    if (!lib_ready()) return ORIN_FA_E_NOT_INIT;
    if (n_mat < 1 || n_mat > 3 || !x || !aligned(x, 16) || (norm_w && !aligned(norm_w, 16))) return ORIN_FA_E_INVALID;
    GemvArgs a{};
    for (int i = 0; i < n_mat; ++i) {
        const int rc = check_matrix(types[i], w[i], n_in, n_out[i]);
        if (rc != ORIN_FA_OK) return rc;
        if (!y[i] || !aligned(y[i], 4) || (bias && bias[i] && !aligned(bias[i], 4))) return ORIN_FA_E_INVALID;
        a.seg[i] = GemvSeg{w[i], bias ? bias[i] : nullptr, y[i], n_out[i], types[i], 0};
    }
    a.n_seg = n_mat;
    a.x = x;
    a.norm_w = norm_w;
    a.eps = eps;
    a.n_in = n_in;
    const hipError_t e = gemv_mixed_launch(a, lib_cu_count() > 0 ? lib_cu_count() : 256, lib_stream());
    return e == hipErrorNotSupported ? kNotMixed : hip_rc(e);
}

int gemv_one(int type, const void* w, const float* bias, float* y, int n_out, const void* w_up, const float* x,
             const float* norm_w, float eps, int n_in, int accumulate) {
    return gemv_call(type, 1, &w, &bias, &y, &n_out, w_up, x, norm_w, eps, n_in, accumulate);
}

// The staged activation for a product over n_in elements: the first n_in of what the last
// orin_quantize_activation staged.  The reference's products read the first n_in elements of its g_q8 block
// whatever length was quantised (src/kernels.cu:1786-1836), and its decode_layer relies on that: it stages
// n_embd elements of d_attn_ and multiplies by wo, whose rows have n_head * head_dim (src/model_gpu.cu:284-285),
// which is shorter in models whose heads do not add up to n_embd.  A product longer than what was staged would
// read elements nobody staged: refused.
int staged(int n_in, const float** x) {
    if (!lib_ready()) return ORIN_FA_E_NOT_INIT;
    if (!lib_stage() || g_staged_n < n_in) return ORIN_FA_E_INVALID;
    *x = lib_stage();
    return ORIN_FA_OK;
}

} // namespace
} // namespace orin_fa

using namespace orin_fa;

extern "C" {

void orin_gemv_use_matrix_cores(int on) { gemv_set_use_mfma(on != 0); }

void orin_gemv_row_shares(int shares) { gemv_set_row_shares(shares); }

size_t orin_row_bytes(int type, int n) { return n < 0 ? 0 : weight_row_bytes(type, n); }

int orin_rms_norm(const float* x, const float* w, int n, float eps, float* y) {
    return orin_rms_norm_rows(x, w, 1, n, eps, y);
}

int orin_rms_norm_rows(const float* x, const float* w, int rows, int cols, float eps, float* y) {
    if (!lib_ready()) return ORIN_FA_E_NOT_INIT;
    if (!x || !w || !y || rows < 0 || cols <= 0) return ORIN_FA_E_INVALID;
    if (rows == 0) return ORIN_FA_OK;
    return hip_rc(rms_norm_launch(x, w, rows, cols, eps, y, lib_stream()));
}

int orin_quantize_activation(const float* x, int n_in) {
    if (!lib_ready()) return ORIN_FA_E_NOT_INIT;
    if (!x || n_in <= 0 || n_in > kStageFloats || !lib_stage()) return ORIN_FA_E_INVALID;
    g_staged_n = n_in;
    return hip_rc(stage_launch(x, lib_stage(), n_in, lib_stream()));
}

int orin_gemv_q8(int type, const void* W, float* y, int n_in, int n_out) {
    const float* x = nullptr;
    const int rc = staged(n_in, &x);
    return rc != ORIN_FA_OK ? rc : gemv_one(type, W, nullptr, y, n_out, nullptr, x, nullptr, 0.0f, n_in, 0);
}

int orin_gemv_q8_bias(int type, const void* W, const float* bias, float* y, int n_in, int n_out) {
    const float* x = nullptr;
    const int rc = staged(n_in, &x);
    if (rc != ORIN_FA_OK) return rc;
    if (!bias) return ORIN_FA_E_INVALID;
    return gemv_one(type, W, bias, y, n_out, nullptr, x, nullptr, 0.0f, n_in, 0);
}

int orin_gemv_q8_add(int type, const void* W, float* y, int n_in, int n_out) {
    const float* x = nullptr;
    const int rc = staged(n_in, &x);
    return rc != ORIN_FA_OK ? rc : gemv_one(type, W, nullptr, y, n_out, nullptr, x, nullptr, 0.0f, n_in, 1);
}

int orin_gemv_fused_gate_up_swiglu(int type, const void* Wg, const void* Wu, float* out, int n_in, int n_out) {
    const float* x = nullptr;
    const int rc = staged(n_in, &x);
    if (rc != ORIN_FA_OK) return rc;
    if (!Wu) return ORIN_FA_E_INVALID;
    return gemv_one(type, Wg, nullptr, out, n_out, Wu, x, nullptr, 0.0f, n_in, 0);
}

int orin_gemv(int type, const void* W, const float* x, float* y, int n_in, int n_out) {
    return gemv_one(type, W, nullptr, y, n_out, nullptr, x, nullptr, 0.0f, n_in, 0);
}

int orin_dequant_row(int type, const void* src, float* y, int n) {
    if (!lib_ready()) return ORIN_FA_E_NOT_INIT;
    if (!src || !y || n <= 0 || weight_row_bytes(type, n) == 0 || !aligned(src, type == kF32 ? 4 : 2)) return ORIN_FA_E_INVALID;
    return hip_rc(dequant_row_launch(type, src, y, n, lib_stream()));
}

int orin_swiglu(float* act, const float* gate, const float* up, int n) {
    if (!lib_ready()) return ORIN_FA_E_NOT_INIT;
    if (!act || !gate || !up || n < 0) return ORIN_FA_E_INVALID;
    if (n == 0) return ORIN_FA_OK;
    return hip_rc(swiglu_launch(act, gate, up, n, lib_stream()));
}

int orin_gemv_multi(int type, int n_mat, const void* const* W, const float* const* bias, float* const* y,
                    const int* n_out, const float* x, const float* norm_w, float eps, int n_in, int accumulate) {
    if (!W || !y || !n_out) return ORIN_FA_E_INVALID;
    return gemv_call(type, n_mat, W, bias, y, n_out, nullptr, x, norm_w, eps, n_in, accumulate);
}

int orin_gemv_multi_types(const int* types, int n_mat, const void* const* W, const float* const* bias, float* const* y,
                          const int* n_out, const float* x, const float* norm_w, float eps, int n_in) {
    if (!types || !W || !y || !n_out) return ORIN_FA_E_INVALID;
    int rc = gemv_call_mixed(types, n_mat, W, bias, y, n_out, x, norm_w, eps, n_in);
    if (rc != kNotMixed) return rc;
    for (int i = 0; i < n_mat; ++i) { // one launch per matrix
        const float* bi = bias ? bias[i] : nullptr;
        if ((rc = gemv_call(types[i], 1, &W[i], &bi, &y[i], &n_out[i], nullptr, x, norm_w, eps, n_in, 0)) != ORIN_FA_OK) return rc;
    }
    return ORIN_FA_OK;
}

int orin_gemv_norm_gate_up_swiglu(int type, const void* Wg, const void* Wu, const float* x, const float* norm_w,
                                  float eps, float* out, int n_in, int n_out) {
    if (!Wu) return ORIN_FA_E_INVALID;
    return gemv_one(type, Wg, nullptr, out, n_out, Wu, x, norm_w, eps, n_in, 0);
}

int orin_decode_layer(const orin_decode_layer_desc* L) {
    if (!lib_ready()) return ORIN_FA_E_NOT_INIT;
    if (!L || !L->x || !L->q || !L->k || !L->v || !L->attn || !L->act || !L->attn_norm || !L->ffn_norm || !L->d_pos)
        return ORIN_FA_E_INVALID;
    if (L->n_embd <= 0 || L->n_head <= 0 || L->n_kv <= 0 || L->head_dim <= 0 || L->n_ff <= 0) return ORIN_FA_E_INVALID;
    if (!L->wq || !L->wk || !L->wv || !L->wo || !L->ffn_gate || !L->ffn_up || !L->ffn_down || !L->kc || !L->vc) return ORIN_FA_E_INVALID;
    if (L->gate_type != L->up_type && !L->up_tmp) return ORIN_FA_E_INVALID; // (checked here so that nothing has run when it fails)
    const int nq = L->n_head * L->head_dim, nkv = L->n_kv * L->head_dim;
    int rc;
    // Every product's row length against the kernels' limit, before the first launch: a layer refused half way
    // would leave x updated by its first half.
    {
        const int n_in[7] = {L->n_embd, L->n_embd, L->n_embd, nq, L->n_embd, L->n_embd, L->n_ff};
        const int n_out[7] = {nq, nkv, nkv, L->n_embd, L->n_ff, L->n_ff, L->n_embd};
        const int t[7] = {L->wq_type, L->wk_type, L->wv_type, L->wo_type, L->gate_type, L->up_type, L->down_type};
        const void* w[7] = {L->wq, L->wk, L->wv, L->wo, L->ffn_gate, L->ffn_up, L->ffn_down};
        for (int i = 0; i < 7; ++i)
            if ((rc = check_matrix(t[i], w[i], n_in[i], n_out[i])) != ORIN_FA_OK) return rc;
    }
    // ---- attn_norm + q, k, v projections: matrices of one type share a launch ----
    {
        const void* w[3] = {L->wq, L->wk, L->wv};
        const float* b[3] = {L->bq, L->bk, L->bv};
        float* y[3] = {L->q, L->k, L->v};
        const int n[3] = {nq, nkv, nkv}, t[3] = {L->wq_type, L->wk_type, L->wv_type};
        bool done[3] = {false, false, false};
        if (t[0] != t[1] || t[1] != t[2]) { // (a file that keeps attn_v in Q6_K beside Q4_K: still one launch)
            rc = gemv_call_mixed(t, 3, w, b, y, n, L->x, L->attn_norm, L->rms_eps, L->n_embd);
            if (rc == ORIN_FA_OK) done[0] = done[1] = done[2] = true;
            else if (rc != kNotMixed) return rc;
        }
        for (int i = 0; i < 3; ++i) {
            if (done[i]) continue;
            const void* gw[3];
            const float* gb[3];
            float* gy[3];
            int gn[3], m = 0;
            for (int j = i; j < 3; ++j)
                if (!done[j] && t[j] == t[i]) {
                    gw[m] = w[j]; gb[m] = b[j]; gy[m] = y[j]; gn[m] = n[j];
                    ++m;
                    done[j] = true;
                }
            rc = gemv_call(t[i], m, gw, gb, gy, gn, nullptr, L->x, L->attn_norm, L->rms_eps, L->n_embd, 0);
            if (rc != ORIN_FA_OK) return rc;
        }
    }
    // ---- per-head norms of q and k (reference: src/model_gpu.cu:274-275) ----
    if (L->q_norm && (rc = orin_rms_norm_rows(L->q, L->q_norm, L->n_head, L->head_dim, L->rms_eps, L->q)) != ORIN_FA_OK) return rc;
    if (L->k_norm && (rc = orin_rms_norm_rows(L->k, L->k_norm, L->n_kv, L->head_dim, L->rms_eps, L->k)) != ORIN_FA_OK) return rc;
    // ---- rotary embedding, cache store, attention (reference: src/model_gpu.cu:277-282) ----
    const bool fused_rope = !L->neox || L->n_rot == 0 || L->n_rot == L->head_dim;
    if (fused_rope) {
        rc = orin_fa_decode_rope_store_ind(L->q, L->k, L->v, L->kc, L->vc, L->attn, L->n_head, L->n_kv, L->head_dim, L->n_ctx,
                                           L->d_pos, L->scale, L->n_rot, L->rope_theta, L->freq_factors, L->neox, L->rope_angles);
        if (rc != ORIN_FA_OK) return rc;
    } else {
        if ((rc = orin_fa_rope_ind(L->q, L->n_head, L->head_dim, L->n_rot, L->rope_theta, L->d_pos, L->freq_factors, L->neox)) != ORIN_FA_OK) return rc;
        if ((rc = orin_fa_rope_ind(L->k, L->n_kv, L->head_dim, L->n_rot, L->rope_theta, L->d_pos, L->freq_factors, L->neox)) != ORIN_FA_OK) return rc;
        rc = orin_fa_decode_store_ind(L->q, L->k, L->v, L->kc, L->vc, L->attn, L->n_head, L->n_kv, L->head_dim, L->n_ctx, L->d_pos, L->scale);
        if (rc != ORIN_FA_OK) return rc;
    }
    // ---- output projection into the residual stream ----
    if ((rc = gemv_one(L->wo_type, L->wo, nullptr, L->x, L->n_embd, nullptr, L->attn, nullptr, 0.0f, nq, 1)) != ORIN_FA_OK) return rc;
    // ---- ffn_norm + gate / up + SwiGLU ----
    if (L->gate_type == L->up_type) {
        rc = gemv_one(L->gate_type, L->ffn_gate, nullptr, L->act, L->n_ff, L->ffn_up, L->x, L->ffn_norm, L->rms_eps, L->n_embd, 0);
        if (rc != ORIN_FA_OK) return rc;
    } else {
        if ((rc = gemv_one(L->gate_type, L->ffn_gate, nullptr, L->act, L->n_ff, nullptr, L->x, L->ffn_norm, L->rms_eps, L->n_embd, 0)) != ORIN_FA_OK) return rc;
        if ((rc = gemv_one(L->up_type, L->ffn_up, nullptr, L->up_tmp, L->n_ff, nullptr, L->x, L->ffn_norm, L->rms_eps, L->n_embd, 0)) != ORIN_FA_OK) return rc;
        if ((rc = orin_swiglu(L->act, L->act, L->up_tmp, L->n_ff)) != ORIN_FA_OK) return rc;
    }
    // ---- down projection into the residual stream ----
    return gemv_one(L->down_type, L->ffn_down, nullptr, L->x, L->n_embd, nullptr, L->act, nullptr, 0.0f, L->n_ff, 1);
}

} // extern "C"
