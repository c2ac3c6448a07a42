// Shared pieces of the decode-layer operators around attention (gemv.hip, layer_ops.hip,
// layer_api.hip): weight types, launch arguments, launchers.
#pragma once

#include "fa_common.hpp"

namespace orin_fa {

// Weight types, numbered as the reference numbers them (reference: src/common.h:47-54).
enum : int { kF32 = 0, kF16 = 1, kQ8_0 = 8, kQ4_K = 12, kQ5_K = 13, kQ6_K = 14 };

constexpr int kMaxGemvIn = 32768;   // elements per weight row, at most (4 waves x 64 lanes x 4 slots x 32; the staged activation's size)
constexpr int kStageFloats = 32768; // the staged activation of the *_q8 entry points

struct GemvSeg {
    const void* w;     // n_out rows
    const float* bias; // or null
    float* y;
    int n_out;
    int type;         // used by launches that mix types (n_seg_types != 0), with row_bytes
    size_t row_bytes;
};

struct GemvArgs {
    GemvSeg seg[3];      // matrices of one type that share the activation
    int n_seg;
    const void* w_up;    // not null: seg[0].w is the gate matrix, this the up matrix, y = SiLU(gate x) * (up x)
    const float* x;      // activation, n_in floats, 16-byte aligned
    const float* norm_w; // not null: the activation is RMS-normalised with this weight first
    float eps;
    int n_in;
    int accumulate;      // y += instead of y =
    // filled in by the launcher
    size_t row_bytes;
    int team_waves, wgs_per_cu, mfma_wgs_per_cu, n_seg_types, k_split_override;
    int share_blocks, share_extra; // blocks of a row per share of it (gridDim.z shares), and how many shares take one more
    int few_workgroups;            // not 0: the launch leaves resident places empty (see gemv_rows_body's prologue)
};

size_t weight_row_bytes(int type, int n); // 0: unknown type or n not a whole number of blocks
int weight_align(int type);               // alignment the kernels need of a matrix's base address
hipError_t gemv_launch(int type, GemvArgs args, int cu_count, hipStream_t stream);
// Q4_K and Q6_K on the matrix cores (gemv_mfma.hip): whether type and shape fit, the launch, and the once-only
// permission for large LDS blocks.
bool gemv_mfma_ok(int type, const GemvArgs& args);
hipError_t gemv_mfma_launch(int type, const GemvArgs& args, int cu_count, hipStream_t stream);
hipError_t gemv_mfma_allow_lds();
// Up to three matrices, each Q4_K or Q6_K (GemvSeg::type), in one launch on the matrix cores.
hipError_t gemv_mixed_launch(GemvArgs args, int cu_count, hipStream_t stream);
hipError_t gemv_mfma_mixed_launch(GemvArgs args, int cu_count, hipStream_t stream);
bool gemv_use_mfma();
void gemv_set_use_mfma(bool on);
int gemv_row_shares();          // 0: chosen by shape; 1: accumulating projections never cut a row into shares
void gemv_set_row_shares(int n);

hipError_t rms_norm_launch(const float* x, const float* w, int rows, int cols, float eps, float* y, hipStream_t stream);
hipError_t stage_launch(const float* x, float* stage, int n, hipStream_t stream);
hipError_t swiglu_launch(float* act, const float* gate, const float* up, int n, hipStream_t stream);
hipError_t dequant_row_launch(int type, const void* src, float* y, int n, hipStream_t stream);

// Library state the operators share with the attention entry points (fa_api.hip).
bool lib_ready();
int lib_cu_count();
hipStream_t lib_stream();
float* lib_stage(); // device address of the staged activation on the current device, or null

} // namespace orin_fa
