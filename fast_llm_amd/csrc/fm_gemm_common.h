// Arguments and small device helpers shared by the grouped-GEMM kernels.
#pragma once

#include "fm_common.h"

namespace fm {

enum GemmMode { kOutputSparse = 0, kInputInnerSparse = 1, kInputRowSparse = 2 };

// What the MFMA kernel's epilogue does besides storing the product (output-sparse mode, gated MLP):
//   kFusionGatedForward: the product is layer 1's output [rows, 2 * half] = [gate | up]; a tile holds 128 gate columns
//     and the 128 up columns that go with them, `out` (may be null) receives both and `fused_out` [rows, half] receives
//     act(gate) * up;
//   kFusionGatedBackward: the product is the gradient of the activation's output [rows, half]; it is not stored:
//     `fused_in` is layer 1's output, `out` receives the gradient of it (both [rows, 2 * half], same strides) and
//     `fused_out` (may be null) the recomputed activation output.
enum GemmFusion { kFusionNone = 0, kFusionGatedForward = 1, kFusionGatedBackward = 2 };

struct GemmArgs {
    const void *lhs;
    const void *rhs;
    void *out;
    const void *expert_ends;        // null: dense product
    const void *expert_pad_begins;  // row-sparse mode only
    int64_t lhs_stride_row, lhs_stride_inner, rhs_stride_inner, rhs_stride_col, out_stride_row, out_stride_col;
    int64_t rows;         // rows of out
    int64_t cols;         // columns of out
    int64_t inner;        // length of the reduction axis as stored (per expert for input-inner-sparse)
    int64_t sparse_size;  // N_s, K_s or M_s
    int num_experts;
    int mode;
    int accumulate;
    int index_dtype;
    int out_dtype;
    int tiles_m, tiles_n;
    float *partials;  // the caller's workspace when the MFMA kernel splits reductions, else null; set by its launcher
    int fusion;       // GemmFusion
    int activation;   // fm_activation tag, for the fused epilogues
    const void *fused_in;
    void *fused_out;
    int64_t fused_stride;  // row stride of fused_out, elements
    int64_t half;          // columns of the activation output per expert
    int num_ids;           // workgroup ids that may have a tile (set by the MFMA kernel's launcher)
    void *tile_table;      // one record per id, written by the plan kernel into the caller's workspace, or null
};

template <typename OutT>
__device__ __forceinline__ void store_out(void *out, int64_t offset, float value, bool accumulate) {
    OutT *pointer = static_cast<OutT *>(out) + offset;
    if (accumulate) value += to_float(*pointer);
    *pointer = from_float<OutT>(value);
}

__device__ __forceinline__ void store_out_dyn(void *out, int out_dtype, int64_t offset, float value, bool accumulate) {
    if (out_dtype == FM_DTYPE_F32) store_out<float>(out, offset, value, accumulate);
    else if (out_dtype == FM_DTYPE_BF16) store_out<bf16_t>(out, offset, value, accumulate);
    else store_out<f16_t>(out, offset, value, accumulate);
}

// Fast path (fm_gemm_mfma.hip). `eligible` says whether the MFMA kernel can take the problem as described by
// `args` (with `dtype` operands); `launch` fills in the tile counts and launches it.
bool mfma_gemm_eligible(const GemmArgs &args, int dtype);
bool mfma_gemm_fusion_eligible(const GemmArgs &args, int dtype);  // with args.fusion set
// `workspace` (may be null: no split) must hold mfma_gemm_workspace_size(args) bytes when that is not 0.
size_t mfma_gemm_workspace_size(GemmArgs args);
int mfma_gemm_launch(GemmArgs args, int dtype, void *workspace, size_t workspace_size, hipStream_t stream);

}  // namespace fm
