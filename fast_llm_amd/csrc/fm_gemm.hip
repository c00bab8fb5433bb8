// Grouped ("sparse") matrix products of the dropless MoE MLP: entry points, dispatch, and the generic kernel.
//
// The three products differ only in how an output tile finds its operands:
//   output-sparse      : row block -> expert e -> columns [e*N_s, (e+1)*N_s) of rhs
//   input-inner-sparse : row block -> expert e -> rows    [e*K_s, (e+1)*K_s) of rhs
//   input-row-sparse   : row block of out -> expert e -> reduction over rows [begin_e, pad_begin_e) of the
//                        token axis, everything outside replaced by zero before the multiply
// (reference semantics: fast_llm/functional/triton/sparse_linear.py:185-258, 310-385, 437-517).
//
// Half-precision operands with vectorisable layouts go to the MFMA kernel (fm_gemm_mfma.hip). fp32 operands go to
// the fp32 matrix-core kernel below (tiles of v_mfma_f32_32x32x2_f32: true fp32 multiply-adds, which is what the
// 1e-5 fp32 parity bound needs; 59-63 TFLOP/s at 16384 x 4096 x 2048 over 8 experts). Everything else
// (half-precision operands with odd strides or sizes) goes to the generic kernel: a 64 x 64 x 16 LDS-tiled kernel of
// scalar multiply-adds. Both compute a row block that straddles an expert boundary in one pass per expert, so they
// take any padding multiple, and both check every bound.
#include "fm_gemm_common.h"

namespace fm {

// Where one output tile (or the part of it that belongs to one expert) reads and writes. Offsets are in elements.
struct TileWork {
    int64_t lhs_offset;  // element (first row of tile, k = 0)
    int64_t rhs_offset;  // element (k = 0, first column of tile)
    int64_t out_offset;
    int64_t k_lo, k_hi;  // valid reduction range; outside it operands count as zero
    int row_lo, row_hi;  // rows of the tile, relative to its first row, that this piece of work covers
    bool skip;
};

// Number of experts whose end is <= row (expert_ends is non-decreasing): the expert owning `row`.
__device__ __forceinline__ int expert_of_row(const GemmArgs &args, int64_t row) {
    int lo = 0, hi = args.num_experts;
    while (lo < hi) {
        const int mid = (lo + hi) >> 1;
        if (load_index(args.expert_ends, args.index_dtype, mid) <= row) lo = mid + 1;
        else hi = mid;
    }
    return lo;
}

constexpr int kGenTile = 64, kGenK = 16, kGenThreads = 256;

// The work of the tile at (row0, col0) for the expert that owns its row `first_row` (relative to row0): in the
// products whose rows are grouped by expert, a tile that straddles an expert boundary (any padding multiple is
// allowed) is computed in one piece per expert.
__device__ __forceinline__ TileWork resolve_tile(const GemmArgs &args, int64_t row0, int64_t col0, int first_row,
                                                 int tile_rows = kGenTile) {
    TileWork work;
    work.skip = false;
    work.k_lo = 0;
    work.k_hi = args.inner;
    work.row_lo = first_row;
    work.row_hi = tile_rows;
    work.out_offset = row0 * args.out_stride_row + col0 * args.out_stride_col;
    const bool dense = args.expert_ends == nullptr;
    if (args.mode == kInputRowSparse) {
        const int64_t expert = row0 / args.sparse_size;
        const int64_t row_in_expert = row0 - expert * args.sparse_size;
        work.lhs_offset = row_in_expert * args.lhs_stride_row;
        work.rhs_offset = col0 * args.rhs_stride_col;
        if (!dense) {
            work.k_lo = expert > 0 ? load_index(args.expert_ends, args.index_dtype, expert - 1) : 0;
            work.k_hi = load_index(args.expert_pad_begins, args.index_dtype, expert);
            if (work.k_hi > args.inner) work.k_hi = args.inner;
            if (work.k_lo < 0) work.k_lo = 0;
        }
    } else {
        const int expert = dense ? 0 : expert_of_row(args, row0 + first_row);
        if (expert >= args.num_experts) {
            work.skip = true;  // phantom rows past the last expert
            return work;
        }
        if (!dense) {
            const int64_t end = load_index(args.expert_ends, args.index_dtype, expert);
            if (end - row0 < work.row_hi) work.row_hi = static_cast<int>(end - row0);
        }
        work.lhs_offset = row0 * args.lhs_stride_row;
        if (args.mode == kOutputSparse)
            work.rhs_offset = (static_cast<int64_t>(expert) * args.sparse_size + col0) * args.rhs_stride_col;
        else
            work.rhs_offset = static_cast<int64_t>(expert) * args.sparse_size * args.rhs_stride_inner +
                              col0 * args.rhs_stride_col;
    }
    return work;
}

// =========================================================================================================
// Generic path
// =========================================================================================================
template <typename T>
__global__ __launch_bounds__(kGenThreads) void grouped_gemm_generic_kernel(GemmArgs args) {
    __shared__ float lds_a[kGenK][kGenTile + 1];
    __shared__ float lds_b[kGenK][kGenTile + 1];
    const int tile_n = blockIdx.x % args.tiles_n, tile_m = blockIdx.x / args.tiles_n;
    const int64_t row0 = static_cast<int64_t>(tile_m) * kGenTile, col0 = static_cast<int64_t>(tile_n) * kGenTile;
    // Rows/columns of this tile that exist (a row-sparse tile must also stay inside its expert's block of out).
    int64_t rows_here = args.rows - row0, cols_here = args.cols - col0;
    if (args.mode == kInputRowSparse) {
        const int64_t left_in_expert = args.sparse_size - row0 % args.sparse_size;
        if (left_in_expert < rows_here) rows_here = left_in_expert;
    }
    if (rows_here > kGenTile) rows_here = kGenTile;
    const int thread_m = threadIdx.x / 16, thread_n = threadIdx.x % 16;

    // One pass per expert that owns rows of the tile (a single pass unless the tile straddles a boundary).
    for (int first_row = 0; first_row < rows_here;) {
        const TileWork work = resolve_tile(args, row0, col0, first_row);
        if (work.skip) return;  // the rest of the tile lies past the last expert
        const int row_hi = work.row_hi < rows_here ? work.row_hi : static_cast<int>(rows_here);
        const T *lhs = static_cast<const T *>(args.lhs) + work.lhs_offset;
        const T *rhs = static_cast<const T *>(args.rhs) + work.rhs_offset;
        float acc[4][4] = {};

        for (int64_t k0 = work.k_lo / kGenK * kGenK; k0 < work.k_hi; k0 += kGenK) {
            for (int i = threadIdx.x; i < kGenK * kGenTile; i += kGenThreads) {
                // lhs: consecutive threads along the axis with the smaller stride
                int k_local, r_local;
                if (args.lhs_stride_inner <= args.lhs_stride_row) { k_local = i % kGenK; r_local = i / kGenK; }
                else { r_local = i % kGenTile; k_local = i / kGenTile; }
                int64_t k = k0 + k_local;
                float value = 0.f;
                if (r_local >= first_row && r_local < row_hi && k >= work.k_lo && k < work.k_hi)
                    value = to_float(lhs[r_local * args.lhs_stride_row + k * args.lhs_stride_inner]);
                lds_a[k_local][r_local] = value;

                int c_local;
                if (args.rhs_stride_inner <= args.rhs_stride_col) { k_local = i % kGenK; c_local = i / kGenK; }
                else { c_local = i % kGenTile; k_local = i / kGenTile; }
                k = k0 + k_local;
                value = 0.f;
                if (c_local < cols_here && k >= work.k_lo && k < work.k_hi)
                    value = to_float(rhs[k * args.rhs_stride_inner + c_local * args.rhs_stride_col]);
                lds_b[k_local][c_local] = value;
            }
            __syncthreads();
#pragma unroll
            for (int k = 0; k < kGenK; ++k) {
                float a[4], b[4];
#pragma unroll
                for (int i = 0; i < 4; ++i) a[i] = lds_a[k][thread_m + 16 * i];
#pragma unroll
                for (int j = 0; j < 4; ++j) b[j] = lds_b[k][thread_n + 16 * j];
#pragma unroll
                for (int i = 0; i < 4; ++i)
#pragma unroll
                    for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], b[j], acc[i][j]);
            }
            __syncthreads();
        }

#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int row = thread_m + 16 * i;
            if (row < first_row || row >= row_hi) continue;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int column = thread_n + 16 * j;
                if (column >= cols_here) continue;
                store_out_dyn(args.out, args.out_dtype,
                              work.out_offset + row * args.out_stride_row + column * args.out_stride_col, acc[i][j],
                              args.accumulate != 0);
            }
        }
        first_row = row_hi;
    }
}

// =========================================================================================================
// fp32 operands on the matrix cores
// =========================================================================================================
// kTile x kTile output tile per workgroup, 4 wavefronts (2 x 2), each kTile / 2 squared as accumulators of
// v_mfma_f32_32x32x2_f32 (true fp32 multiply-adds: the 1e-5 parity bound holds), K in slices of kK. Operands of any
// strides are fetched element by element (consecutive lanes along the axis with the smaller stride) into registers
// one slice ahead and stored to LDS as [k][row], double-buffered, one barrier per slice; several workgroups share a
// CU. Tiles lie on a fixed grid of kTile rows: one that straddles an expert boundary is computed in one pass per
// expert, like the generic kernel's, so any padding multiple works (the reference's multiple of 128 gives one pass).
// Two shapes: 128 x 128 x 16 for launches that fill the device (59-63 TFLOP/s at 16384 x 4096 x 2048 over 8 experts),
// and 64 x 64 x 32 for launches of fewer 128-tiles than there are CUs (the 512-token configuration: 32 to 128 of
// them), which are bound by the memory latency of one slice after the other: four times the workgroups, each with a
// quarter of the multiply-adds and half the slices.
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float gemm_f32x16_t;
constexpr int kF32Tile = 128, kF32SmallTile = 64, kF32Threads = 256;
constexpr int kF32SmallLaunchTiles = 256;  // fewer 128-tiles than this (the CUs of the device): tiles of 64

template <int kTile, int kK>
__global__ __launch_bounds__(kF32Threads) void grouped_gemm_f32_mfma_kernel(GemmArgs args) {
    constexpr int kPitch = kTile + 4;                       // floats per K-row in LDS; +4 spreads the banks
    constexpr int kPerThread = kTile * kK / kF32Threads;    // operand elements per thread and slice
    constexpr int kWaveTile = kTile / 2, kBlocks = kWaveTile / 32;  // a wavefront's part, in 32 x 32 accumulators
    static_assert(kPerThread * kF32Threads == kTile * kK && kBlocks >= 1 && kK % 2 == 0, "tile shape");
    __shared__ float lds_a[2][kK][kPitch];
    __shared__ float lds_b[2][kK][kPitch];
    const int tile_n = blockIdx.x % args.tiles_n, tile_m = blockIdx.x / args.tiles_n;
    const int64_t row0 = static_cast<int64_t>(tile_m) * kTile, col0 = static_cast<int64_t>(tile_n) * kTile;
    int64_t rows_here = args.rows - row0, cols_here = args.cols - col0;
    if (args.mode == kInputRowSparse) {
        const int64_t left_in_expert = args.sparse_size - row0 % args.sparse_size;
        if (left_in_expert < rows_here) rows_here = left_in_expert;
    }
    if (rows_here > kTile) rows_here = kTile;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int wave_m = wave >> 1, wave_n = wave & 1;
    const bool lhs_k_fastest = args.lhs_stride_inner <= args.lhs_stride_row;
    const bool rhs_k_fastest = args.rhs_stride_inner <= args.rhs_stride_col;
    const float *lhs_all = static_cast<const float *>(args.lhs), *rhs_all = static_cast<const float *>(args.rhs);

    for (int first_row = 0; first_row < rows_here;) {
        const TileWork work = resolve_tile(args, row0, col0, first_row, kTile);
        if (work.skip) return;  // the rest of the tile lies past the last expert
        const int row_hi = work.row_hi < rows_here ? work.row_hi : static_cast<int>(rows_here);
        const float *lhs = lhs_all + work.lhs_offset, *rhs = rhs_all + work.rhs_offset;
        gemm_f32x16_t acc[kBlocks][kBlocks];
#pragma unroll
        for (int i = 0; i < kBlocks; ++i)
#pragma unroll
            for (int j = 0; j < kBlocks; ++j)
#pragma unroll
                for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

        // Element e of this thread in a slice: (k, row) with the memory-contiguous axis fastest over the lanes.
        float staged_a[kPerThread], staged_b[kPerThread];
        auto fetch = [&](int64_t k0) {
#pragma unroll
            for (int e = 0; e < kPerThread; ++e) {
                const int i = threadIdx.x + e * kF32Threads;
                int k_local = lhs_k_fastest ? i % kK : i / kTile;
                const int r_local = lhs_k_fastest ? i / kK : i % kTile;
                int64_t k = k0 + k_local;
                staged_a[e] = 0.f;
                if (r_local >= first_row && r_local < row_hi && k >= work.k_lo && k < work.k_hi)
                    staged_a[e] = lhs[r_local * args.lhs_stride_row + k * args.lhs_stride_inner];
                k_local = rhs_k_fastest ? i % kK : i / kTile;
                const int c_local = rhs_k_fastest ? i / kK : i % kTile;
                k = k0 + k_local;
                staged_b[e] = 0.f;
                if (c_local < cols_here && k >= work.k_lo && k < work.k_hi)
                    staged_b[e] = rhs[k * args.rhs_stride_inner + c_local * args.rhs_stride_col];
            }
        };
        auto stage = [&](int buffer) {
#pragma unroll
            for (int e = 0; e < kPerThread; ++e) {
                const int i = threadIdx.x + e * kF32Threads;
                lds_a[buffer][lhs_k_fastest ? i % kK : i / kTile][lhs_k_fastest ? i / kK : i % kTile] = staged_a[e];
                lds_b[buffer][rhs_k_fastest ? i % kK : i / kTile][rhs_k_fastest ? i / kK : i % kTile] = staged_b[e];
            }
        };

        const int64_t k_begin = work.k_lo / kK * kK;
        if (k_begin < work.k_hi) {
            fetch(k_begin);
            stage(0);
        }
        __syncthreads();
        int buffer = 0;
        for (int64_t k0 = k_begin; k0 < work.k_hi; k0 += kK, buffer ^= 1) {
            const bool more = k0 + kK < work.k_hi;
            if (more) fetch(k0 + kK);  // in flight during the multiplications
#pragma unroll
            for (int kstep = 0; kstep < kK / 2; ++kstep) {
                // Lane l supplies row (or column) l % 32 at k = 2 kstep + l / 32.
                const int k_local = 2 * kstep + (lane >> 5);
                float a[kBlocks], b[kBlocks];
#pragma unroll
                for (int i = 0; i < kBlocks; ++i) a[i] = lds_a[buffer][k_local][wave_m * kWaveTile + i * 32 + (lane & 31)];
#pragma unroll
                for (int j = 0; j < kBlocks; ++j) b[j] = lds_b[buffer][k_local][wave_n * kWaveTile + j * 32 + (lane & 31)];
#pragma unroll
                for (int i = 0; i < kBlocks; ++i)
#pragma unroll
                    for (int j = 0; j < kBlocks; ++j)
                        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[i], b[j], acc[i][j], 0, 0, 0);
            }
            // The other buffer was last read a slice ago, before the previous barrier.
            if (more) stage(buffer ^ 1);
            __syncthreads();
        }

        // Lane l holds column l % 32 of each 32 x 32 accumulator; register v is row 8 (v / 4) + 4 (l / 32) + v % 4.
#pragma unroll
        for (int i = 0; i < kBlocks; ++i)
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int row = wave_m * kWaveTile + i * 32 + 8 * (v / 4) + 4 * (lane >> 5) + v % 4;
                if (row < first_row || row >= row_hi) continue;
#pragma unroll
                for (int j = 0; j < kBlocks; ++j) {
                    const int column = wave_n * kWaveTile + j * 32 + (lane & 31);
                    if (column >= cols_here) continue;
                    store_out_dyn(args.out, args.out_dtype,
                                  work.out_offset + row * args.out_stride_row + column * args.out_stride_col,
                                  acc[i][j][v], args.accumulate != 0);
                }
            }
        first_row = row_hi;
        __syncthreads();  // the next pass stages into the buffers again
    }
}

// =========================================================================================================
// Host dispatch
// =========================================================================================================
static int run_gemm(const char *name, GemmArgs args, int dtype, void *workspace, size_t workspace_size, void *stream_) {
    FM_REQUIRE(valid_dtype(dtype) && valid_dtype(args.out_dtype), "%s: bad dtype", name);
    FM_REQUIRE(valid_index_dtype(args.index_dtype), "%s: bad index_dtype %d", name, args.index_dtype);
    FM_REQUIRE(args.rows >= 0 && args.cols >= 0 && args.inner >= 0 && args.sparse_size >= 0 && args.num_experts >= 1,
               "%s: negative shape", name);
    FM_REQUIRE(args.mode != kInputRowSparse || args.expert_ends == nullptr || args.expert_pad_begins != nullptr,
               "%s: null expert_pad_begins", name);
    FM_REQUIRE(workspace != nullptr || workspace_size == 0, "%s: null workspace of %zu bytes", name, workspace_size);
    if (args.rows == 0 || args.cols == 0) return FM_OK;
    FM_REQUIRE(args.out && (args.inner == 0 || (args.lhs && args.rhs)), "%s: null tensor", name);
    hipStream_t stream = static_cast<hipStream_t>(stream_);

    int note = FM_OK;
    if (mfma_gemm_eligible(args, dtype)) {
        if (int status = mfma_gemm_launch(args, dtype, workspace, workspace_size, stream)) return status;
    } else {
        // Half-precision operands that the matrix-core kernel cannot take: correct, but far slower. Say so.
        if (dtype != FM_DTYPE_F32) note = FM_NOTE_GENERIC_KERNEL;
        // A row-sparse tile must not cross into the next expert's block of out.
        if (args.mode == kInputRowSparse && args.num_experts > 1 && args.sparse_size % kGenTile != 0)
            return fail(FM_ERR_UNSUPPORTED, "%s: row_sparse_dim=%lld must be a multiple of %d", name,
                        (long long)args.sparse_size, kGenTile);
        // fp32 operands go to the matrix cores when the row-sparse product's blocks of out are whole tiles there too:
        // tiles of 128, or of 64 when there are fewer 128-tiles than CUs (see the kernel).
        const auto whole_tiles = [&](int tile) {
            return !(args.mode == kInputRowSparse && args.num_experts > 1 && args.sparse_size % tile != 0);
        };
        const int64_t large_tiles = ((args.rows + kF32Tile - 1) / kF32Tile) * ((args.cols + kF32Tile - 1) / kF32Tile);
        const bool f32_small = dtype == FM_DTYPE_F32 && large_tiles < kF32SmallLaunchTiles && whole_tiles(kF32SmallTile);
        const bool f32_mfma = dtype == FM_DTYPE_F32 && (f32_small || whole_tiles(kF32Tile));
        const int tile = f32_small ? kF32SmallTile : (f32_mfma ? kF32Tile : kGenTile);
        args.tiles_m = static_cast<int>((args.rows + tile - 1) / tile);
        args.tiles_n = static_cast<int>((args.cols + tile - 1) / tile);
        FM_REQUIRE(static_cast<int64_t>(args.tiles_m) * args.tiles_n < (int64_t(1) << 31), "%s: too many tiles", name);
        const int grid = args.tiles_m * args.tiles_n;
        if (f32_small) {
            grouped_gemm_f32_mfma_kernel<kF32SmallTile, 32><<<grid, kF32Threads, 0, stream>>>(args);
        } else if (f32_mfma) {
            grouped_gemm_f32_mfma_kernel<kF32Tile, 16><<<grid, kF32Threads, 0, stream>>>(args);
        } else {
            FM_DISPATCH_DTYPE(dtype, T, { grouped_gemm_generic_kernel<T><<<grid, kGenThreads, 0, stream>>>(args); });
        }
    }
    if (int status = check_launch(name)) return status;
    return note;
}

}  // namespace fm

using namespace fm;

extern "C" int fm_output_sparse_matmul(const void *lhs, const void *rhs, void *out, const void *expert_ends,
                                       int64_t row_dim, int64_t col_sparse_dim, int64_t inner_dim, int64_t num_experts,
                                       int64_t lhs_stride_row, int64_t lhs_stride_inner, int64_t rhs_stride_inner,
                                       int64_t rhs_stride_col, int64_t out_stride_row, int64_t out_stride_col,
                                       int accumulate, int dtype, int out_dtype, int index_dtype, void *workspace,
                                       size_t workspace_size, void *stream) {
    GemmArgs args{lhs, rhs, out, expert_ends, nullptr, lhs_stride_row, lhs_stride_inner, rhs_stride_inner,
                  rhs_stride_col, out_stride_row, out_stride_col, row_dim, col_sparse_dim, inner_dim, col_sparse_dim,
                  static_cast<int>(expert_ends ? num_experts : 1), kOutputSparse, accumulate, index_dtype, out_dtype, 0, 0, nullptr};
    FM_REQUIRE(num_experts >= 1 && num_experts < (1 << 20), "fm_output_sparse_matmul: bad num_experts");
    return run_gemm("fm_output_sparse_matmul", args, dtype, workspace, workspace_size, stream);
}

extern "C" int fm_input_inner_sparse_matmul(const void *lhs, const void *rhs, void *out, const void *expert_ends,
                                            int64_t row_dim, int64_t col_dim, int64_t inner_sparse_dim,
                                            int64_t num_experts, int64_t lhs_stride_row, int64_t lhs_stride_inner,
                                            int64_t rhs_stride_inner, int64_t rhs_stride_col, int64_t out_stride_row,
                                            int64_t out_stride_col, int accumulate, int dtype, int out_dtype,
                                            int index_dtype, void *workspace, size_t workspace_size, void *stream) {
    GemmArgs args{lhs, rhs, out, expert_ends, nullptr, lhs_stride_row, lhs_stride_inner, rhs_stride_inner,
                  rhs_stride_col, out_stride_row, out_stride_col, row_dim, col_dim, inner_sparse_dim, inner_sparse_dim,
                  static_cast<int>(expert_ends ? num_experts : 1), kInputInnerSparse, accumulate, index_dtype, out_dtype, 0, 0, nullptr};
    FM_REQUIRE(num_experts >= 1 && num_experts < (1 << 20), "fm_input_inner_sparse_matmul: bad num_experts");
    return run_gemm("fm_input_inner_sparse_matmul", args, dtype, workspace, workspace_size, stream);
}

extern "C" int fm_input_row_sparse_matmul(const void *lhs, const void *rhs, void *out, const void *expert_ends,
                                          const void *expert_pad_begins, int64_t row_sparse_dim, int64_t col_dim,
                                          int64_t inner_dim, int64_t num_experts, int64_t lhs_stride_row,
                                          int64_t lhs_stride_inner, int64_t rhs_stride_inner, int64_t rhs_stride_col,
                                          int64_t out_stride_row, int64_t out_stride_col, int accumulate, int dtype,
                                          int out_dtype, int index_dtype, void *workspace, size_t workspace_size,
                                          void *stream) {
    FM_REQUIRE(num_experts >= 1 && num_experts < (1 << 20), "fm_input_row_sparse_matmul: bad num_experts");
    const int64_t experts = expert_ends ? num_experts : 1;
    GemmArgs args{lhs, rhs, out, expert_ends, expert_pad_begins, lhs_stride_row, lhs_stride_inner, rhs_stride_inner,
                  rhs_stride_col, out_stride_row, out_stride_col, row_sparse_dim * experts, col_dim, inner_dim,
                  row_sparse_dim, static_cast<int>(experts), kInputRowSparse, accumulate, index_dtype, out_dtype, 0, 0, nullptr};
    return run_gemm("fm_input_row_sparse_matmul", args, dtype, workspace, workspace_size, stream);
}

static size_t workspace_size_of(int mode, int64_t row_dim, int64_t col_dim, int64_t inner_dim, int64_t num_experts,
                                int dtype) {
    if (dtype != FM_DTYPE_BF16 && dtype != FM_DTYPE_F16) return 0;  // fp32 operands never take the matrix-core kernel
    if (row_dim <= 0 || col_dim <= 0 || inner_dim <= 0 || num_experts < 0 || num_experts >= (1 << 20)) return 0;
    GemmArgs args{};
    args.num_experts = static_cast<int>(num_experts > 1 ? num_experts : 1);
    args.rows = mode == kInputRowSparse ? row_dim * args.num_experts : row_dim;
    args.cols = col_dim;
    args.inner = inner_dim;
    args.sparse_size = mode == kInputRowSparse ? row_dim : 0;
    args.mode = mode;
    return mfma_gemm_workspace_size(args);
}

extern "C" size_t fm_grouped_gemm_workspace_size(int64_t row_dim, int64_t col_dim, int64_t inner_dim,
                                                 int64_t num_experts, int dtype) {
    return workspace_size_of(kOutputSparse, row_dim, col_dim, inner_dim, num_experts, dtype);  // input-inner-sparse: same
}

extern "C" size_t fm_input_row_sparse_matmul_workspace_size(int64_t row_sparse_dim, int64_t col_dim, int64_t inner_dim,
                                                            int64_t num_experts, int dtype) {
    return workspace_size_of(kInputRowSparse, row_sparse_dim, col_dim, inner_dim, num_experts, dtype);
}

// ---- grouped products with the gated activation fused into the epilogue ------------------------------------
static int run_fused_gemm(const char *name, GemmArgs args, int dtype, void *stream) {
    FM_REQUIRE(valid_dtype(dtype) && valid_index_dtype(args.index_dtype), "%s: bad dtype", name);
    FM_REQUIRE(args.activation >= FM_ACT_GELU && args.activation <= FM_ACT_IDENTITY, "%s: bad activation %d", name,
               args.activation);
    FM_REQUIRE(args.rows >= 0 && args.half > 0 && args.inner > 0 && args.num_experts >= 1 &&
                   args.num_experts < (1 << 20),
               "%s: bad shape", name);
    if (args.rows == 0) return FM_OK;
    FM_REQUIRE(args.lhs && args.rhs, "%s: null tensor", name);
    if (!mfma_gemm_fusion_eligible(args, dtype))
        return fail(FM_ERR_UNSUPPORTED,
                    "%s: needs bf16/fp16, 16-byte aligned K-contiguous operands, K a multiple of 64 and an activation "
                    "width that is a multiple of 128 (forward) or 8 (backward); run the product and the activation "
                    "separately",
                    name);
    if (int status = mfma_gemm_launch(args, dtype, nullptr, 0, static_cast<hipStream_t>(stream))) return status;
    return check_launch(name);
}

extern "C" int fm_output_sparse_matmul_gated_activation(
    const void *lhs, const void *rhs, void *layer_1_out, void *activation_out, const void *expert_ends,
    int64_t row_dim, int64_t activation_dim, int64_t inner_dim, int64_t num_experts, int64_t lhs_stride_row,
    int64_t lhs_stride_inner, int64_t rhs_stride_inner, int64_t rhs_stride_col, int activation, int dtype,
    int index_dtype, void *stream) {
    const char *name = "fm_output_sparse_matmul_gated_activation";
    FM_REQUIRE(activation_out, "%s: null activation_out", name);
    GemmArgs args{lhs, rhs, layer_1_out, expert_ends, nullptr, lhs_stride_row, lhs_stride_inner, rhs_stride_inner,
                  rhs_stride_col, 2 * activation_dim, 1, row_dim, 2 * activation_dim, inner_dim, 2 * activation_dim,
                  static_cast<int>(expert_ends ? num_experts : 1), kOutputSparse, 0, index_dtype, dtype, 0, 0, nullptr};
    args.fusion = kFusionGatedForward;
    args.activation = activation;
    args.fused_out = activation_out;
    args.fused_stride = activation_dim;
    args.half = activation_dim;
    return run_fused_gemm(name, args, dtype, stream);
}

extern "C" int fm_output_sparse_matmul_gated_activation_backward(
    const void *lhs, const void *rhs, const void *layer_1_out, void *grad_layer_1_out, void *activation_out,
    const void *expert_ends, int64_t row_dim, int64_t activation_dim, int64_t inner_dim, int64_t num_experts,
    int64_t lhs_stride_row, int64_t lhs_stride_inner, int64_t rhs_stride_inner, int64_t rhs_stride_col, int activation,
    int dtype, int index_dtype, void *stream) {
    const char *name = "fm_output_sparse_matmul_gated_activation_backward";
    FM_REQUIRE(layer_1_out && grad_layer_1_out, "%s: null tensor", name);
    GemmArgs args{lhs, rhs, grad_layer_1_out, expert_ends, nullptr, lhs_stride_row, lhs_stride_inner, rhs_stride_inner,
                  rhs_stride_col, 2 * activation_dim, 1, row_dim, activation_dim, inner_dim, activation_dim,
                  static_cast<int>(expert_ends ? num_experts : 1), kOutputSparse, 0, index_dtype, dtype, 0, 0, nullptr};
    args.fusion = kFusionGatedBackward;
    args.activation = activation;
    args.fused_in = layer_1_out;
    args.fused_out = activation_out;
    args.fused_stride = activation_dim;
    args.half = activation_dim;
    return run_fused_gemm(name, args, dtype, stream);
}
