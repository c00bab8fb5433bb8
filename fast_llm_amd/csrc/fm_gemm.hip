// Grouped ("sparse") matrix products of the dropless MoE MLP on gfx950 matrix cores.
//
// One kernel template serves the three products; they differ only in how an output tile finds its operands:
//   output-sparse      : 128-row block -> expert e -> columns [e*N_s, (e+1)*N_s) of rhs
//   input-inner-sparse : 128-row block -> expert e -> rows    [e*K_s, (e+1)*K_s) of rhs
//   input-row-sparse   : 128-row block of out -> expert e -> reduction over rows [begin_e, pad_begin_e) of the
//                        token axis, everything outside replaced by zero when it is staged into LDS
// (reference semantics: fast_llm/functional/triton/sparse_linear.py:185-258, 310-385, 437-517).
//
// Fast path (bf16/fp16): workgroup tile 128 x BN x 64, four wavefronts in a 2 x 2 grid, each wavefront owns
// 64 x BN/2 of the tile as 32x32x16 MFMA accumulators in fp32. Operand tiles go HBM -> registers (16-byte
// vectors, prefetched one K-step ahead) -> LDS (XOR-swizzled 16-byte chunks, conflict-free for both the
// writes and the 128-bit fragment reads) -> MFMA. Either operand may be contiguous along the reduction axis or
// along its other axis; both end up in the same LDS layout, so the inner loop is identical.
// Workgroups are renumbered so that consecutive tiles run on the same XCD (shared L2) and walk a group of row
// blocks before moving to the next column block.
//
// Generic path (fp32, or any shape/stride the fast path does not take): 64 x 64 x 16 LDS-tiled FMA kernel
// with full bounds checks; fp32 multiply-add, so it also serves the 1e-5 parity configuration.
#include "fm_common.h"

namespace fm {

enum GemmMode { kOutputSparse = 0, kInputInnerSparse = 1, kInputRowSparse = 2 };

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
};

// Where one output tile reads and writes. Offsets are in elements.
struct TileWork {
    int64_t lhs_offset;  // element (first row of tile, k = 0)
    int64_t rhs_offset;  // element (k = 0, first column of tile)
    int64_t out_offset;
    int64_t k_lo, k_hi;  // valid reduction range; outside it operands count as zero
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

__device__ __forceinline__ TileWork resolve_tile(const GemmArgs &args, int64_t row0, int64_t col0) {
    TileWork work;
    work.skip = false;
    work.k_lo = 0;
    work.k_hi = args.inner;
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
        const int expert = dense ? 0 : expert_of_row(args, row0);
        if (expert >= args.num_experts) {
            work.skip = true;  // phantom rows past the last expert
            return work;
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

// Map the hardware workgroup id to a tile. Hardware deals consecutive ids round-robin to the 8 XCDs; undo that
// so each XCD gets a contiguous range of logical ids, then walk `kGroupRows` row blocks per column block.
__device__ __forceinline__ void tile_of_block(const GemmArgs &args, int &tile_m, int &tile_n) {
    constexpr int kXcds = 8, kGroupRows = 16;
    const int total = args.tiles_m * args.tiles_n;
    const int pid = blockIdx.x;
    const int per_xcd = (total + kXcds - 1) / kXcds;
    const int tall = total % kXcds == 0 ? kXcds : total % kXcds;
    const int xcd = pid % kXcds, local = pid / kXcds;
    const int logical = xcd < tall ? xcd * per_xcd + local : tall * per_xcd + (xcd - tall) * (per_xcd - 1) + local;
    const int width = kGroupRows * args.tiles_n;
    const int group = logical / width;
    const int first_m = group * kGroupRows;
    const int group_rows = min(args.tiles_m - first_m, kGroupRows);
    const int in_group = logical - group * width;
    tile_m = first_m + in_group % group_rows;
    tile_n = in_group / group_rows;
}

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

// =========================================================================================================
// Fast path
// =========================================================================================================
typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8_t;
typedef __attribute__((__vector_size__(8 * sizeof(_Float16)))) _Float16 f16x8_t;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float f32x16_t;
typedef __attribute__((__vector_size__(4 * sizeof(uint32_t)))) uint32_t u32x4_t;

template <typename T>
struct Mfma;
template <>
struct Mfma<bf16_t> {
    static __device__ __forceinline__ f32x16_t run(u32x4_t a, u32x4_t b, f32x16_t c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b),
                                                       c, 0, 0, 0);
    }
};
template <>
struct Mfma<f16_t> {
    static __device__ __forceinline__ f32x16_t run(u32x4_t a, u32x4_t b, f32x16_t c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8_t, a), __builtin_bit_cast(f16x8_t, b),
                                                      c, 0, 0, 0);
    }
};

constexpr int kBM = 128, kBK = 64, kGemmThreads = 256;
constexpr int kChunksPerRow = kBK / 8;  // 16-byte chunks along K in one LDS row

// Byte offset of chunk `chunk` (8 elements along K) of row `row` in an LDS operand tile [rows][kBK].
// The XOR spreads 16 consecutive rows of one chunk column over all 64 banks.
__device__ __forceinline__ int lds_chunk_offset(int row, int chunk) {
    return row * (kBK * 2) + ((chunk ^ ((row >> 1) & 7)) << 4);
}

// Stage one operand tile (kRows x kBK) from global memory into registers.
// kContiguousK: element (r, k) at base[r * stride + k]; chunk q -> row q / 8, K-chunk q % 8.
// otherwise   : element (r, k) at base[k * stride + r]; chunk q -> K-row q / (kRows / 8), row-chunk q % (kRows / 8).
template <typename T, int kRows, bool kContiguousK>
struct OperandStage {
    static constexpr int kChunks = kRows * kChunksPerRow / kGemmThreads;
    u32x4_t regs[kChunks];

    __device__ __forceinline__ void load(const T *base, int64_t stride, int64_t k0) {
#pragma unroll
        for (int i = 0; i < kChunks; ++i) {
            const int q = threadIdx.x + i * kGemmThreads;
            const T *pointer;
            if constexpr (kContiguousK) pointer = base + static_cast<int64_t>(q >> 3) * stride + k0 + ((q & 7) << 3);
            else pointer = base + (k0 + q / (kRows / 8)) * stride + ((q % (kRows / 8)) << 3);
            regs[i] = *reinterpret_cast<const u32x4_t *>(pointer);
        }
    }

    // Write the staged tile to LDS; elements whose reduction index is outside [k_lo, k_hi) become zero.
    __device__ __forceinline__ void store(char *lds, int64_t k0, int64_t k_lo, int64_t k_hi, bool masked) {
#pragma unroll
        for (int i = 0; i < kChunks; ++i) {
            const int q = threadIdx.x + i * kGemmThreads;
            u32x4_t value = regs[i];
            if constexpr (kContiguousK) {
                const int row = q >> 3, chunk = q & 7;
                if (masked) {
                    const int64_t k = k0 + (chunk << 3);
                    if (k < k_lo || k + 8 > k_hi) {
#pragma unroll
                        for (int j = 0; j < 4; ++j) {
                            uint32_t word = value[j];
                            if (k + 2 * j < k_lo || k + 2 * j >= k_hi) word &= 0xffff0000u;
                            if (k + 2 * j + 1 < k_lo || k + 2 * j + 1 >= k_hi) word &= 0x0000ffffu;
                            value[j] = word;
                        }
                    }
                }
                *reinterpret_cast<u32x4_t *>(lds + lds_chunk_offset(row, chunk)) = value;
            } else {
                const int k_row = q / (kRows / 8), row0 = (q % (kRows / 8)) << 3;
                if (masked && (k0 + k_row < k_lo || k0 + k_row >= k_hi)) value = u32x4_t{0, 0, 0, 0};
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    const int row = row0 + j;
                    const uint16_t element = static_cast<uint16_t>(value[j >> 1] >> ((j & 1) * 16));
                    *reinterpret_cast<uint16_t *>(lds + lds_chunk_offset(row, k_row >> 3) + ((k_row & 7) << 1)) = element;
                }
            }
        }
    }
};

template <typename T, int kBN, bool kLhsContiguousK, bool kRhsContiguousK>
__global__ __launch_bounds__(kGemmThreads, 2) void grouped_gemm_mfma_kernel(GemmArgs args) {
    constexpr int kWaveM = 64, kWaveN = kBN / 2;
    constexpr int kTilesM = kWaveM / 32, kTilesN = kWaveN / 32;
    extern __shared__ __attribute__((aligned(16))) char lds[];
    char *lds_a = lds;
    char *lds_b = lds + kBM * kBK * 2;

    int tile_m, tile_n;
    tile_of_block(args, tile_m, tile_n);
    const int64_t row0 = static_cast<int64_t>(tile_m) * kBM, col0 = static_cast<int64_t>(tile_n) * kBN;
    const TileWork work = resolve_tile(args, row0, col0);
    if (work.skip) return;

    const T *lhs = static_cast<const T *>(args.lhs) + work.lhs_offset;
    const T *rhs = static_cast<const T *>(args.rhs) + work.rhs_offset;
    const int64_t lhs_stride = kLhsContiguousK ? args.lhs_stride_row : args.lhs_stride_inner;
    const int64_t rhs_stride = kRhsContiguousK ? args.rhs_stride_col : args.rhs_stride_inner;
    const bool masked = args.mode == kInputRowSparse;
    const int64_t k_first = work.k_lo / kBK * kBK;
    const int64_t k_last = (work.k_hi + kBK - 1) / kBK * kBK;

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int wave_m = wave >> 1, wave_n = wave & 1;
    const int frag_row = lane & 31, frag_chunk = lane >> 5;

    f32x16_t acc[kTilesM][kTilesN];
#pragma unroll
    for (int i = 0; i < kTilesM; ++i)
#pragma unroll
        for (int j = 0; j < kTilesN; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

    OperandStage<T, kBM, kLhsContiguousK> stage_a;
    OperandStage<T, kBN, kRhsContiguousK> stage_b;
    if (k_first < k_last) {
        stage_a.load(lhs, lhs_stride, k_first);
        stage_b.load(rhs, rhs_stride, k_first);
    }

    for (int64_t k0 = k_first; k0 < k_last; k0 += kBK) {
        __syncthreads();  // the previous step's fragment reads are done
        stage_a.store(lds_a, k0, work.k_lo, work.k_hi, masked);
        stage_b.store(lds_b, k0, work.k_lo, work.k_hi, masked);
        __syncthreads();
        if (k0 + kBK < k_last) {
            stage_a.load(lhs, lhs_stride, k0 + kBK);
            stage_b.load(rhs, rhs_stride, k0 + kBK);
        }
#pragma unroll
        for (int step = 0; step < kBK / 16; ++step) {
            u32x4_t frag_a[kTilesM], frag_b[kTilesN];
            const int chunk = step * 2 + frag_chunk;
#pragma unroll
            for (int i = 0; i < kTilesM; ++i)
                frag_a[i] = *reinterpret_cast<const u32x4_t *>(
                    lds_a + lds_chunk_offset(wave_m * kWaveM + i * 32 + frag_row, chunk));
#pragma unroll
            for (int j = 0; j < kTilesN; ++j)
                frag_b[j] = *reinterpret_cast<const u32x4_t *>(
                    lds_b + lds_chunk_offset(wave_n * kWaveN + j * 32 + frag_row, chunk));
#pragma unroll
            for (int i = 0; i < kTilesM; ++i)
#pragma unroll
                for (int j = 0; j < kTilesN; ++j) acc[i][j] = Mfma<T>::run(frag_a[i], frag_b[j], acc[i][j]);
        }
    }

    // Accumulator layout of a 32x32 tile: register v of lane l holds row 8*(v/4) + 4*(l/32) + v%4, column l%32.
    const bool accumulate = args.accumulate != 0;
#pragma unroll
    for (int i = 0; i < kTilesM; ++i) {
#pragma unroll
        for (int j = 0; j < kTilesN; ++j) {
            const int column = wave_n * kWaveN + j * 32 + (lane & 31);
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int row = wave_m * kWaveM + i * 32 + 8 * (v >> 2) + 4 * (lane >> 5) + (v & 3);
                store_out_dyn(args.out, args.out_dtype, work.out_offset + row * args.out_stride_row + column,
                              acc[i][j][v], accumulate);
            }
        }
    }
}

// =========================================================================================================
// Generic path
// =========================================================================================================
constexpr int kGenTile = 64, kGenK = 16, kGenThreads = 256;

template <typename T>
__global__ __launch_bounds__(kGenThreads) void grouped_gemm_generic_kernel(GemmArgs args) {
    __shared__ float lds_a[kGenK][kGenTile + 1];
    __shared__ float lds_b[kGenK][kGenTile + 1];
    const int tile_n = blockIdx.x % args.tiles_n, tile_m = blockIdx.x / args.tiles_n;
    const int64_t row0 = static_cast<int64_t>(tile_m) * kGenTile, col0 = static_cast<int64_t>(tile_n) * kGenTile;
    const TileWork work = resolve_tile(args, row0, col0);
    if (work.skip) return;

    const T *lhs = static_cast<const T *>(args.lhs) + work.lhs_offset;
    const T *rhs = static_cast<const T *>(args.rhs) + work.rhs_offset;
    // Rows/columns of this tile that exist (a row-sparse tile must also stay inside its expert's block of out).
    int64_t rows_here = args.rows - row0, cols_here = args.cols - col0;
    if (args.mode == kInputRowSparse) {
        const int64_t left_in_expert = args.sparse_size - row0 % args.sparse_size;
        if (left_in_expert < rows_here) rows_here = left_in_expert;
    }
    const int thread_m = threadIdx.x / 16, thread_n = threadIdx.x % 16;
    float acc[4][4] = {};

    for (int64_t k0 = work.k_lo / kGenK * kGenK; k0 < work.k_hi; k0 += kGenK) {
        for (int i = threadIdx.x; i < kGenK * kGenTile; i += kGenThreads) {
            // lhs: consecutive threads along the axis with the smaller stride
            int k_local, r_local;
            if (args.lhs_stride_inner <= args.lhs_stride_row) { k_local = i % kGenK; r_local = i / kGenK; }
            else { r_local = i % kGenTile; k_local = i / kGenTile; }
            int64_t k = k0 + k_local;
            float value = 0.f;
            if (r_local < rows_here && k >= work.k_lo && k < work.k_hi)
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
        if (row >= rows_here) continue;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int column = thread_n + 16 * j;
            if (column >= cols_here) continue;
            store_out_dyn(args.out, args.out_dtype,
                          work.out_offset + row * args.out_stride_row + column * args.out_stride_col, acc[i][j],
                          args.accumulate != 0);
        }
    }
}

// =========================================================================================================
// Host dispatch
// =========================================================================================================
template <typename T, int kBN, bool kLhsK, bool kRhsK>
static int launch_mfma(const GemmArgs &args, hipStream_t stream) {
    constexpr int lds_bytes = (kBM + kBN) * kBK * 2;
    auto kernel = grouped_gemm_mfma_kernel<T, kBN, kLhsK, kRhsK>;
    static bool configured = false;  // idempotent attribute; a benign race sets it twice
    if (!configured) {
        hipError_t error = hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                                               hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes);
        if (error != hipSuccess) return fail(FM_ERR_LAUNCH, "hipFuncSetAttribute: %s", hipGetErrorString(error));
        configured = true;
    }
    kernel<<<args.tiles_m * args.tiles_n, kGemmThreads, lds_bytes, stream>>>(args);
    return FM_OK;
}

template <typename T, int kBN>
static int launch_mfma_layout(const GemmArgs &args, bool lhs_k, bool rhs_k, hipStream_t stream) {
    if (lhs_k && rhs_k) return launch_mfma<T, kBN, true, true>(args, stream);
    if (lhs_k) return launch_mfma<T, kBN, true, false>(args, stream);
    if (rhs_k) return launch_mfma<T, kBN, false, true>(args, stream);
    return launch_mfma<T, kBN, false, false>(args, stream);
}

static bool vector_ok(const void *pointer, int64_t stride) { return aligned16(pointer) && stride % 8 == 0; }

static int run_gemm(const char *name, GemmArgs args, int dtype, void *stream_) {
    FM_REQUIRE(valid_dtype(dtype) && valid_dtype(args.out_dtype), "%s: bad dtype", name);
    FM_REQUIRE(valid_index_dtype(args.index_dtype), "%s: bad index_dtype %d", name, args.index_dtype);
    FM_REQUIRE(args.rows >= 0 && args.cols >= 0 && args.inner >= 0 && args.sparse_size >= 0 && args.num_experts >= 1,
               "%s: negative shape", name);
    FM_REQUIRE(args.mode != kInputRowSparse || args.expert_ends == nullptr || args.expert_pad_begins != nullptr,
               "%s: null expert_pad_begins", name);
    if (args.rows == 0 || args.cols == 0) return FM_OK;
    FM_REQUIRE(args.out && (args.inner == 0 || (args.lhs && args.rhs)), "%s: null tensor", name);
    hipStream_t stream = static_cast<hipStream_t>(stream_);

    // Fast path: half-precision operands, unit column stride of out, vectorisable operand layouts, tile-aligned.
    const bool lhs_k = args.lhs_stride_inner == 1, lhs_m = args.lhs_stride_row == 1;
    const bool rhs_k = args.rhs_stride_inner == 1, rhs_n = args.rhs_stride_col == 1;
    bool fast = dtype != FM_DTYPE_F32 && args.out_stride_col == 1 && (lhs_k || lhs_m) && (rhs_k || rhs_n);
    fast = fast && vector_ok(args.lhs, lhs_k ? args.lhs_stride_row : args.lhs_stride_inner);
    fast = fast && vector_ok(args.rhs, rhs_k ? args.rhs_stride_col : args.rhs_stride_inner);
    fast = fast && args.inner % kBK == 0 && args.inner > 0 && args.sparse_size % 8 == 0;
    fast = fast && (args.mode == kInputRowSparse ? args.sparse_size % kBM == 0 : args.rows % kBM == 0);
    const int block_n = args.cols % 256 == 0 ? 256 : (args.cols % 128 == 0 ? 128 : 0);
    fast = fast && block_n != 0;
    // Prefer a reduction-contiguous view when both strides are 1 (single row/column operands).
    const bool lhs_contiguous_k = lhs_k, rhs_contiguous_k = rhs_k;

    if (fast) {
        args.tiles_m = static_cast<int>(args.rows / kBM);
        args.tiles_n = static_cast<int>(args.cols / block_n);
        FM_REQUIRE(static_cast<int64_t>(args.tiles_m) * args.tiles_n < (int64_t(1) << 31), "%s: too many tiles", name);
        int status;
        if (dtype == FM_DTYPE_BF16) {
            status = block_n == 256 ? launch_mfma_layout<bf16_t, 256>(args, lhs_contiguous_k, rhs_contiguous_k, stream)
                                    : launch_mfma_layout<bf16_t, 128>(args, lhs_contiguous_k, rhs_contiguous_k, stream);
        } else {
            status = block_n == 256 ? launch_mfma_layout<f16_t, 256>(args, lhs_contiguous_k, rhs_contiguous_k, stream)
                                    : launch_mfma_layout<f16_t, 128>(args, lhs_contiguous_k, rhs_contiguous_k, stream);
        }
        if (status != FM_OK) return status;
    } else {
        FM_REQUIRE(args.mode != kInputRowSparse || args.sparse_size > 0, "%s: empty sparse dimension", name);
        // A row-sparse tile must not cross into the next expert's block of out.
        if (args.mode == kInputRowSparse && args.num_experts > 1 && args.sparse_size % kGenTile != 0)
            return fail(FM_ERR_UNSUPPORTED, "%s: row_sparse_dim=%lld must be a multiple of %d", name,
                        (long long)args.sparse_size, kGenTile);
        args.tiles_m = static_cast<int>((args.rows + kGenTile - 1) / kGenTile);
        args.tiles_n = static_cast<int>((args.cols + kGenTile - 1) / kGenTile);
        FM_REQUIRE(static_cast<int64_t>(args.tiles_m) * args.tiles_n < (int64_t(1) << 31), "%s: too many tiles", name);
        const int grid = args.tiles_m * args.tiles_n;
        FM_DISPATCH_DTYPE(dtype, T, { grouped_gemm_generic_kernel<T><<<grid, kGenThreads, 0, stream>>>(args); });
    }
    return check_launch(name);
}

}  // namespace fm

using namespace fm;

extern "C" int fm_output_sparse_matmul(const void *lhs, const void *rhs, void *out, const void *expert_ends,
                                       int64_t row_dim, int64_t col_sparse_dim, int64_t inner_dim, int64_t num_experts,
                                       int64_t lhs_stride_row, int64_t lhs_stride_inner, int64_t rhs_stride_inner,
                                       int64_t rhs_stride_col, int64_t out_stride_row, int64_t out_stride_col,
                                       int accumulate, int dtype, int out_dtype, int index_dtype, void *stream) {
    GemmArgs args{lhs, rhs, out, expert_ends, nullptr, lhs_stride_row, lhs_stride_inner, rhs_stride_inner,
                  rhs_stride_col, out_stride_row, out_stride_col, row_dim, col_sparse_dim, inner_dim, col_sparse_dim,
                  static_cast<int>(expert_ends ? num_experts : 1), kOutputSparse, accumulate, index_dtype, out_dtype, 0, 0};
    FM_REQUIRE(num_experts >= 1 && num_experts < (1 << 20), "fm_output_sparse_matmul: bad num_experts");
    return run_gemm("fm_output_sparse_matmul", args, dtype, stream);
}

extern "C" int fm_input_inner_sparse_matmul(const void *lhs, const void *rhs, void *out, const void *expert_ends,
                                            int64_t row_dim, int64_t col_dim, int64_t inner_sparse_dim,
                                            int64_t num_experts, int64_t lhs_stride_row, int64_t lhs_stride_inner,
                                            int64_t rhs_stride_inner, int64_t rhs_stride_col, int64_t out_stride_row,
                                            int64_t out_stride_col, int accumulate, int dtype, int out_dtype,
                                            int index_dtype, void *stream) {
    GemmArgs args{lhs, rhs, out, expert_ends, nullptr, lhs_stride_row, lhs_stride_inner, rhs_stride_inner,
                  rhs_stride_col, out_stride_row, out_stride_col, row_dim, col_dim, inner_sparse_dim, inner_sparse_dim,
                  static_cast<int>(expert_ends ? num_experts : 1), kInputInnerSparse, accumulate, index_dtype, out_dtype, 0, 0};
    FM_REQUIRE(num_experts >= 1 && num_experts < (1 << 20), "fm_input_inner_sparse_matmul: bad num_experts");
    return run_gemm("fm_input_inner_sparse_matmul", args, dtype, stream);
}

extern "C" int fm_input_row_sparse_matmul(const void *lhs, const void *rhs, void *out, const void *expert_ends,
                                          const void *expert_pad_begins, int64_t row_sparse_dim, int64_t col_dim,
                                          int64_t inner_dim, int64_t num_experts, int64_t lhs_stride_row,
                                          int64_t lhs_stride_inner, int64_t rhs_stride_inner, int64_t rhs_stride_col,
                                          int64_t out_stride_row, int64_t out_stride_col, int accumulate, int dtype,
                                          int out_dtype, int index_dtype, void *stream) {
    FM_REQUIRE(num_experts >= 1 && num_experts < (1 << 20), "fm_input_row_sparse_matmul: bad num_experts");
    const int64_t experts = expert_ends ? num_experts : 1;
    GemmArgs args{lhs, rhs, out, expert_ends, expert_pad_begins, lhs_stride_row, lhs_stride_inner, rhs_stride_inner,
                  rhs_stride_col, out_stride_row, out_stride_col, row_sparse_dim * experts, col_dim, inner_dim,
                  row_sparse_dim, static_cast<int>(experts), kInputRowSparse, accumulate, index_dtype, out_dtype, 0, 0};
    return run_gemm("fm_input_row_sparse_matmul", args, dtype, stream);
}
