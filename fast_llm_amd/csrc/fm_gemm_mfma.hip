// Grouped matrix products on the gfx950 matrix cores (bf16 / fp16 operands, fp32 accumulation).
//
// One workgroup = 8 wavefronts = one 256 x 256 tile of `out`, reduced 64 elements of K at a time:
//   * Operand tiles go from global memory straight into LDS (`global_load_lds_dwordx4`, 16 bytes per lane, no
//     VGPR staging) into a two-stage ring; the loads of K-step t+1 are in flight while step t is multiplied.
//   * An operand may be contiguous along K (activations [rows, K], `weight.t()`) or along its other axis
//     (`weight` [K, N], `activations.t()`). K-contiguous tiles are stored [row][K] and read as 128-bit MFMA
//     fragments; the others are stored [K][row] as they lie in memory and read with the LDS transpose load
//     `ds_read_b64_tr_b16`, which hands every lane four consecutive K values of one row. Both layouts are
//     XOR-swizzled so that fragment reads hit all 64 banks; the swizzle is applied on the global-address side
//     because a direct-to-LDS load writes lane i to LDS slot i.
//   * Wavefronts form a 2 x 4 grid, each owns 128 x 64 of the tile as 4 x 2 accumulators of
//     v_mfma_f32_32x32x16 (128 fp32 registers per lane), two wavefronts per SIMD.
//   * Tiles never straddle experts: the row tiles of an expert are enumerated from `expert_ends` on the device
//     (ceil(rows_e / 256) each), a last partial tile loads clamped rows and stores only its valid rows, so any
//     padding multiple works and phantom rows past the last expert are never touched. For the row-sparse product
//     the reduction runs over [begin_e, pad_begin_e); a K-tile that sticks out of that range is zeroed in LDS
//     after it lands (zero-fill, not multiply-by-zero, so NaN in padding rows cannot leak).
//   * Hardware hands consecutive workgroup ids to the 8 XCDs round-robin; ids are renumbered so every XCD works
//     on a contiguous run of tiles (8 row tiles per column tile) and re-reads operands from its own L2.
// Results are deterministic: one workgroup per output tile, fixed summation order, no atomics.
#include "fm_gemm_common.h"

namespace fm {

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8_t;
typedef __attribute__((__vector_size__(8 * sizeof(_Float16)))) _Float16 f16x8_t;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float f32x16_t;
typedef __attribute__((__vector_size__(4 * sizeof(uint32_t)))) uint32_t u32x4_t;
typedef __attribute__((__vector_size__(2 * sizeof(uint32_t)))) uint32_t u32x2_t;
typedef __attribute__((__vector_size__(4 * sizeof(short)))) short i16x4_t;

#define FM_LDS(T) __attribute__((address_space(3))) T
#define FM_GLOBAL(T) __attribute__((address_space(1))) T

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

constexpr int kTile = 256, kBK = 64, kMfmaThreads = 512;
constexpr int kOperandBytes = kTile * kBK * 2;  // one operand tile in LDS: 32 KiB in either layout
constexpr int kStageBytes = 2 * kOperandBytes;  // lhs tile, then rhs tile
constexpr int kStages = 2;
constexpr int kLdsBytes = kStages * kStageBytes;
constexpr int kWaveRows = 128, kWaveCols = 64;  // 2 x 4 wavefronts

// ---- LDS layouts ---------------------------------------------------------------------------------------
// K-contiguous operand, [256 rows][64 k]: 16-byte chunk c (8 k values) of row r sits at r * 128 + ((c ^ ((r >> 1) & 7)) * 16.
// The 16 lanes that read one chunk column of 16 consecutive rows then cover all 64 banks.
__device__ __forceinline__ int lds_offset_k_major(int row, int chunk) {
    return row * (kBK * 2) + ((chunk ^ ((row >> 1) & 7)) << 4);
}
// Row-contiguous operand, [64 k][256 rows]: the 32-byte group g (16 rows) of K-row k sits at k * 512 + (g ^ (2 * (k & 3))) * 32.
// A transpose load by 32 lanes touches 4 K-rows x 2 groups; the XOR sends them to 8 different bank octets.
__device__ __forceinline__ int lds_offset_row_major(int k, int row) {
    return k * (kTile * 2) + ((((row >> 4) ^ ((k & 3) << 1)) << 5) | ((row & 15) << 1));
}

// Direct global -> LDS loader of one operand tile per K-step. Each of the 8 wavefronts issues 4 loads of
// 64 lanes x 16 bytes; load j of wavefront w fills LDS slots [(4 w + j) * 64, +64) of the operand tile.
template <bool kContiguousK>
struct TileLoader {
    const char *pointer[4];
    int64_t step;

    // `base`: element (first row of the tile, first k of the loop). `stride`: bytes between rows (K-contiguous)
    // or between K-rows (row-contiguous). Rows >= valid_rows are replaced by in-range ones (never stored).
    __device__ __forceinline__ void setup(const char *base, int64_t stride, int valid_rows, int wave, int lane) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int slot = (wave * 4 + j) * 64 + lane;
            if constexpr (kContiguousK) {
                const int row = slot >> 3;
                const int chunk = (slot & 7) ^ ((row >> 1) & 7);
                pointer[j] = base + static_cast<int64_t>(min(row, valid_rows - 1)) * stride + chunk * 16;
            } else {
                const int k = slot >> 5, position = slot & 31;
                const int group = (position >> 1) ^ ((k & 3) << 1);
                int first_row = (group * 2 + (position & 1)) * 8;
                if (first_row >= valid_rows) first_row = 0;
                pointer[j] = base + k * stride + first_row * 2;
            }
        }
        step = kContiguousK ? kBK * 2 : kBK * stride;
    }

    __device__ __forceinline__ void issue(FM_LDS(char) * operand_lds, int wave) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            __builtin_amdgcn_global_load_lds((const FM_GLOBAL(void) *)(pointer[j]),
                                             reinterpret_cast<FM_LDS(void) *>(operand_lds + (wave * 4 + j) * 1024), 16,
                                             0, 0);
            pointer[j] += step;
        }
    }
};

// MFMA operand fragment (8 consecutive k of one row per lane; lane l: row l % 32, k half l / 32) of the 32 rows
// starting at `row_base`, for the 16-wide K slice `kstep` of the tile.
template <bool kContiguousK>
__device__ __forceinline__ u32x4_t load_fragment(FM_LDS(char) * operand_lds, int row_base, int kstep, int lane) {
    if constexpr (kContiguousK) {
        const int offset = lds_offset_k_major(row_base + (lane & 31), kstep * 2 + (lane >> 5));
        return *reinterpret_cast<FM_LDS(u32x4_t) *>(operand_lds + offset);
    } else {
        // ds_read_b64_tr_b16 works on groups of 16 lanes: lane s of a group supplies the address of 4 rows
        // (row0 + 4 (s % 4) ..) at K-row k0 + s / 4 and receives k0 .. k0 + 3 of row row0 + s.
        const int s = lane & 15, group = lane >> 4;
        const int row = row_base + ((group & 1) << 4) + ((s & 3) << 2);
        const int k = kstep * 16 + ((group >> 1) << 3) + (s >> 2);
        const i16x4_t low = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
            reinterpret_cast<FM_LDS(i16x4_t) *>(operand_lds + lds_offset_row_major(k, row)));
        const i16x4_t high = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
            reinterpret_cast<FM_LDS(i16x4_t) *>(operand_lds + lds_offset_row_major(k + 4, row)));
        const u32x2_t low_words = __builtin_bit_cast(u32x2_t, low), high_words = __builtin_bit_cast(u32x2_t, high);
        return u32x4_t{low_words[0], low_words[1], high_words[0], high_words[1]};
    }
}

// Zero, in a landed LDS tile whose K origin is k0, everything whose reduction index is outside [k_lo, k_hi).
template <bool kContiguousK>
__device__ __forceinline__ void mask_tile(FM_LDS(char) * operand_lds, int64_t k0, int64_t k_lo, int64_t k_hi) {
    for (int slot = threadIdx.x; slot < kOperandBytes / 16; slot += kMfmaThreads) {
        FM_LDS(u32x4_t) *pointer = reinterpret_cast<FM_LDS(u32x4_t) *>(operand_lds + slot * 16);
        if constexpr (kContiguousK) {
            const int row = slot >> 3;
            const int64_t k = k0 + (((slot & 7) ^ ((row >> 1) & 7)) << 3);
            if (k >= k_lo && k + 8 <= k_hi) continue;
            u32x4_t value = *pointer;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                uint32_t word = value[j];
                if (k + 2 * j < k_lo || k + 2 * j >= k_hi) word &= 0xffff0000u;
                if (k + 2 * j + 1 < k_lo || k + 2 * j + 1 >= k_hi) word &= 0x0000ffffu;
                value[j] = word;
            }
            *pointer = value;
        } else {
            const int64_t k = k0 + (slot >> 5);
            if (k < k_lo || k >= k_hi) *pointer = u32x4_t{0, 0, 0, 0};
        }
    }
}

// ---- which tile ----------------------------------------------------------------------------------------
struct TileWork {
    int64_t lhs_offset, rhs_offset, out_offset;  // elements
    int rows_valid, cols_valid;
    int64_t k_lo, k_hi;
};

// The t-th 256-row tile over all experts, in expert order (expert e contributes ceil(rows_e / 256) tiles).
// Every wavefront scans `expert_ends` 64 experts at a time; returns false if there are fewer than t + 1 tiles.
__device__ __forceinline__ bool find_row_tile(const GemmArgs &args, int tile, int &expert, int64_t &row0,
                                              int &rows_valid) {
    if (args.expert_ends == nullptr) {
        expert = 0;
        row0 = static_cast<int64_t>(tile) * kTile;
        if (row0 >= args.rows) return false;
        rows_valid = static_cast<int>(min(static_cast<int64_t>(kTile), args.rows - row0));
        return true;
    }
    const int lane = threadIdx.x & 63;
    int tiles_before = 0;
    for (int base = 0; base < args.num_experts; base += 64) {
        const int e = base + lane;
        int64_t begin = 0, end = 0;
        if (e < args.num_experts) {
            end = min(load_index(args.expert_ends, args.index_dtype, e), args.rows);
            begin = e > 0 ? load_index(args.expert_ends, args.index_dtype, e - 1) : 0;
        }
        const int count = end > begin ? static_cast<int>((end - begin + kTile - 1) / kTile) : 0;
        int inclusive = count;
#pragma unroll
        for (int offset = 1; offset < 64; offset <<= 1) {
            const int other = __shfl_up(inclusive, offset, 64);
            if (lane >= offset) inclusive += other;
        }
        const int total = __shfl(inclusive, 63, 64);
        if (tile < tiles_before + total) {
            const uint64_t owners = __ballot(tiles_before + inclusive > tile);
            const int owner = __ffsll(static_cast<unsigned long long>(owners)) - 1;
            const int first_tile = tiles_before + __shfl(inclusive - count, owner, 64);
            const int64_t owner_begin = __shfl(begin, owner, 64), owner_end = __shfl(end, owner, 64);
            expert = base + owner;
            row0 = owner_begin + static_cast<int64_t>(tile - first_tile) * kTile;
            rows_valid = static_cast<int>(min(static_cast<int64_t>(kTile), owner_end - row0));
            return true;
        }
        tiles_before += total;
    }
    return false;
}

__device__ __forceinline__ bool resolve_tile(const GemmArgs &args, int tile_m, int tile_n, TileWork &work) {
    const int64_t col0 = static_cast<int64_t>(tile_n) * kTile;
    work.cols_valid = static_cast<int>(min(static_cast<int64_t>(kTile), args.cols - col0));
    work.k_lo = 0;
    work.k_hi = args.inner;
    if (args.mode == kInputRowSparse) {
        const int tiles_per_expert = static_cast<int>((args.sparse_size + kTile - 1) / kTile);
        const int expert = tile_m / tiles_per_expert;
        const int64_t row_in_expert = static_cast<int64_t>(tile_m - expert * tiles_per_expert) * kTile;
        work.rows_valid = static_cast<int>(min(static_cast<int64_t>(kTile), args.sparse_size - row_in_expert));
        if (args.expert_ends != nullptr) {
            work.k_lo = expert > 0 ? load_index(args.expert_ends, args.index_dtype, expert - 1) : 0;
            work.k_hi = load_index(args.expert_pad_begins, args.index_dtype, expert);
            work.k_lo = max(work.k_lo, static_cast<int64_t>(0));
            work.k_hi = min(work.k_hi, args.inner);
        }
        work.lhs_offset = row_in_expert * args.lhs_stride_row;
        work.rhs_offset = col0 * args.rhs_stride_col;
        work.out_offset = (expert * args.sparse_size + row_in_expert) * args.out_stride_row + col0;
        return true;
    }
    int expert;
    int64_t row0;
    if (!find_row_tile(args, tile_m, expert, row0, work.rows_valid)) return false;
    work.lhs_offset = row0 * args.lhs_stride_row;
    work.out_offset = row0 * args.out_stride_row + col0;
    if (args.mode == kOutputSparse)
        work.rhs_offset = (static_cast<int64_t>(expert) * args.sparse_size + col0) * args.rhs_stride_col;
    else
        work.rhs_offset =
            static_cast<int64_t>(expert) * args.sparse_size * args.rhs_stride_inner + col0 * args.rhs_stride_col;
    return true;
}

// Hardware workgroup id -> (row tile, column tile): contiguous runs per XCD, 8 row tiles per column tile.
__device__ __forceinline__ void tile_of_block(const GemmArgs &args, int &tile_m, int &tile_n) {
    constexpr int kXcds = 8, kGroupRows = 8;
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

// ---- the kernel ----------------------------------------------------------------------------------------
template <typename OutT>
__device__ __forceinline__ void store_tile(const f32x16_t (&acc)[4][2], OutT *out, int64_t stride, int rows_valid,
                                           int cols_valid, bool accumulate, int wave_m, int wave_n, int lane) {
    // Accumulator register v of lane l in a 32x32 tile: row 8 (v / 4) + 4 (l / 32) + v % 4, column l % 32.
#pragma unroll
    for (int i = 0; i < 4; ++i) {
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const int column = wave_n * kWaveCols + j * 32 + (lane & 31);
            if (column >= cols_valid) continue;
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int row = wave_m * kWaveRows + i * 32 + 8 * (v >> 2) + 4 * (lane >> 5) + (v & 3);
                if (row >= rows_valid) continue;
                OutT *pointer = out + row * stride + column;
                float value = acc[i][j][v];
                if (accumulate) value += to_float(*pointer);
                *pointer = from_float<OutT>(value);
            }
        }
    }
}

template <typename T, bool kLhsContiguousK, bool kRhsContiguousK>
__global__ __launch_bounds__(kMfmaThreads, 2) void grouped_gemm_mfma_kernel(GemmArgs args) {
    extern __shared__ __attribute__((aligned(1024))) char lds_generic[];
    FM_LDS(char) *lds = (FM_LDS(char) *)(lds_generic);  // C-style: address-space cast

    int tile_m, tile_n;
    tile_of_block(args, tile_m, tile_n);
    TileWork work;
    if (!resolve_tile(args, tile_m, tile_n, work)) return;

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int wave_m = wave >> 2, wave_n = wave & 3;
    const bool masked = args.mode == kInputRowSparse;
    const int64_t k_first = work.k_lo / kBK * kBK;
    const int64_t k_last = work.k_hi > work.k_lo ? (work.k_hi + kBK - 1) / kBK * kBK : k_first;
    const int num_steps = static_cast<int>((k_last - k_first) / kBK);

    TileLoader<kLhsContiguousK> load_lhs;
    TileLoader<kRhsContiguousK> load_rhs;
    {
        const char *lhs = static_cast<const char *>(args.lhs) +
                          (work.lhs_offset + k_first * args.lhs_stride_inner) * static_cast<int64_t>(sizeof(T));
        const char *rhs = static_cast<const char *>(args.rhs) +
                          (work.rhs_offset + k_first * args.rhs_stride_inner) * static_cast<int64_t>(sizeof(T));
        load_lhs.setup(lhs, (kLhsContiguousK ? args.lhs_stride_row : args.lhs_stride_inner) * sizeof(T),
                       work.rows_valid, wave, lane);
        load_rhs.setup(rhs, (kRhsContiguousK ? args.rhs_stride_col : args.rhs_stride_inner) * sizeof(T),
                       work.cols_valid, wave, lane);
    }

    f32x16_t acc[4][2];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

    if (num_steps > 0) {
        load_lhs.issue(lds, wave);
        load_rhs.issue(lds + kOperandBytes, wave);
    }
    for (int step = 0; step < num_steps; ++step) {
        FM_LDS(char) *stage = lds + (step & 1) * kStageBytes;
        // This wavefront's loads of `stage` have landed; after the barrier everybody's have, and everybody is done
        // reading the other stage, which the next loads overwrite.
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        if (masked) {
            const int64_t k0 = k_first + static_cast<int64_t>(step) * kBK;
            if (k0 < work.k_lo || k0 + kBK > work.k_hi) {
                mask_tile<kLhsContiguousK>(stage, k0, work.k_lo, work.k_hi);
                mask_tile<kRhsContiguousK>(stage + kOperandBytes, k0, work.k_lo, work.k_hi);
                __syncthreads();
            }
        }
        if (step + 1 < num_steps) {
            FM_LDS(char) *next = lds + ((step + 1) & 1) * kStageBytes;
            load_lhs.issue(next, wave);
            load_rhs.issue(next + kOperandBytes, wave);
        }
#pragma unroll
        for (int kstep = 0; kstep < kBK / 16; ++kstep) {
            u32x4_t frag_a[4], frag_b[2];
#pragma unroll
            for (int i = 0; i < 4; ++i)
                frag_a[i] = load_fragment<kLhsContiguousK>(stage, wave_m * kWaveRows + i * 32, kstep, lane);
#pragma unroll
            for (int j = 0; j < 2; ++j)
                frag_b[j] =
                    load_fragment<kRhsContiguousK>(stage + kOperandBytes, wave_n * kWaveCols + j * 32, kstep, lane);
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 2; ++j) acc[i][j] = Mfma<T>::run(frag_a[i], frag_b[j], acc[i][j]);
        }
    }

    const bool accumulate = args.accumulate != 0;
    if (accumulate && num_steps == 0) return;  // nothing to add
    if (args.out_dtype == FM_DTYPE_F32)
        store_tile(acc, static_cast<float *>(args.out) + work.out_offset, args.out_stride_row, work.rows_valid,
                   work.cols_valid, accumulate, wave_m, wave_n, lane);
    else if (args.out_dtype == FM_DTYPE_BF16)
        store_tile(acc, static_cast<bf16_t *>(args.out) + work.out_offset, args.out_stride_row, work.rows_valid,
                   work.cols_valid, accumulate, wave_m, wave_n, lane);
    else
        store_tile(acc, static_cast<f16_t *>(args.out) + work.out_offset, args.out_stride_row, work.rows_valid,
                   work.cols_valid, accumulate, wave_m, wave_n, lane);
}

// ---- host side -----------------------------------------------------------------------------------------
template <typename T, bool kLhsK, bool kRhsK>
static int launch_instance(const GemmArgs &args, hipStream_t stream) {
    auto kernel = grouped_gemm_mfma_kernel<T, kLhsK, kRhsK>;
    static bool configured = false;  // setting the attribute twice from racing threads is harmless
    if (!configured) {
        hipError_t error = hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                                               hipFuncAttributeMaxDynamicSharedMemorySize, kLdsBytes);
        if (error != hipSuccess) return fail(FM_ERR_LAUNCH, "hipFuncSetAttribute: %s", hipGetErrorString(error));
        configured = true;
    }
    kernel<<<args.tiles_m * args.tiles_n, kMfmaThreads, kLdsBytes, stream>>>(args);
    return FM_OK;
}

template <typename T>
static int launch_layout(const GemmArgs &args, hipStream_t stream) {
    const bool lhs_k = args.lhs_stride_inner == 1, rhs_k = args.rhs_stride_inner == 1;
    if (lhs_k && rhs_k) return launch_instance<T, true, true>(args, stream);
    if (lhs_k) return launch_instance<T, true, false>(args, stream);
    if (rhs_k) return launch_instance<T, false, true>(args, stream);
    return launch_instance<T, false, false>(args, stream);
}

static bool vector_ok(const void *pointer, int64_t stride) { return aligned16(pointer) && stride % 8 == 0; }

bool mfma_gemm_eligible(const GemmArgs &args, int dtype) {
    if (dtype == FM_DTYPE_F32 || args.out_stride_col != 1) return false;
    const bool lhs_k = args.lhs_stride_inner == 1, lhs_m = args.lhs_stride_row == 1;
    const bool rhs_k = args.rhs_stride_inner == 1, rhs_n = args.rhs_stride_col == 1;
    if (!(lhs_k || lhs_m) || !(rhs_k || rhs_n)) return false;
    if (!vector_ok(args.lhs, lhs_k ? args.lhs_stride_row : args.lhs_stride_inner)) return false;
    if (!vector_ok(args.rhs, rhs_k ? args.rhs_stride_col : args.rhs_stride_inner)) return false;
    // The reduction axis is walked in whole 64-element tiles that must exist in memory; 16-byte chunks along the
    // contiguous axis of a row-contiguous operand must not straddle the end of an expert's block.
    if (args.inner <= 0 || args.inner % kBK != 0 || args.sparse_size % 8 != 0 || args.cols % 8 != 0) return false;
    if (!lhs_k && args.mode != kInputRowSparse && args.rows % 8 != 0) return false;
    return true;
}

int mfma_gemm_launch(GemmArgs args, int dtype, hipStream_t stream) {
    if (args.mode == kInputRowSparse) {
        args.tiles_m = static_cast<int>((args.sparse_size + kTile - 1) / kTile) * args.num_experts;
    } else {
        // Upper bound of sum_e ceil(rows_e / 256); surplus workgroups find no tile and exit.
        args.tiles_m = static_cast<int>((args.rows + kTile - 1) / kTile + (args.expert_ends ? args.num_experts : 0));
    }
    args.tiles_n = static_cast<int>((args.cols + kTile - 1) / kTile);
    if (static_cast<int64_t>(args.tiles_m) * args.tiles_n >= (int64_t(1) << 31))
        return fail(FM_ERR_UNSUPPORTED, "grouped gemm: too many tiles");
    return dtype == FM_DTYPE_BF16 ? launch_layout<bf16_t>(args, stream) : launch_layout<f16_t>(args, stream);
}

}  // namespace fm
