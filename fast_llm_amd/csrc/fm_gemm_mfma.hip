// Grouped matrix products on the gfx950 matrix cores (bf16 / fp16 operands, fp32 accumulation).
//
// One workgroup = 4 wavefronts = one 256 x 256 tile of `out`, reduced one K-slice (kBK = 64 elements) at a time:
//   * Operand slices are loaded straight into LDS (`buffer_load ... lds`), never through registers. A slot that is
//     being filled cannot be read, so LDS (160 KiB = five slices of 32 KiB) is split into three lhs and two rhs
//     slots: lhs loads run two slices ahead and are issued evenly, rhs loads are issued in the half slice after
//     their slot is released. One barrier per slice, placed before the last K-step of a slice, whose MFMAs overlap
//     the first fragment reads of the next slice.
//   * An operand may be contiguous along K (activations [rows, K], `weight.t()`) or along its other axis
//     (`weight` [K, N], `activations.t()`). K-contiguous tiles are stored [row][K] and read as 128-bit MFMA
//     fragments; the others are stored [K][row] as they lie in memory and read with the LDS transpose load
//     `ds_read_b64_tr_b16`, which hands every lane four consecutive K values of one row. Both layouts are
//     XOR-swizzled so that the fragment reads hit all 64 banks; the swizzle is applied when choosing which 16-byte
//     chunk a lane fetches.
//   * Wavefronts form a 2 x 2 grid, one per SIMD, each owns 128 x 128 of the tile as 4 x 4 accumulators of
//     v_mfma_f32_32x32x16 (256 accumulation registers per lane). A single wavefront keeps the matrix pipe busy as
//     long as its MFMAs are back to back, so every K-step is a fixed sequence of "one MFMA, one memory instruction
//     in its shadow".
//   * Tiles never straddle experts: the row tiles of an expert are enumerated from `expert_ends` on the device
//     (ceil(rows_e / 256) each), a last partial tile stores only its valid rows, so any padding multiple works and
//     phantom rows past the last expert are never touched. For the row-sparse product the reduction runs over
//     [begin_e, pad_begin_e); what a K-slice holds outside that range is zeroed in LDS before it is multiplied
//     (zero-fill, not multiply-by-zero, so NaN in padding rows cannot leak).
//   * The loop has no branch around a transfer: the range of the buffer descriptors makes loads past the last slice
//     (and rows past a partial tile of a K-contiguous operand) bring zeros.
//   * The tile is written through LDS, already rounded to the output type, as 16-byte streaming stores that cover
//     full 256-byte row segments.
//   * Hardware hands consecutive workgroup ids to the 8 XCDs round-robin; ids are renumbered so that the tiles an XCD
//     runs at the same time are about 8 row tiles x 4 column tiles of one expert, which re-read operands from its L2.
//   * The grid is one workgroup per CU; a workgroup walks its share of the tiles and issues the first loads of a
//     tile before it writes the previous one out. With a workspace from the caller, where a tile lies is looked up
//     in a table that a small kernel fills first (one scalar load instead of a scan of the expert map per tile),
//     and, when a launch has few rounds of long tiles, the reductions of the last round's tiles are split over the
//     idle CUs and a second kernel adds the pieces in a fixed order.
// Results are deterministic: one workgroup per output tile (or a fixed split), fixed summation order, no atomics.
#include <type_traits>

#include "fm_activation_math.h"
#include "fm_gemm_common.h"

#include <atomic>

namespace fm {

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8_t;
typedef __attribute__((__vector_size__(8 * sizeof(_Float16)))) _Float16 f16x8_t;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float f32x16_t;
typedef __attribute__((__vector_size__(4 * sizeof(uint32_t)))) uint32_t u32x4_t;
typedef __attribute__((__vector_size__(2 * sizeof(uint32_t)))) uint32_t u32x2_t;
typedef __attribute__((__vector_size__(4 * sizeof(short)))) short i16x4_t;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float f32x4_t;

// Four consecutive output elements, moved as one 8- or 16-byte access.
template <typename T>
struct alignas(4 * sizeof(T)) Vec16x4 {
    T v[4];
};

// The output tile is written once and not read again by this kernel: keep it from displacing operand panels in L2.
template <typename T>
__device__ __forceinline__ void store_streaming(T *pointer, const Vec16x4<T> &value) {
    typedef __attribute__((__vector_size__(4 * sizeof(T)))) std::conditional_t<sizeof(T) == 4, uint32_t, uint16_t> Raw;
    __builtin_nontemporal_store(__builtin_bit_cast(Raw, value), reinterpret_cast<Raw *>(pointer));
}

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

constexpr int kTile = 256;
constexpr int kWavesM = 2, kWavesN = 2;  // wavefront grid over the tile
constexpr int kWaves = kWavesM * kWavesN, kMfmaThreads = 64 * kWaves;
constexpr int kBK = 64;      // K elements per slice (32 or 64)
constexpr int kStages = 2;     // LDS slots of the rhs operand
constexpr int kLhsStages = 3;  // LDS slots of the lhs operand
constexpr int kOperandBytes = kTile * kBK * 2;  // one operand slice in LDS, same size in either layout
constexpr int kLdsBytes = (kStages + kLhsStages) * kOperandBytes;  // the rhs slots, then the lhs slots
constexpr int kWaveRows = kTile / kWavesM, kWaveCols = kTile / kWavesN;  // a wavefront's part of the tile
constexpr int kTilesM = kWaveRows / 32, kTilesN = kWaveCols / 32;        // in 32x32 MFMA accumulators
constexpr int kChunksPerRow = kBK / 8;          // 16-byte chunks of a K-major row
constexpr int kLoadsPerOperand = kOperandBytes / 16 / kMfmaThreads;  // 16-byte loads per lane, operand and slice
constexpr int kBufferResourceFlags = 0x00020000;  // raw buffer, 32-bit data format, no swizzle
constexpr int kEpiloguePadBytes = 16;  // after each staged row of the epilogue; keeps 16-byte alignment and spreads
                                       // the rows over the banks
constexpr int kStagingBase = kOperandBytes;  // the epilogue stages rows in LDS from here up to the last lhs slot
static_assert(kBK == 64 && kLoadsPerOperand == 8, "pipeline shape");
static_assert(kLdsBytes <= 160 * 1024 && kStagingBase + kWaves * 32 * (kWaveCols * 4 + kEpiloguePadBytes) <=
                                             kLdsBytes - kOperandBytes,
              "LDS budget: staging between rhs slot 0 and the last lhs slot");

// ---- LDS layouts ---------------------------------------------------------------------------------------
// K-contiguous operand, [256 rows][kBK k]: 16-byte chunk c (8 k values) of row r sits at
// r * 2 kBK + (c ^ swizzle(r)) * 16 with swizzle(r) = (r / rows-per-256-bytes) mod chunks-per-row.
// The 16 lanes that read one chunk column of 16 consecutive rows then cover all 64 banks.
__device__ __forceinline__ int k_major_swizzle(int row) {
    return (row / (128 / kBK)) & (kChunksPerRow - 1);
}
__device__ __forceinline__ int lds_offset_k_major(int row, int chunk) {
    return row * (kBK * 2) + ((chunk ^ k_major_swizzle(row)) << 4);
}
// Row-contiguous operand, [kBK k][256 rows]: the 32-byte group g (16 rows) of K-row k sits at k * 512 + (g ^ (2 * (k & 3))) * 32.
// A transpose load by 32 lanes touches 4 K-rows x 2 groups; the XOR sends them to 8 different bank octets.
__device__ __forceinline__ int lds_offset_row_major(int k, int row) {
    return k * (kTile * 2) + ((((row >> 4) ^ ((k & 3) << 1)) << 5) | ((row & 15) << 1));
}

// The same value, but the compiler cannot tell: what is computed from it is computed where it is written, not hoisted
// out of an enclosing loop into registers that stay occupied across the loop.
__device__ __forceinline__ int opaque(int value) {
    asm volatile("" : "+v"(value));
    return value;
}

// Tell the compiler that a pointer computed from tile coordinates is the same in every lane (it then lives in
// scalar registers and the loads use the scalar-base addressing form).
__device__ __forceinline__ const char *uniform_pointer(const char *pointer) {
    const uint64_t bits = reinterpret_cast<uint64_t>(pointer);
    const uint32_t low = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(bits));
    const uint32_t high = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(bits >> 32));
    return reinterpret_cast<const char *>((static_cast<uint64_t>(high) << 32) | low);
}

__device__ __forceinline__ int64_t uniform_int64(int64_t value) {
    const uint32_t low = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(value));
    const uint32_t high = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(static_cast<uint64_t>(value) >> 32));
    return static_cast<int64_t>((static_cast<uint64_t>(high) << 32) | low);
}

// Loader of one operand slice: global memory -> LDS, without passing through registers (`buffer_load ... lds`: lane
// l of the wavefront fetches 16 bytes at its own offset and the hardware puts them at M0 + 16 l in LDS; lanes outside
// the descriptor's range bring zeros). Writing LDS from registers instead (ds_write_b128) sustains only ~78 bytes per
// cycle and CU, a third of the LDS read rate, and was the busiest pipe of this kernel.
// The slice is 256 * kBK / 8 chunks of 16 bytes; chunk slot p of the LDS slice is fetched by lane p % 64 of wavefront
// (p / 64) / kLoadsPerOperand as its load number (p / 64) % kLoadsPerOperand, so a load instruction fills 1 KiB of
// consecutive LDS and the swizzle is applied on the global side (which chunk a lane fetches).
// The compiler does not see these loads: whoever reads a slot counts the loads issued since (`s_waitcnt vmcnt`, loads
// complete in order) and passes a barrier first.
// `kHalves` (row-contiguous only): loads 0..3 of a wavefront fill the first 32 K-rows of the slot and loads 4..7 the
// last 32, so that either half of a slot can be refilled on its own (see the pipeline of the kernel).
template <bool kContiguousK, bool kHalves = false>
struct TileLoader {
    static_assert(!(kContiguousK && kHalves), "only a row-contiguous slice splits into halves along K");
    // The 1 KiB block of an operand slot that load j of wavefront `wave` fills.
    static __device__ __forceinline__ int block_of(int wave, int j) {
        return kHalves ? (j >> 2) * (2 * kLoadsPerOperand) + wave * (kLoadsPerOperand / 2) + (j & 3) : wave * kLoadsPerOperand + j;
    }
    const char *fetch_base;  // wave-uniform: first row of the tile, first k of the slice being fetched
    uint32_t offset[2];      // per lane, bytes from `fetch_base`, of loads 0 and 1 (fits 32 bits: checked on the host)
    uint32_t pair_stride;    // wave-uniform: bytes from load j to load j + 2 (the swizzles repeat with period 2)
    uint32_t num_records;    // wave-uniform: lane offsets >= this bring zeros
    int64_t step;            // bytes from one slice to the next
    int slices_left;         // slices after the one being fetched
    uint32_t last_records;   // row-contiguous: `num_records` of the last slice (its K-rows past the reduction range
                             // bring zeros)
    int wave_index;          // wave-uniform

    // `stride`: bytes between rows (K-contiguous) or between K-rows (row-contiguous). Rows >= valid_rows are never
    // stored; a K-contiguous operand gets zeros for them (they lie past the range of the buffer descriptor), a
    // row-contiguous one gets in-range rows in their place.
    // `split_rows` (K-contiguous only, 0: off): rows 64..127 and 192..255 of the tile are not the rows after 0..63 and
    // 128..191 but lie `split_rows` rows after them, i.e. tile row n is memory row
    // (n / 128) * 64 + n % 64 + (n / 64 % 2) * split_rows (the gate and up halves of a gated layer's weight).
    // `k_count`: reduction indices from the first one of slice 0 to the end of the reduction range; a row-contiguous
    // operand gets zeros for the K-rows of its last slice that lie past it.
    __device__ __forceinline__ void setup(const char *tile_base, int64_t stride, int valid_rows, int num_slices,
                                          int k_count, int wave, int lane, int split_rows = 0) {
        static_assert(kLoadsPerOperand % 2 == 0, "loads come in (even, odd) pairs");
        fetch_base = tile_base;
        slices_left = num_slices - 1;
        wave_index = wave;
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const int slot = block_of(wave, j) * 64 + lane;
            if constexpr (kContiguousK) {
                const int row = slot / kChunksPerRow;
                const int chunk = (slot % kChunksPerRow) ^ k_major_swizzle(row);
                const int64_t memory_row =
                    split_rows == 0 ? row : (row >> 7) * 64 + (row & 63) + static_cast<int64_t>((row >> 6) & 1) * split_rows;
                offset[j] = static_cast<uint32_t>(memory_row * stride + chunk * 16);
            } else {
                const int k = slot >> 5, position = slot & 31;
                const int group = (position >> 1) ^ ((k & 3) << 1);
                int first_row = (group * 2 + (position & 1)) * 8;
                if (first_row >= valid_rows) first_row = 0;
                offset[j] = static_cast<uint32_t>(k * stride + first_row * 2);
            }
        }
        // Two loads further on: 128 slots = 16 rows of a K-contiguous slice, 4 K-rows of a row-contiguous one.
        pair_stride = static_cast<uint32_t>((kContiguousK ? 128 / kChunksPerRow : 4) * stride);
        const int64_t last_row = split_rows == 0 ? valid_rows - 1 : split_rows + kTile / 2 - 1;
        step = kContiguousK ? kBK * 2 : kBK * stride;
        if constexpr (kContiguousK) {
            num_records = last_records = static_cast<uint32_t>(last_row * stride + kBK * 2);
        } else {
            last_records = static_cast<uint32_t>((k_count - (num_slices - 1) * kBK) * stride);
            num_records = num_slices == 1 ? last_records : 0xffffffffu;
        }
    }

    // Move on to the next slice. Past the last slice the descriptor's range becomes empty, so that every further
    // load fills LDS with zeros without touching memory: the pipeline can run a slice too far without a branch.
    __device__ __forceinline__ void advance() {
        // Said to be wave-uniform once more: loop-carried values otherwise end up in vector registers.
        fetch_base = uniform_pointer(fetch_base + step);
        slices_left = __builtin_amdgcn_readfirstlane(slices_left - 1);
        num_records = __builtin_amdgcn_readfirstlane(slices_left < 0 ? 0u : (slices_left == 0 ? last_records : num_records));
    }

    // Chunk j of the slice being fetched -> the operand slot that starts at LDS byte address `slot_address`.
    // Buffer load: scalar base (in the resource descriptor) + 32-bit lane offset, so the addresses cost two registers
    // per operand and advancing to the next slice is scalar arithmetic.
    __device__ __forceinline__ void load(int slot_address, int j) {
        const __amdgpu_buffer_rsrc_t resource = __builtin_amdgcn_make_buffer_rsrc(
            const_cast<char *>(uniform_pointer(fetch_base)), 0,
            static_cast<int>(__builtin_amdgcn_readfirstlane(num_records)), kBufferResourceFlags);
        // Two loads further on the blocks are two further on (`pair_stride`); with halves, four loads further on they
        // are 16 further on: 32 K-rows, eight times the four K-rows of `pair_stride`.
        const uint32_t lane_offset =
            offset[j & 1] + static_cast<uint32_t>(kHalves ? ((j >> 1) & 1) + 8 * (j >> 2) : j >> 1) * pair_stride;
        // M0 = slot + the wavefront's part of the block number + the load's part: the last addition is made into M0
        // itself, with the load's part as an immediate (one scalar instruction per load instead of two).
        const int wave_address = __builtin_amdgcn_readfirstlane(slot_address + block_of(wave_index, 0) * 1024);
        // M0 is not handed out by the register allocator and nothing else in this file uses it.
        asm volatile("s_add_i32 m0, %0, %3\n\tbuffer_load_dwordx4 %1, %2, 0 offen lds"
                     :
                     : "s"(wave_address), "v"(lane_offset), "s"(resource), "n"((block_of(0, j) - block_of(0, 0)) * 1024)
                     : "memory", "scc");
    }
};

// Returns once at most `kNewest` of the loads this wavefront has issued are still on their way.
template <int kNewest>
__device__ __forceinline__ void wait_for_loads() {
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(kNewest) : "memory");
}

// MFMA operand fragments (8 consecutive k of one row per lane; lane l: row l % 32, k half l / 32). A wavefront reads
// 4 fragments (32 rows each, `i`) for each of the 4 K-steps of a slice, from either LDS slot. Thanks to the period of
// the swizzles, 4 per-lane addresses per operand are enough; everything else is an immediate offset of the LDS
// instruction: a K-contiguous operand needs one address per K-step (fragment i is 32 rows = 4 KiB further on), a
// row-contiguous one needs one per fragment (K-step s is 16 K-rows = 8 KiB further on).
template <bool kContiguousK>
__device__ __forceinline__ int fragment_base(int row_base, int q, int lane) {
    if constexpr (kContiguousK) {
        return lds_offset_k_major(row_base + (lane & 31), q * 2 + (lane >> 5));
    } else {
        // ds_read_b64_tr_b16 works on groups of 16 lanes: lane s of a group supplies the address of 4 rows
        // (row0 + 4 (s % 4) ..) at K-row k0 + s / 4 and receives k0 .. k0 + 3 of row row0 + s.
        const int s = lane & 15, group = lane >> 4;
        const int row = row_base + q * 32 + ((group & 1) << 4) + ((s & 3) << 2);
        const int k = ((group >> 1) << 3) + (s >> 2);
        return lds_offset_row_major(k, row);
    }
}
// `bases`: fragment_base of q = 0..3 plus the LDS offset of the operand's slot 0.
template <bool kContiguousK>
__device__ __forceinline__ u32x4_t load_fragment(FM_LDS(char) * lds, const int (&bases)[4], int slot, int i, int kstep) {
    // The kernel's only LDS is the dynamic allocation, which starts at LDS address 0 (the transfers above put absolute
    // addresses into M0 as well). The address of that array is not a constant the compiler knows, though: formed as
    // `lds + offset`, every fragment address costs an addition of zero in the main loop.
    (void)lds;
    if constexpr (kContiguousK) {
        return *(FM_LDS(u32x4_t) *)static_cast<uint32_t>(bases[kstep] + (slot * kOperandBytes + i * 32 * kBK * 2));
    } else {
        FM_LDS(char) *address = (FM_LDS(char) *)static_cast<uint32_t>(bases[i] + (slot * kOperandBytes + kstep * 16 * kTile * 2));
        const i16x4_t low = __builtin_amdgcn_ds_read_tr16_b64_v4i16(reinterpret_cast<FM_LDS(i16x4_t) *>(address));
        const i16x4_t high =
            __builtin_amdgcn_ds_read_tr16_b64_v4i16(reinterpret_cast<FM_LDS(i16x4_t) *>(address + 4 * kTile * 2));
        const u32x2_t low_words = __builtin_bit_cast(u32x2_t, low), high_words = __builtin_bit_cast(u32x2_t, high);
        return u32x4_t{low_words[0], low_words[1], high_words[0], high_words[1]};
    }
}

// Zero, in a slice that sits in LDS and whose first reduction index is k0, everything whose reduction index is
// outside [k_lo, k_hi). Runs between two barriers, for the first/last slice of a ragged reduction range only.
template <bool kContiguousK>
__device__ __forceinline__ void mask_tile(FM_LDS(char) * operand_lds, int k0, int k_lo, int k_hi) {
    for (int slot = opaque(static_cast<int>(threadIdx.x)); slot < kOperandBytes / 16; slot += kMfmaThreads) {
        FM_LDS(u32x4_t) *pointer = reinterpret_cast<FM_LDS(u32x4_t) *>(operand_lds + slot * 16);
        if constexpr (kContiguousK) {
            const int row = slot / kChunksPerRow;
            const int k = k0 + (((slot % kChunksPerRow) ^ k_major_swizzle(row)) << 3);
            if (k >= k_lo && k + 8 <= k_hi) continue;
            u32x4_t value = *pointer;
#pragma unroll
            for (int w = 0; w < 4; ++w) {
                uint32_t word = value[w];
                if (k + 2 * w < k_lo || k + 2 * w >= k_hi) word &= 0xffff0000u;
                if (k + 2 * w + 1 < k_lo || k + 2 * w + 1 >= k_hi) word &= 0x0000ffffu;
                value[w] = word;
            }
            *pointer = value;
        } else {
            const int k = k0 + (slot >> 5);
            if (k < k_lo || k >= k_hi) *pointer = u32x4_t{0, 0, 0, 0};
        }
    }
}

// ---- which tile ----------------------------------------------------------------------------------------
struct TileWork {
    int64_t lhs_offset, rhs_offset, out_offset;  // elements
    int64_t fused_offset;                        // of the tile in `fused_out`, elements
    int rows_valid, cols_valid;
    int64_t k_lo, k_hi;
};

constexpr int kXcds = 8, kGroupRows = 8, kChunkTiles = 32;
constexpr int kHalfTileMaxSlices = 64;  // reductions of this many slices or more have no half tiles (see find_tile)

// Logical order of the tiles of a product whose rows are grouped by expert (output-sparse, input-inner-sparse,
// dense): expert after expert; within an expert its row tiles (ceil(rows_e / 256)) are cut into ceil(count / 8)
// groups of nearly equal size (9 row tiles: 5 + 4), and a group is walked column tile by column tile, row tiles
// fastest. 32 consecutive tiles (what an XCD runs at one time) are then about 8 row tiles x 4 column tiles of ONE
// expert, i.e. 8 lhs panels and 4 rhs panels shared in that XCD's L2; with groups that ignore the expert boundaries
// most chunks straddled two experts and needed twice the rhs panels.
// Every wavefront scans `expert_ends` 64 experts at a time; returns false if `logical` is past the last tile.
struct RowTile {
    int expert, tile_n, rows_valid;
    int64_t row0;
};

__device__ __forceinline__ void place_in_expert(int local, int count, int tiles_n, int &row_tile, int &tile_n) {
    const int groups = (count + kGroupRows - 1) / kGroupRows;
    const int base = count / groups, larger = count % groups;  // the first `larger` groups have base + 1 row tiles
    const int larger_tiles = larger * (base + 1) * tiles_n;
    int first_row, rows, in_group;
    if (local < larger_tiles) {
        const int group = local / ((base + 1) * tiles_n);
        rows = base + 1;
        first_row = group * rows;
        in_group = local - group * rows * tiles_n;
    } else {
        const int rest = local - larger_tiles;
        const int group = rest / (base * tiles_n);
        rows = base;
        first_row = larger * (base + 1) + group * rows;
        in_group = rest - group * rows * tiles_n;
    }
    row_tile = first_row + in_group % rows;
    tile_n = in_group / rows;
}

__device__ __forceinline__ bool locate_tile(const GemmArgs &args, int logical, RowTile &tile) {
    const int tiles_n = args.tiles_n;
    if (args.expert_ends == nullptr) {
        const int count = static_cast<int>((args.rows + kTile - 1) / kTile);
        if (logical >= count * tiles_n) return false;
        int row_tile;
        place_in_expert(logical, count, tiles_n, row_tile, tile.tile_n);
        tile.expert = 0;
        tile.row0 = static_cast<int64_t>(row_tile) * kTile;
        tile.rows_valid = static_cast<int>(min(static_cast<int64_t>(kTile), args.rows - tile.row0));
        return true;
    }
    const int lane = opaque(static_cast<int>(threadIdx.x & 63));
    int tiles_before = 0;  // row tiles of the experts before this block of 64
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
        if (logical < (tiles_before + total) * tiles_n) {
            const uint64_t owners = __ballot((tiles_before + inclusive) * tiles_n > logical);
            const int owner = __ffsll(static_cast<unsigned long long>(owners)) - 1;
            const int owner_count = __shfl(count, owner, 64);
            const int first_tile = tiles_before + __shfl(inclusive - count, owner, 64);
            const int64_t owner_begin = __shfl(begin, owner, 64), owner_end = __shfl(end, owner, 64);
            int row_tile;
            place_in_expert(logical - first_tile * tiles_n, owner_count, tiles_n, row_tile, tile.tile_n);
            tile.expert = base + owner;
            tile.row0 = owner_begin + static_cast<int64_t>(row_tile) * kTile;
            tile.rows_valid = static_cast<int>(min(static_cast<int64_t>(kTile), owner_end - tile.row0));
            return true;
        }
        tiles_before += total;
    }
    return false;
}

// Logical tile -> (row tile, column tile) for the row-sparse product, whose row tiles are expert-aligned by
// construction: groups of 8 row tiles, column by column inside a group.
__device__ __forceinline__ void tile_coordinates(int logical, int tiles_m, int tiles_n, int &tile_m, int &tile_n) {
    const int width = kGroupRows * tiles_n;
    const int group = logical / width;
    const int first_m = group * kGroupRows;
    const int group_rows = min(tiles_m - first_m, kGroupRows);
    const int in_group = logical - group * width;
    tile_m = first_m + in_group % group_rows;
    tile_n = in_group / group_rows;
}

// Where the operands and the output of logical tile `logical` are. False: there is no such tile.
__device__ __forceinline__ bool resolve_tile(const GemmArgs &args, int logical, TileWork &work) {
    work.k_lo = 0;
    work.k_hi = args.inner;
    work.fused_offset = 0;
    if (args.mode == kInputRowSparse) {
        if (logical >= args.tiles_m * args.tiles_n) return false;
        int tile_m, tile_n;
        tile_coordinates(logical, args.tiles_m, args.tiles_n, tile_m, tile_n);
        const int64_t col0 = static_cast<int64_t>(tile_n) * kTile;
        work.cols_valid = static_cast<int>(min(static_cast<int64_t>(kTile), args.cols - col0));
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
    RowTile tile;
    if (!locate_tile(args, logical, tile)) return false;
    // A tile of the fused gated forward product has 128 gate columns (and their up columns).
    const bool paired = args.fusion == kFusionGatedForward;
    const int64_t col0 = static_cast<int64_t>(tile.tile_n) * (paired ? kTile / 2 : kTile);
    work.cols_valid = paired ? kTile : static_cast<int>(min(static_cast<int64_t>(kTile), args.cols - col0));
    work.rows_valid = tile.rows_valid;
    work.lhs_offset = tile.row0 * args.lhs_stride_row;
    work.out_offset = tile.row0 * args.out_stride_row + col0;
    work.fused_offset = tile.row0 * args.fused_stride + col0;
    if (args.mode == kOutputSparse)
        work.rhs_offset = (static_cast<int64_t>(tile.expert) * args.sparse_size + col0) * args.rhs_stride_col;
    else
        work.rhs_offset =
            static_cast<int64_t>(tile.expert) * args.sparse_size * args.rhs_stride_inner + col0 * args.rhs_stride_col;
    return true;
}

// Hardware workgroup id -> position in the logical tile order. The hardware hands consecutive workgroup ids to the
// 8 XCDs in turn, so the 32 CUs of XCD x run the ids x, x + 8, x + 16, ... in that order. Those are mapped to chunks
// of 32 consecutive logical tiles, chunk c going to XCD c % 8: the tiles an XCD runs at the same time are then one
// chunk, i.e. 8 row tiles x 4 column tiles that share operand panels in that XCD's L2, while consecutive chunks go to
// different XCDs, so that experts with many and with few tokens (long and short tiles of the row-sparse product)
// are spread over all of them. A permutation of every aligned block of 256 ids.
constexpr int kRound = kXcds * kChunkTiles;  // workgroups that run at the same time: one per CU
constexpr int kSlotRotation = 5;
__device__ __forceinline__ int logical_of_block(int pid) {
    const int xcd = pid % kXcds, local = pid / kXcds;
    // Which tile of its chunk a CU takes rotates from round to round: the last row tiles of the experts, which are
    // often half tiles and shorter, would otherwise always fall to the same CUs, and those would run further and
    // further ahead of the CUs they share operand panels with.
    const int round = local / kChunkTiles;
    // Which of the round's eight chunks an XCD takes rotates as well. With chunk c always on XCD c % 8 the XCDs ran
    // the products whose rows are grouped by expert at paces that differed by up to +-5 % launch after launch (the same
    // XCDs always ahead, the weight-gradient product within +-0.4 %): chunks of one residue are not the same work as
    // chunks of another (they meet the expert and row-group boundaries at different places). Rotated, every XCD sees
    // every residue (Mixtral-like step -0.9 %, measured A-B-A-B; what is left of the spread is the XCDs' own).
    return (round * kXcds + (xcd + round) % kXcds) * kChunkTiles + (local + round * kSlotRotation) % kChunkTiles;
}

// ---- splitting the reduction of the last tiles ---------------------------------------------------------------
// With T tiles and 256 CUs the launch runs in ceil(T / 256) rounds, and the last one keeps only T % 256 CUs busy: a
// large loss when there are few, long tiles (4.25 rounds cost 5). When the caller passes a workspace, the tiles of that
// last round are cut along the reduction axis into `pieces` pieces each, so that they fill the CUs; a piece writes its
// fp32 accumulators to the workspace and a second kernel adds the pieces of a tile, always in the same order, and
// stores the result. The plan is a function of the arguments and the expert map only, and every workgroup of both
// kernels computes the same one.
constexpr int kMaxPartials = 512;          // workspace slots of 256 x 256 floats
constexpr int kMinPieceSlices = 16;        // do not cut a reduction into pieces shorter than this
constexpr int kPieceOverheadSlices = 8;    // set-up, prologue and epilogue of a piece, in slice times
constexpr int kPartialFloats = kTile * kTile;

struct SplitPlan {
    int tiles_m;       // row tiles that exist
    int whole;         // logical tiles [0, whole) are computed by one workgroup each
    int tail;          // the tiles after them
    int pieces;        // pieces per tail tile (1: not split)
    int piece_slices;  // slices per piece (the last piece may have fewer)
};

// sum over experts of ceil(rows_e / 256). Wave-uniform.
__device__ __forceinline__ int count_row_tiles(const GemmArgs &args) {
    if (args.expert_ends == nullptr) return static_cast<int>((args.rows + kTile - 1) / kTile);
    const int lane = opaque(static_cast<int>(threadIdx.x & 63));
    int tiles = 0;
    for (int base = 0; base < args.num_experts; base += 64) {
        const int e = base + lane;
        int64_t begin = 0, end = 0;
        if (e < args.num_experts) {
            end = min(load_index(args.expert_ends, args.index_dtype, e), args.rows);
            begin = e > 0 ? load_index(args.expert_ends, args.index_dtype, e - 1) : 0;
        }
        int count = end > begin ? static_cast<int>((end - begin + kTile - 1) / kTile) : 0;
#pragma unroll
        for (int offset = 32; offset > 0; offset >>= 1) count += __shfl_xor(count, offset, 64);
        tiles += count;
    }
    return __builtin_amdgcn_readfirstlane(tiles);
}

// `with_pieces` false: only tiles_m, whole and tail are wanted (what a workgroup of the whole tiles needs to know; the
// search for the best cut is a dozen integer divisions).
__device__ __forceinline__ SplitPlan plan_split(const GemmArgs &args, bool with_pieces = true) {
    SplitPlan plan;
    plan.tiles_m = count_row_tiles(args);
    const int total = plan.tiles_m * args.tiles_n;
    plan.tail = total % kRound;
    plan.whole = total - plan.tail;
    plan.pieces = 1;
    const int num_slices = static_cast<int>(args.inner / kBK);
    plan.piece_slices = num_slices;
    int best = num_slices;
    if (plan.tail > 0 && with_pieces) {
#pragma unroll
        for (int split = 2; split <= 8; split *= 2) {
            if (plan.tail * split > kMaxPartials || num_slices / split < kMinPieceSlices) continue;
            const int length = ((num_slices + split - 1) / split + 1) / 2 * 2;  // even: slices are multiplied in pairs
            const int pieces = (num_slices + length - 1) / length;
            const int cost = (plan.tail * pieces + kRound - 1) / kRound * (length + kPieceOverheadSlices);
            if (cost < best) {
                best = cost;
                plan.pieces = pieces;
                plan.piece_slices = length;
            }
        }
    }
    return plan;
}

// The logical tile the workgroup `pid` of the main kernel computes, whole (piece_slot < 0) or as piece `piece` of a
// split reduction. Without a workspace, ids past the tiles that exist are weeded out later, by resolve_tile.
__device__ __forceinline__ bool tile_of_block(const GemmArgs &args, int pid, int &logical, int &piece,
                                              int &piece_slices, int &piece_slot) {
    logical = logical_of_block(pid);
    piece = 0;
    piece_slices = 0;
    piece_slot = -1;
    if (args.partials == nullptr) return true;
    SplitPlan plan = plan_split(args, false);
    if (logical >= plan.whole) {
        plan = plan_split(args);
        const int index = logical - plan.whole;
        if (index >= plan.tail * plan.pieces) return false;
        if (plan.pieces > 1) {
            piece = index / plan.tail;
            piece_slices = plan.piece_slices;
            piece_slot = index;
            logical = plan.whole + index - piece * plan.tail;
        }
    }
    return true;
}

// ---- the tile table -----------------------------------------------------------------------------------------
// What a workgroup needs to know about the tile of an id: found by `compute_tile_record` from the expert map (a scan
// of `expert_ends` with lane shuffles, a few integer divisions, a few thousand cycles), either by the workgroup itself
// or, when the caller brings a workspace, once per launch by `grouped_gemm_plan_kernel`, which leaves one record per id
// in a table that the workgroups then read with one scalar load per tile.
struct alignas(64) TileRecord {
    int64_t lhs_offset, rhs_offset, out_offset, fused_offset;  // elements
    int rows_valid, cols_valid;
    int k_lo, k_hi;    // reduction range (a piece of it for a split tile; ragged for the row-sparse product)
    int piece_slot;    // >= 0: a piece of a split reduction, stored to that workspace slot
    int found;         // 0: the id has no tile (and no later id has one)
    int unused[2];
};
static_assert(sizeof(TileRecord) == 64, "one s_load_dwordx16 per record");

// Wave-uniform result; every lane of the wavefront must call it.
__device__ __forceinline__ bool compute_tile_record(const GemmArgs &args, int id, TileRecord &record) {
    int logical, piece, piece_slices, piece_slot;
    TileWork work;
    const bool found = tile_of_block(args, id, logical, piece, piece_slices, piece_slot) && resolve_tile(args, logical, work);
    record.found = __builtin_amdgcn_readfirstlane(found);
    if (!record.found) return false;
    record.piece_slot = __builtin_amdgcn_readfirstlane(piece_slot);
    if (record.piece_slot >= 0) {  // a piece of a tile whose reduction is split (never the row-sparse product)
        work.k_lo = static_cast<int64_t>(piece) * piece_slices * kBK;
        work.k_hi = min(work.k_hi, work.k_lo + static_cast<int64_t>(piece_slices) * kBK);
    }
    record.lhs_offset = uniform_int64(work.lhs_offset);
    record.rhs_offset = uniform_int64(work.rhs_offset);
    record.out_offset = uniform_int64(work.out_offset);
    record.fused_offset = uniform_int64(work.fused_offset);
    record.rows_valid = __builtin_amdgcn_readfirstlane(work.rows_valid);
    record.cols_valid = __builtin_amdgcn_readfirstlane(work.cols_valid);
    record.k_lo = __builtin_amdgcn_readfirstlane(static_cast<int>(work.k_lo));
    record.k_hi = __builtin_amdgcn_readfirstlane(static_cast<int>(work.k_hi));
    return true;
}

// The 64 bytes in front of the records: how the launch splits its last round, for the kernel that adds the pieces.
struct alignas(64) TableHeader {
    SplitPlan plan;
};
static_assert(sizeof(TableHeader) == 64 && sizeof(TableHeader) == sizeof(TileRecord), "the header is record -1");

// One wavefront per id; the wavefront of id 0 also leaves the split plan of the launch in the table's header.
__global__ __launch_bounds__(256) void grouped_gemm_plan_kernel(GemmArgs args, TileRecord *table) {
    const int id = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (id >= args.num_ids) return;
    if (id == 0 && args.partials != nullptr) {
        const SplitPlan plan = plan_split(args);
        if ((threadIdx.x & 63) == 0) reinterpret_cast<TableHeader *>(table)[-1].plan = plan;
    }
    TileRecord record;
    record.unused[0] = record.unused[1] = 0;
    if (!compute_tile_record(args, id, record)) {
        record.lhs_offset = record.rhs_offset = record.out_offset = record.fused_offset = 0;
        record.rows_valid = record.cols_valid = record.k_lo = record.k_hi = 0;
        record.piece_slot = -1;
    }
    if ((threadIdx.x & 63) == 0) table[id] = record;
}

// ---- the kernel ----------------------------------------------------------------------------------------
// Write the wavefront's 128 x 128 accumulators through its own LDS region, 32 rows at a time. The MFMAs are issued
// with the operands swapped (rhs fragment first), so a lane holds, of each 32 x 32 accumulator, one row and four
// groups of four consecutive columns. Values are rounded to the output type first (unless they are to be added to
// what `out` holds: then they stay fp32 and are rounded once after the addition), a group goes to LDS as one 8- or
// 16-byte write, and the staged rows are read back as 16-byte chunks in row-major order, all reads of a 32-row block
// before the first store, so that a store instruction covers full 256-byte row segments.
// `source(i)` yields the wavefront's accumulators of its i-th block of 32 rows, as something indexed [j][register].
// `row_base`: first tile row of this wavefront; `blocks`: how many 32-row blocks it holds (4, or 2 in a half tile).
template <typename OutT, bool kAccumulate, typename Source>
__device__ __forceinline__ void store_tile(Source &&source, FM_LDS(char) * lds, OutT *out, int64_t stride,
                                           int rows_valid, int cols_valid, int wave, int lane, int row_base,
                                           int blocks) {
    using StageT = std::conditional_t<kAccumulate, float, OutT>;
    constexpr int kChunk = 16 / sizeof(StageT);         // elements per 16-byte chunk
    constexpr int kLanesPerRow = kWaveCols / kChunk;    // 16 or 32
    constexpr int kRowsPerRead = 64 / kLanesPerRow;     // 4 or 2
    constexpr int kReads = 32 / kRowsPerRead;           // 8 or 16
    constexpr int kRowBytes = kWaveCols * sizeof(StageT) + kEpiloguePadBytes;
    const int wave_n = wave % kWavesN;
    FM_LDS(char) *staging = lds + wave * (32 * kRowBytes);
    // (Two-byte values: a lane writes 8 bytes and the rows are 272 bytes apart, so rows r and r + 16 meet in the same
    // banks: two-way conflicts on these writes. Swapping the halves of every 16-byte chunk in half of the rows removes
    // them, measured with the bank-conflict counter, and the kernel is no faster for it: not done.)
    FM_LDS(char) *write_base = staging + (lane & 31) * kRowBytes + (lane >> 5) * 4 * sizeof(StageT);
    const int read_row = lane / kLanesPerRow, read_column = (lane % kLanesPerRow) * kChunk;
    FM_LDS(char) *read_base = staging + read_row * kRowBytes + read_column * sizeof(StageT);
    const int column_in_tile = wave_n * kWaveCols + read_column;
    // cols_valid is a multiple of 8, so a chunk of 4 or 8 columns is valid or not as a whole.
    const bool column_ok = column_in_tile < cols_valid;
    const int first_row = row_base + read_row;
    OutT *pointer = out + first_row * stride + column_in_tile;
    const bool whole_tile = rows_valid == kTile && cols_valid == kTile;
    constexpr bool kAhead = sizeof(OutT) == 2;
    Vec16x4<OutT> previous[kAccumulate && kAhead ? 2 : 1][kAccumulate ? kReads : 1];
    auto load_previous = [&](int i, Vec16x4<OutT>(&values)[kAccumulate ? kReads : 1]) {
        const OutT *source_row = pointer + static_cast<int64_t>(i) * 32 * stride;
#pragma unroll
        for (int t = 0; t < kReads; ++t, source_row += kRowsPerRead * stride)
            if (whole_tile || (first_row + i * 32 + t * kRowsPerRead < rows_valid && column_ok))
                values[t] = *reinterpret_cast<const Vec16x4<OutT> *>(source_row);
    };
#pragma unroll
    for (int i = 0; i < kTilesM; ++i) {
        if (i >= blocks) break;  // wave-uniform
        auto &&block = source(i);
        // When adding to `out`: what it holds is requested ahead of time, all chunks of a row block at once and one
        // block ahead of the block being staged, so that the loads are on their way while accumulators go through
        // LDS (loads issued one by one between the stores would each wait out a full memory latency: the compiler
        // cannot move them across stores to the same array).
        // (One block ahead only where the values are two bytes wide: two blocks of fp32 do not fit the registers.)
        if constexpr (kAccumulate && kAhead) {
            if (i == 0) load_previous(0, previous[0]);
            if (i + 1 < blocks) load_previous(i + 1, previous[(i + 1) & 1]);
        } else if constexpr (kAccumulate) {
            load_previous(i, previous[0]);
        }
#pragma unroll
        for (int j = 0; j < kTilesN; ++j)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                Vec16x4<StageT> group;
#pragma unroll
                for (int c = 0; c < 4; ++c) group.v[c] = from_float<StageT>(block[j][4 * g + c]);
                using Raw = std::conditional_t<sizeof(StageT) == 4, u32x4_t, u32x2_t>;
                *reinterpret_cast<FM_LDS(Raw) *>(write_base + (j * 32 + 8 * g) * sizeof(StageT)) =
                    __builtin_bit_cast(Raw, group);
            }
        // Only this wavefront touches its staging region and the LDS executes a wavefront's operations in order,
        // so no barrier is needed; the empty asm only keeps the compiler from moving accesses across the phases.
        asm volatile("" ::: "memory");
        u32x4_t staged[kReads];
#pragma unroll
        for (int t = 0; t < kReads; ++t)
            staged[t] = *reinterpret_cast<FM_LDS(u32x4_t) *>(read_base + t * kRowsPerRead * kRowBytes);
        // A running pointer, and no per-store checks when the whole tile is valid (wave-uniform).
        auto store_rows = [&](auto whole_tile) {
            OutT *target = pointer + static_cast<int64_t>(i) * 32 * stride;
#pragma unroll
            for (int t = 0; t < kReads; ++t, target += kRowsPerRead * stride) {
                if constexpr (!decltype(whole_tile)::value) {
                    if (!(first_row + i * 32 + t * kRowsPerRead < rows_valid && column_ok)) continue;
                }
                if constexpr (kAccumulate) {
                    const f32x4_t value = __builtin_bit_cast(f32x4_t, staged[t]);
                    Vec16x4<OutT> packed = previous[kAhead ? i & 1 : 0][t];
#pragma unroll
                    for (int c = 0; c < 4; ++c) packed.v[c] = from_float<OutT>(value[c] + to_float(packed.v[c]));
                    store_streaming(target, packed);
                } else {
                    __builtin_nontemporal_store(staged[t], reinterpret_cast<u32x4_t *>(target));
                }
            }
        };
        if (whole_tile) store_rows(std::true_type{});
        else store_rows(std::false_type{});
        asm volatile("" ::: "memory");
    }
    // vmcnt(0). The compiler cannot tell that every load above has been waited for (loads and uses sit in separate
    // conditionals) and would otherwise wait for all memory operations at the top of the caller's tile loop, in
    // launches that do not accumulate as well: there that wait held a tile's first transfers back until the previous
    // tile's stores had been acknowledged.
    if constexpr (kAccumulate) __builtin_amdgcn_s_waitcnt(0x0F70);
}

// ---- fused epilogues of the gated MLP ---------------------------------------------------------------------
// Both round the product to T first and compute from the rounded values, exactly what the separate activation
// kernels would read back from memory, so fused and unfused results are bit-identical.

// The tile is the gradient of the activation output. Per 32-row block: the lane's chunks of layer 1's output (gate and
// up, 16 bytes each) are requested first, then the accumulators go through LDS as in store_tile, and each staged
// chunk of 8 gradients becomes 8 gate and 8 up gradients (and, if asked for, the 8 recomputed outputs).
template <typename T, int kActivation>
__device__ __forceinline__ void store_tile_gated_backward(const f32x16_t (&acc)[kTilesM][kTilesN], FM_LDS(char) * lds,
                                                          T *grad_layer_1, const T *layer_1, T *activation_out,
                                                          int64_t stride, int64_t activation_stride, int64_t half,
                                                          int rows_valid, int cols_valid, int wave, int lane) {
    constexpr int kChunk = 16 / sizeof(T), kLanesPerRow = kWaveCols / kChunk, kRowsPerRead = 64 / kLanesPerRow;
    constexpr int kReads = 32 / kRowsPerRead;
    constexpr int kRowBytes = kWaveCols * sizeof(T) + kEpiloguePadBytes;
    const int wave_m = wave / kWavesN, wave_n = wave % kWavesN;
    FM_LDS(char) *staging = lds + wave * (32 * kRowBytes);
    FM_LDS(char) *write_base = staging + (lane & 31) * kRowBytes + (lane >> 5) * 4 * sizeof(T);
    const int read_row = lane / kLanesPerRow, read_column = (lane % kLanesPerRow) * kChunk;
    FM_LDS(char) *read_base = staging + read_row * kRowBytes + read_column * sizeof(T);
    const int column_in_tile = wave_n * kWaveCols + read_column;
    const bool column_ok = column_in_tile < cols_valid;  // cols_valid is a multiple of 8
    const int first_row = wave_m * kWaveRows + read_row;
#pragma unroll
    for (int i = 0; i < kTilesM; ++i) {
        const int64_t block_offset = static_cast<int64_t>(first_row + i * 32) * stride + column_in_tile;
        Vec16<T> gate[kReads], up[kReads];
        bool valid[kReads];
#pragma unroll
        for (int t = 0; t < kReads; ++t) {
            valid[t] = first_row + i * 32 + t * kRowsPerRead < rows_valid && column_ok;
            if (valid[t]) {
                const T *source = layer_1 + block_offset + static_cast<int64_t>(t) * kRowsPerRead * stride;
                gate[t] = load16_stream(source);
                up[t] = load16_stream(source + half);
            }
        }
#pragma unroll
        for (int j = 0; j < kTilesN; ++j)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                Vec16x4<T> group;
#pragma unroll
                for (int c = 0; c < 4; ++c) group.v[c] = from_float<T>(acc[i][j][4 * g + c]);
                *reinterpret_cast<FM_LDS(u32x2_t) *>(write_base + (j * 32 + 8 * g) * sizeof(T)) =
                    __builtin_bit_cast(u32x2_t, group);
            }
        asm volatile("" ::: "memory");  // one wavefront, in-order LDS: no barrier needed (see store_tile)
        u32x4_t staged[kReads];
#pragma unroll
        for (int t = 0; t < kReads; ++t)
            staged[t] = *reinterpret_cast<FM_LDS(u32x4_t) *>(read_base + t * kRowsPerRead * kRowBytes);
#pragma unroll
        for (int t = 0; t < kReads; ++t) {
            if (!valid[t]) continue;
            const Vec16<T> grad = __builtin_bit_cast(Vec16<T>, staged[t]);
            Vec16<T> grad_gate, grad_up, recomputed;
#pragma unroll
            for (int c = 0; c < kChunk; ++c) {
                float out;
                const float derivative = activation_backward<kActivation>(to_float(gate[t].v[c]), out);
                const float g = to_float(grad.v[c]), other = to_float(up[t].v[c]);
                grad_gate.v[c] = from_float<T>(derivative * other * g);
                grad_up.v[c] = from_float<T>(out * g);
                recomputed.v[c] = from_float<T>(out * other);
            }
            const int64_t row_offset = static_cast<int64_t>(t) * kRowsPerRead;
            T *target = grad_layer_1 + block_offset + row_offset * stride;
            store16_stream(target, grad_gate);
            store16_stream(target + half, grad_up);
            if (activation_out != nullptr)
                store16_stream(activation_out + static_cast<int64_t>(first_row + i * 32 + row_offset) * activation_stride +
                                   column_in_tile,
                               recomputed);
        }
        asm volatile("" ::: "memory");
    }
}

// The tile is 128 gate columns and their 128 up columns of layer 1's output; a wavefront holds gate columns in its
// accumulators j = 0, 1 and the matching up columns in j = 2, 3. Per 32-row block it stages, per row, 64 gate values,
// 64 up values and 64 outputs act(gate) * up, and stores each as 128-byte row segments.
template <typename T, int kActivation>
__device__ __forceinline__ void store_tile_gated_forward(const f32x16_t (&acc)[kTilesM][kTilesN], FM_LDS(char) * lds,
                                                         T *layer_1, T *activation_out, int64_t stride,
                                                         int64_t activation_stride, int64_t half, int rows_valid,
                                                         int wave, int lane) {
    static_assert(kTilesN == 4 && kWaveCols == 128, "two gate and two up accumulators per row block");
    constexpr int kChunk = 16 / sizeof(T);                 // 8
    constexpr int kSegment = kWaveCols / 2;                // 64 columns per segment
    constexpr int kChunksPerRow = 3 * kSegment / kChunk;   // 24
    constexpr int kReads = 32 * kChunksPerRow / 64;        // 12
    constexpr int kRowBytes = 3 * kSegment * sizeof(T) + kEpiloguePadBytes;
    const int wave_m = wave / kWavesN, wave_n = wave % kWavesN;
    FM_LDS(char) *staging = lds + wave * (32 * kRowBytes);
    FM_LDS(char) *write_base = staging + (lane & 31) * kRowBytes + (lane >> 5) * 4 * sizeof(T);
#pragma unroll
    for (int i = 0; i < kTilesM; ++i) {
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                Vec16x4<T> gate, up, result;
#pragma unroll
                for (int c = 0; c < 4; ++c) {
                    gate.v[c] = from_float<T>(acc[i][j][4 * g + c]);
                    up.v[c] = from_float<T>(acc[i][j + 2][4 * g + c]);
                    result.v[c] =
                        from_float<T>(activation_forward<kActivation>(to_float(gate.v[c])) * to_float(up.v[c]));
                }
                FM_LDS(char) *position = write_base + (j * 32 + 8 * g) * sizeof(T);
                *reinterpret_cast<FM_LDS(u32x2_t) *>(position) = __builtin_bit_cast(u32x2_t, gate);
                *reinterpret_cast<FM_LDS(u32x2_t) *>(position + kSegment * sizeof(T)) = __builtin_bit_cast(u32x2_t, up);
                *reinterpret_cast<FM_LDS(u32x2_t) *>(position + 2 * kSegment * sizeof(T)) =
                    __builtin_bit_cast(u32x2_t, result);
            }
        asm volatile("" ::: "memory");
        u32x4_t staged[kReads];
#pragma unroll
        for (int t = 0; t < kReads; ++t) {
            const int id = t * 64 + lane;
            staged[t] = *reinterpret_cast<FM_LDS(u32x4_t) *>(staging + (id / kChunksPerRow) * kRowBytes +
                                                             (id % kChunksPerRow) * 16);
        }
#pragma unroll
        for (int t = 0; t < kReads; ++t) {
            const int id = t * 64 + lane;
            const int row = wave_m * kWaveRows + i * 32 + id / kChunksPerRow, chunk = id % kChunksPerRow;
            const int segment = chunk / (kSegment / kChunk);
            const int column = wave_n * kSegment + (chunk % (kSegment / kChunk)) * kChunk;
            if (row >= rows_valid) continue;
            if (segment == 2) {
                __builtin_nontemporal_store(
                    staged[t], reinterpret_cast<u32x4_t *>(activation_out + row * activation_stride + column));
            } else if (layer_1 != nullptr) {
                __builtin_nontemporal_store(
                    staged[t], reinterpret_cast<u32x4_t *>(layer_1 + row * stride + segment * half + column));
            }
        }
        asm volatile("" ::: "memory");
    }
}

template <typename Work, typename Source>
__device__ __forceinline__ void store_result(const GemmArgs &args, const Work &work, Source &&source,
                                             FM_LDS(char) * lds, int wave, int lane, int row_base, int blocks) {
    const bool accumulate = args.accumulate != 0;
    auto store = [&](auto *out) {
        if (accumulate)
            store_tile<std::remove_pointer_t<decltype(out)>, true>(source, lds, out + work.out_offset,
                                                                   args.out_stride_row, work.rows_valid,
                                                                   work.cols_valid, wave, lane, row_base, blocks);
        else
            store_tile<std::remove_pointer_t<decltype(out)>, false>(source, lds, out + work.out_offset,
                                                                    args.out_stride_row, work.rows_valid,
                                                                    work.cols_valid, wave, lane, row_base, blocks);
    };
    if (args.out_dtype == FM_DTYPE_F32) store(static_cast<float *>(args.out));
    else if (args.out_dtype == FM_DTYPE_BF16) store(static_cast<bf16_t *>(args.out));
    else store(static_cast<f16_t *>(args.out));
}

// A piece's accumulators in the workspace: register by register, 16 bytes per lane, so that every store and load
// covers 1 KiB of consecutive addresses. [wave][accumulator][group of 4 registers][lane][4]
template <typename FloatT>
__device__ __forceinline__ FloatT *partial_of_lane(FloatT *slot, int wave, int lane) {
    return slot + wave * (kPartialFloats / kWaves) + lane * 4;
}

__device__ __forceinline__ void store_partial(const f32x16_t (&acc)[kTilesM][kTilesN], float *slot, int wave, int lane) {
    float *partial = partial_of_lane(slot, wave, lane);
#pragma unroll
    for (int i = 0; i < kTilesM; ++i)
#pragma unroll
        for (int j = 0; j < kTilesN; ++j)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                f32x4_t value;
#pragma unroll
                for (int c = 0; c < 4; ++c) value[c] = acc[i][j][4 * g + c];
                *reinterpret_cast<f32x4_t *>(partial + ((i * kTilesN + j) * 4 + g) * 256) = value;
            }
}

// kMasked: the row-sparse product, whose reduction range [k_lo, k_hi) is ragged.
// kFusion: a GemmFusion, the epilogue to run instead of the plain store.
template <typename T, bool kLhsContiguousK, bool kRhsContiguousK, bool kMasked, int kFusion = kFusionNone>
__global__ __launch_bounds__(kMfmaThreads, kWaves / 4) void grouped_gemm_mfma_kernel(GemmArgs launch_args) {
    static_assert(kFusion == kFusionNone || (kRhsContiguousK && !kMasked), "fused epilogues: output-sparse, K-major rhs");
    extern __shared__ __attribute__((aligned(1024))) char lds_generic[];
    FM_LDS(char) *lds = (FM_LDS(char) *)(lds_generic);  // C-style: address-space cast
    // The arguments are read from the kernel-argument segment where they are needed, through a pointer the compiler
    // cannot see through, and read again after the main loop (`forget_arguments`): otherwise it keeps all of them in
    // scalar registers across the main loop, which then no longer fit.
    typedef const __attribute__((address_space(4))) GemmArgs *ArgumentPointer;
    ArgumentPointer argument_pointer = (ArgumentPointer)__builtin_amdgcn_kernarg_segment_ptr();
    auto forget_arguments = [&]() { asm volatile("" : "+s"(argument_pointer)); };
    forget_arguments();
#define args (*(const GemmArgs *)argument_pointer)

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int wave_m = wave / kWavesN, wave_n = wave % kWavesN;

    // ---- the tiles of this workgroup ---------------------------------------------------------------------
    // Workgroup b computes the tiles of the ids b, b + gridDim.x, b + 2 gridDim.x, ... below args.num_ids. With one
    // workgroup per id that is one tile; with one workgroup per CU (a persistent grid) it is the sequence the hardware
    // would hand that CU if all tiles took the same time, and the first loads of a tile are issued before the
    // previous tile is written out. Ids map to tiles in increasing order, so the first id without a tile ends the walk.
    // Everything about a tile is the same in every lane and is said to be, so that it lives in scalar registers.
    constexpr bool kSlicesFromRangeStart = kMasked && !kLhsContiguousK && !kRhsContiguousK;
    // When the loads of the rhs slices are issued (see the pipeline below). Measured per product on the 12 to 64
    // slice reductions of the fine-grained and wide workloads: -1..-5 % for the two unmasked products; the
    // weight-gradient product gains nothing from either of the other two schedules, and a product that masks slices in
    // LDS works on whole slices that have landed.
    constexpr int kScheduleSplit = 0, kScheduleLate = 1, kScheduleHalves = 2;
    constexpr int kSchedule = kMasked ? kScheduleSplit : (kRhsContiguousK ? kScheduleLate : kScheduleHalves);
    constexpr bool kRhsHalves = kSchedule == kScheduleHalves;
    // Loads that may still be on their way at the barrier before the last K-step and at the one after K-step 0.
    constexpr int kBarrierNewest = kSchedule == kScheduleSplit ? 6 : (kSchedule == kScheduleLate ? 8 : 16);
    constexpr int kMidBarrierNewest = 18;
    typedef TileLoader<kLhsContiguousK> LhsLoader;
    typedef TileLoader<kRhsContiguousK, kRhsHalves> RhsLoader;
    struct Tile {
        TileRecord work;
        int piece_slot;   // >= 0: a piece of a split reduction, stored to that workspace slot
        int k_first;      // first reduction index of slice 0
        int num_slices;
        bool half;        // at most 128 valid rows: the wavefronts share them, 64 each, and issue half the MFMAs
    };
    typedef __attribute__((__vector_size__(16 * sizeof(uint32_t)))) uint32_t u32x16_t;
    // The rest of `tile` from its record.
    auto finish_tile = [&](Tile &tile) {
        const TileRecord &work = tile.work;
        tile.piece_slot = work.piece_slot;
        // Slices start at multiples of kBK, except where both operands are row-contiguous (any K-row can start a
        // slice then): the ragged range of the row-sparse product starts with its first slice and needs no masking.
        tile.k_first = kSlicesFromRangeStart ? work.k_lo : work.k_lo / kBK * kBK;
        const int k_last = work.k_hi > work.k_lo ? tile.k_first + (work.k_hi - tile.k_first + kBK - 1) / kBK * kBK : tile.k_first;
        tile.num_slices = (k_last - tile.k_first) / kBK;
        // A tile with at most 128 valid rows (the last row tile of an expert whose padded row count is an odd multiple
        // of 128) is a half tile. The transfers stay as they are (the rows past the valid ones bring zeros or repeats
        // that nobody reads). Only where the reduction is short: a half tile takes 85 % of a full tile's time, so the
        // workgroups that got one run ahead of the others of their XCD, and with a long reduction (operand panels of
        // 2 MiB and more against 4 MiB of L2: the 32 tiles of a chunk share their panels only while they are within
        // some ten slices of each other) the panels are then fetched again by those that follow. Measured at 64
        // slices and more: L2-miss traffic 5.6 -> 3.0 and 4.6 -> 3.2 (FETCH_SIZE, layer-1 forward and input gradient of
        // the Mixtral-like workload) and the launches 2 to 4 % faster with full-cost last tiles; at 12 to 44 slices
        // the half tiles win by 1.5 to 5 %.
        tile.half = kFusion == kFusionNone && tile.piece_slot < 0 && work.rows_valid <= kTile / 2 &&
                    tile.num_slices < kHalfTileMaxSlices;
    };
    auto find_tile = [&](int id, Tile &tile) -> bool {
        if (args.tile_table != nullptr) {
            // One scalar load (the table was written by an earlier kernel, so the scalar cache cannot hold stale lines).
            const TileRecord *address = static_cast<const TileRecord *>(args.tile_table) + id;
            u32x16_t raw;
            asm volatile("s_load_dwordx16 %0, %1, 0x0\n\ts_waitcnt lgkmcnt(0)" : "=s"(raw) : "s"(address) : "memory");
            tile.work = __builtin_bit_cast(TileRecord, raw);
            if (!tile.work.found) return false;
        } else if (!compute_tile_record(args, id, tile.work)) {
            return false;
        }
        finish_tile(tile);
        return true;
    };
    // The record of the tile AFTER the next one is requested a whole tile ahead, so that nobody waits for it (the
    // scalar load above takes 0.6 us, of tiles that take 17 to 50 us where the reduction is short): a load straight
    // into LDS, issued right after the next tile's first loads, i.e. before the current tile is written out. It lands
    // in the last 256 bytes of the middle lhs slot, which the epilogue's staging area does not reach and which the
    // next tile's loads fill only in their third K-step; lane l fetches word l % 16 of the record, every wavefront
    // fetches it for itself (the same bytes to the same place) and reads it back once its own loads up to that one
    // have landed, before the barrier that starts the tile. The words then wait in one register per lane.
    constexpr int kRecordSpot = kLdsBytes - kOperandBytes - 256;
    static_assert(kStagingBase + kWaves * 32 * (kWaveCols * 4 + kEpiloguePadBytes) <= kRecordSpot, "record spot is staging");
    auto request_record = [&](int id) {
        const TileRecord *address = static_cast<const TileRecord *>(args.tile_table) + id;
        const __amdgpu_buffer_rsrc_t resource = __builtin_amdgcn_make_buffer_rsrc(
            const_cast<char *>(uniform_pointer(reinterpret_cast<const char *>(address))), 0,
            static_cast<int>(sizeof(TileRecord)), kBufferResourceFlags);
        const uint32_t lane_offset = (opaque(static_cast<int>(threadIdx.x)) & 15) * 4;
        const int spot = __builtin_amdgcn_readfirstlane(kRecordSpot);
        asm volatile("s_mov_b32 m0, %0\n\tbuffer_load_dword %1, %2, 0 offen lds"
                     :
                     : "s"(spot), "v"(lane_offset), "s"(resource)
                     : "memory");
    };
    auto read_record = [&]() -> uint32_t {
        const int lane_offset = (opaque(static_cast<int>(threadIdx.x)) & 15) * 4;
        return *reinterpret_cast<FM_LDS(const uint32_t) *>(lds + kRecordSpot + lane_offset);
    };
    auto tile_of_record = [&](uint32_t words, Tile &tile) -> bool {
        u32x16_t raw;
#pragma unroll
        for (int word = 0; word < 16; ++word) raw[word] = __builtin_amdgcn_readlane(words, word);
        tile.work = __builtin_bit_cast(TileRecord, raw);
        if (!tile.work.found) return false;
        finish_tile(tile);
        return true;
    };

    int id = blockIdx.x;
    Tile tile;
    if (id >= args.num_ids || !find_tile(id, tile)) return;

    LhsLoader load_lhs;
    RhsLoader load_rhs;

    f32x16_t acc[kTilesM][kTilesN];
    auto clear_accumulators = [&]() {
#pragma unroll
        for (int i = 0; i < kTilesM; ++i)
#pragma unroll
            for (int j = 0; j < kTilesN; ++j)
#pragma unroll
                for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;
    };

    // ---- the software pipeline --------------------------------------------------------------------------
    // A slot that is being filled cannot be read, and LDS (160 KiB) has room for five operand slices of 32 KiB: three
    // lhs slots and two rhs slots. Iteration t multiplies slice t (rhs slot t % 2, lhs slot t % 3) in four K-steps. The
    // barrier before K-step 3 makes slice t + 1 visible and ends the reads of slice t's slots (the fragments of K-step 3
    // are in registers by then). The loads of a wavefront complete in order, and before a barrier a wavefront waits
    // until all but its N newest loads have landed; N counts the loads issued since the newest one that the reads
    // after the barrier need. Except under "late", every K-step issues two lhs loads: chunks 2..7 of slice t + 2 in
    // K-steps 0..2, chunks 0, 1 of slice t + 3 in K-step 3 (into the slot slice t just left). The rhs loads follow one
    // of three schedules:
    //   split  : chunks 4..7 of slice t + 1 in K-step 0, chunks 0..3 of slice t + 2 in K-step 3; N = 6. An rhs load
    //            has half a slice of MFMAs or more to land.
    //   late   : all 8 chunks of slice t + 2 in K-step 3, right after the barrier that frees their slot, and the lhs
    //            loads of slice t + 2 in K-steps 0..2 (three, three, two); N = 8, three quarters of a slice for an rhs load.
    //   halves : a row-contiguous rhs slot is refilled in halves (K-rows 0..31, 32..63). A second barrier, after K-step
    //            0, makes the second half of slice t visible and ends the reads of its first half (N = 18); every
    //            K-step then issues two rhs loads: chunks 6, 7 of slice t + 1 in K-step 0, chunks 0..5 of slice t + 2
    //            in K-steps 1..3 (0..3 are its first half), and N = 16 at the barrier before K-step 3. Every load has a
    //            full slice of MFMAs to land, and the loads are spread evenly over the K-steps.
    // A K-contiguous rhs slice does not split along K (a row's 128 bytes are one cache line). Which schedule an instance
    // uses was measured (`kSchedule`).
    // Fragments are double-buffered over K-steps, across slices as well. There is no branch around a transfer: loads
    // past the last slice bring zeros.
    u32x4_t frag_a[2][kTilesM], frag_b[2][kTilesN];
    constexpr int kSteps = kBK / 16;
    constexpr int kLhsBase = kStages * kOperandBytes;  // LDS byte address of lhs slot 0; the rhs slots start at 0
    // LDS byte addresses of the lhs slots of slices t, t + 1, t + 2 (wave-uniform, rotated after every slice) and the
    // fragment addresses of this lane in the first two.
    // A tile starts with slice 0 in the LAST lhs slot and in rhs slot 0, so that the LDS in between, kStagingBase up to
    // that lhs slot, is free for the previous tile's epilogue while those first loads are on their way.
    int lhs_now, lhs_next, lhs_after;
    int lhs_frag0[4], lhs_frag[4], lhs_frag_next[4], rhs_frag[4];
    auto read_rhs_fragment = [&](int slot, int kstep, int buffer, int j) {
        frag_b[buffer][j] = load_fragment<kRhsContiguousK>(lds, rhs_frag, slot, j, kstep);
    };
    auto read_lhs_fragment = [&](bool next_slice, int kstep, int buffer, int i) {
        frag_a[buffer][i] = next_slice ? load_fragment<kLhsContiguousK>(lds, lhs_frag_next, 0, i, kstep)
                                       : load_fragment<kLhsContiguousK>(lds, lhs_frag, 0, i, kstep);
    };
    auto mask_slice = [&](int slice, int lhs_address, int rhs_slot) {
        if constexpr (kMasked && !kSlicesFromRangeStart) {
            const int k_lo = tile.work.k_lo, k_hi = tile.work.k_hi;
            const int k0 = tile.k_first + slice * kBK;
            if (slice < tile.num_slices && (k0 < k_lo || k0 + kBK > k_hi)) {  // wave-uniform
                mask_tile<kLhsContiguousK>(lds + lhs_address, k0, k_lo, k_hi);
                mask_tile<kRhsContiguousK>(lds + rhs_slot * kOperandBytes, k0, k_lo, k_hi);
                __syncthreads();
            }
        }
    };
    // A K-step is 16 slots of "one MFMA, then at most one memory instruction in its shadow" (an MFMA keeps the matrix
    // pipe busy for 32 cycles; a clump of LDS/global instructions longer than that leaves it idle), in an order pinned
    // with a scheduling barrier after every slot:
    //   slots 0..3     rhs fragments 0..3 of the next K-step (other fragment buffer)
    //   slots 4..7     lhs fragments 0..3 of the next K-step
    //   slots 8..11    rhs loads (schedule "late": slots 8..15 of K-step 3)
    //   slots 12..14   lhs loads
    // A half tile has 8 slots per K-step (2 x 4 accumulators): rhs fragments in slots 0..3, the two lhs fragments in
    // slots 4, 5, the rhs loads in slots 2..5 as well ("late": two per slot) and the lhs loads from slot 5 on.
    static_assert(kTilesM == 4 && kTilesN == 4 && kLoadsPerOperand == 8, "the slot table below is written for this shape");
    auto iteration = [&](int t, auto slot_constant, auto half_constant) {
        constexpr int kSlot = decltype(slot_constant)::value, kNextSlot = 1 - kSlot;  // rhs, of slices t, t + 1
        constexpr bool kHalf = decltype(half_constant)::value;
        constexpr int kRowBlocks = kHalf ? kTilesM / 2 : kTilesM;
        constexpr int kSlots = kRowBlocks * kTilesN;
        constexpr int kRhsLoadSlot = kHalf ? 2 : 8;  // first slot of a K-step that issues rhs loads
        constexpr int kLhsLoadSlot = kHalf ? 5 : 12;  // first slot of a K-step that issues lhs loads
#pragma unroll
        for (int kstep = 0; kstep < kSteps; ++kstep) {
            const bool last = kstep + 1 == kSteps;
            const int next_slot = last ? kNextSlot : kSlot, next_kstep = (kstep + 1) % kSteps;
            const int buffer = kstep & 1;
            // What this K-step loads (see the table above): `lhs_count` lhs chunks from `lhs_chunk` on, `rhs_count` rhs
            // chunks from `rhs_chunk` on into rhs slot `rhs_slot`.
            int lhs_chunk = 0, lhs_count = 0, lhs_target = lhs_after, rhs_chunk = 0, rhs_count = 0, rhs_slot = kSlot;
            if constexpr (kSchedule == kScheduleSplit) {
                lhs_chunk = 2 * next_kstep, lhs_count = 2;
                if (last) {
                    load_lhs.advance();
                    load_rhs.advance();
                    lhs_target = lhs_now;
                    rhs_count = 4;
                } else if (kstep == 0) {
                    rhs_chunk = 4, rhs_count = 4, rhs_slot = kNextSlot;
                }
            } else if constexpr (kSchedule == kScheduleLate) {
                lhs_chunk = 3 * kstep, lhs_count = kstep < 2 ? 3 : (last ? 0 : 2);
                if (kstep == 0) load_lhs.advance();
                if (last) {
                    load_rhs.advance();
                    rhs_count = 8;
                }
            } else {
                lhs_chunk = 2 * next_kstep, lhs_count = 2;
                rhs_chunk = kstep == 0 ? 6 : 2 * (kstep - 1), rhs_count = 2;  // 6, 7 of slice t + 1, then 0..5 of slice t + 2
                if (kstep == 0) rhs_slot = kNextSlot;
                if (kstep == 1) load_rhs.advance();
                if (last) {
                    load_lhs.advance();
                    lhs_target = lhs_now;
                }
            }
#pragma unroll
            for (int m = 0; m < kSlots; ++m) {
                // Boustrophedon order: consecutive MFMAs always share one operand (fewer operand-bus toggles).
                const int i = m / kTilesN, j = (i & 1) ? kTilesN - 1 - m % kTilesN : m % kTilesN;
                acc[i][j] = Mfma<T>::run(frag_b[buffer][j], frag_a[buffer][i], acc[i][j]);  // transposed, see store_tile
                if (m < kTilesN) read_rhs_fragment(next_slot, next_kstep, buffer ^ 1, m);
                else if (m < kTilesN + kRowBlocks) read_lhs_fragment(last, next_kstep, buffer ^ 1, m - kTilesN);
                // All rhs loads of a K-step before its lhs loads: the waits before the barriers count on it.
                if (kHalf && rhs_count == 8) {  // two per slot
                    if (m >= kRhsLoadSlot && m < kRhsLoadSlot + 4) {
                        load_rhs.load(rhs_slot * kOperandBytes, 2 * (m - kRhsLoadSlot));
                        load_rhs.load(rhs_slot * kOperandBytes, 2 * (m - kRhsLoadSlot) + 1);
                    }
                } else if (m >= kRhsLoadSlot && m < kRhsLoadSlot + rhs_count) {
                    load_rhs.load(rhs_slot * kOperandBytes, rhs_chunk + m - kRhsLoadSlot);
                }
                if (m >= kLhsLoadSlot && m < kLhsLoadSlot + lhs_count)
                    load_lhs.load(lhs_target, lhs_chunk + m - kLhsLoadSlot);
                __builtin_amdgcn_sched_barrier(0);
            }
            if (kRhsHalves && kstep == 0) {
                wait_for_loads<kMidBarrierNewest>();
                __syncthreads();
            }
            if (kstep == kSteps - 2) {
                wait_for_loads<kBarrierNewest>();
                __syncthreads();
                mask_slice(t + 1, lhs_next, kNextSlot);
            }
        }
        // On to the next slice: rotate the lhs slots.
        const int recycled = lhs_now;
        lhs_now = lhs_next;
        lhs_next = lhs_after;
        lhs_after = recycled;
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            lhs_frag[q] = lhs_frag_next[q];
            lhs_frag_next[q] = lhs_frag0[q] + lhs_next;
        }
    };
    // The loads that start a tile come in two parts: slice 0 of both operands (16 loads per wavefront), which are issued
    // while the previous tile is still being written out, and those that follow (`continue_tile`: slice 1 of both
    // operands and, with rhs halves, lhs chunks 0, 1 of slice 2), in the order the main loop would have issued them.
    // Nothing that `first_loads` computes per lane outlives it: the loaders and fragment addresses of the tile are set
    // up (again) by `setup_tile`, after the previous tile's epilogue, so that they do not occupy registers during it.
    auto setup_loaders = [&](const Tile &next, LhsLoader &lhs_loader, RhsLoader &rhs_loader, int lane) {
        const TileRecord &work = next.work;
        const char *lhs = static_cast<const char *>(args.lhs) +
                          (work.lhs_offset + next.k_first * args.lhs_stride_inner) * static_cast<int64_t>(sizeof(T));
        const char *rhs = static_cast<const char *>(args.rhs) +
                          (work.rhs_offset + next.k_first * args.rhs_stride_inner) * static_cast<int64_t>(sizeof(T));
        lhs_loader.setup(uniform_pointer(lhs),
                         (kLhsContiguousK ? args.lhs_stride_row : args.lhs_stride_inner) * sizeof(T), work.rows_valid,
                         next.num_slices, work.k_hi - next.k_first, wave, lane);
        rhs_loader.setup(uniform_pointer(rhs),
                         (kRhsContiguousK ? args.rhs_stride_col : args.rhs_stride_inner) * sizeof(T), work.cols_valid,
                         next.num_slices, work.k_hi - next.k_first, wave, lane,
                         kFusion == kFusionGatedForward ? static_cast<int>(args.half) : 0);
    };
    constexpr int kFirstLhsSlot = kLhsBase + (kLhsStages - 1) * kOperandBytes;
    auto first_loads = [&](const Tile &next) {
        if (next.num_slices <= 0) return;
        LhsLoader lhs_loader;
        RhsLoader rhs_loader;
        setup_loaders(next, lhs_loader, rhs_loader, opaque(lane));
#pragma unroll
        for (int j = 0; j < kLoadsPerOperand; ++j) lhs_loader.load(kFirstLhsSlot, j);
#pragma unroll
        for (int j = 0; j < kLoadsPerOperand; ++j) rhs_loader.load(0, j);
    };
    auto setup_tile = [&](const Tile &next) {
        const int lane = opaque(static_cast<int>(threadIdx.x & 63));
        setup_loaders(next, load_lhs, load_rhs, lane);
        lhs_now = kFirstLhsSlot;
        lhs_next = kLhsBase;
        lhs_after = kLhsBase + kOperandBytes;
        const int wave_row_base = wave_m * (next.half ? kWaveRows / 2 : kWaveRows);
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            lhs_frag0[q] = fragment_base<kLhsContiguousK>(wave_row_base, q, lane);
            lhs_frag[q] = lhs_frag0[q] + lhs_now;
            lhs_frag_next[q] = lhs_frag0[q] + lhs_next;
            rhs_frag[q] = fragment_base<kRhsContiguousK>(wave_n * kWaveCols, q, lane);
        }
    };
    // rhs chunks of slice 1 and lhs chunks of slice 2 that the prologue issues (the main loop issues the rest).
    constexpr int kPrologueRhs = kSchedule == kScheduleSplit ? 4 : (kSchedule == kScheduleHalves ? 6 : 8);
    constexpr int kPrologueLhs = kSchedule == kScheduleLate ? 0 : 2;
    auto continue_tile = [&]() {
        load_lhs.advance();
        load_rhs.advance();
#pragma unroll
        for (int j = 0; j < kLoadsPerOperand; ++j) load_lhs.load(lhs_next, j);
#pragma unroll
        for (int j = 0; j < kPrologueRhs; ++j) load_rhs.load(kOperandBytes, j);
        if constexpr (kPrologueLhs > 0) {
            load_lhs.advance();
#pragma unroll
            for (int j = 0; j < kPrologueLhs; ++j) load_lhs.load(lhs_after, j);
        }
    };
    constexpr int kLoadsAfterSlice0 = kLoadsPerOperand + kPrologueRhs + kPrologueLhs;

    first_loads(tile);
    // Whether the record of the id after `id` has been requested (with a tile table, for every id that exists).
    bool requested = false;
    auto request_next_record = [&]() {
        requested = args.tile_table != nullptr && id + static_cast<int>(gridDim.x) < args.num_ids;
        if (requested) request_record(id + gridDim.x);
    };
    request_next_record();
    while (true) {
        setup_tile(tile);
        const int num_slices = tile.num_slices;
        uint32_t next_record = 0;
        if (num_slices > 0) {
            // Prologue: slice 0, lhs slice 1 and the first pieces of the slices after them on their way; slice 0 landed.
            continue_tile();
            clear_accumulators();  // 256 register writes, while the first loads are on their way
            wait_for_loads<kLoadsAfterSlice0>();  // slice 0 was loaded first, the next record right after it
            if (requested) next_record = read_record();
            __syncthreads();
            mask_slice(0, lhs_now, 0);
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                read_rhs_fragment(0, 0, 0, q);
                read_lhs_fragment(false, 0, 0, q);
            }
            constexpr std::integral_constant<int, 0> slot0{};
            constexpr std::integral_constant<int, 1> slot1{};
            // Two slices per trip (the rhs slots alternate); an odd count multiplies one slice of zeros. (Leaving the
            // loop before that slice costs far more than it saves: with a second exit the compiler no longer keeps the
            // accumulators in place and the kernel ran five times slower.)
            if (tile.half) {
                for (int t = 0; t < num_slices; t += 2) {
                    iteration(t, slot0, std::true_type{});
                    iteration(t + 1, slot1, std::true_type{});
                }
            } else {
                for (int t = 0; t < num_slices; t += 2) {
                    iteration(t, slot0, std::false_type{});
                    iteration(t + 1, slot1, std::false_type{});
                }
            }
            wait_for_loads<0>();  // the zero-filling loads of slices past the end still write LDS
        } else {
            clear_accumulators();
            if (requested) {
                wait_for_loads<0>();
                next_record = read_record();
            }
        }
        __syncthreads();  // all wavefronts are done reading operand slices; LDS becomes the staging area
        forget_arguments();

        // What the epilogue needs of this tile, before the next one takes its place.
        const TileRecord work = tile.work;
        const int piece_slot = tile.piece_slot;
        const int wave_row_base = wave_m * (tile.half ? kWaveRows / 2 : kWaveRows);
        const int wave_row_blocks = tile.half ? kTilesM / 2 : kTilesM;
        // The next tile is looked up here, not earlier, to keep its coordinates out of the registers of the main loop;
        // its first loads go out before this tile's results do.
        id += gridDim.x;
        const bool have_next = requested ? tile_of_record(next_record, tile) : id < args.num_ids && find_tile(id, tile);
        if (have_next) {
            first_loads(tile);
            request_next_record();
        }

        FM_LDS(char) *staging = lds + kStagingBase;
        const int lane = opaque(static_cast<int>(threadIdx.x & 63));  // per-lane addresses of the epilogue: not hoisted
        if (piece_slot < 0 && args.accumulate != 0 && num_slices == 0) {
            // nothing to add
        } else if constexpr (kFusion == kFusionGatedForward) {
            T *layer_1 = args.out == nullptr ? nullptr : static_cast<T *>(args.out) + work.out_offset;
            FM_DISPATCH_ACTIVATION(args.activation, kActivation,
                                   store_tile_gated_forward<T, kActivation>(
                                       acc, staging, layer_1, static_cast<T *>(args.fused_out) + work.fused_offset,
                                       args.out_stride_row, args.fused_stride, args.half, work.rows_valid, wave, lane));
        } else if constexpr (kFusion == kFusionGatedBackward) {
            T *recomputed = args.fused_out == nullptr ? nullptr : static_cast<T *>(args.fused_out) + work.fused_offset;
            FM_DISPATCH_ACTIVATION(args.activation, kActivation,
                                   store_tile_gated_backward<T, kActivation>(
                                       acc, staging, static_cast<T *>(args.out) + work.out_offset,
                                       static_cast<const T *>(args.fused_in) + work.out_offset, recomputed,
                                       args.out_stride_row, args.fused_stride, args.half, work.rows_valid,
                                       work.cols_valid, wave, lane));
        } else {
            if (piece_slot >= 0)
                store_partial(acc, args.partials + static_cast<int64_t>(piece_slot) * kPartialFloats, wave, lane);
            else
                store_result(
                    args, work, [&](int i) -> const f32x16_t(&)[kTilesN] { return acc[i]; }, staging, wave, lane,
                    wave_row_base, wave_row_blocks);
        }
        if (!have_next) break;
        __syncthreads();  // the staging areas have been read: the next tile's loads may overwrite them
    }
#undef args
}

// Adds the pieces of each tile whose reduction the main kernel split, in piece order, and stores the sums.
// One single-wavefront workgroup per quarter of a tile (what one wavefront of the main kernel computed), so that the
// few tiles of a last round still spread over all CUs.
constexpr int kReduceLdsBytes = kWaves * 32 * (kWaveCols * 4 + kEpiloguePadBytes);  // the staging areas of store_tile
__global__ __launch_bounds__(64) void grouped_gemm_reduce_kernel(GemmArgs args) {
    extern __shared__ __attribute__((aligned(1024))) char lds_generic[];
    FM_LDS(char) *lds = (FM_LDS(char) *)(lds_generic);
    // The plan kernel has left the split plan of this launch in front of the tile records.
    const SplitPlan plan = static_cast<const TableHeader *>(args.tile_table)[-1].plan;
    const int index = blockIdx.x / kWaves;
    if (plan.pieces == 1 || index >= plan.tail) return;
    TileWork work;
    if (!resolve_tile(args, plan.whole + index, work)) return;
    const int lane = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(static_cast<int>(blockIdx.x % kWaves));
    // One block of 32 rows at a time: 64 registers of sums, the loads of a piece all in flight together.
    struct RowBlock {
        f32x16_t values[kTilesN];
        __device__ const f32x16_t &operator[](int j) const { return values[j]; }
    };
    auto summed_block = [&](int i) {
        RowBlock block;
#pragma unroll
        for (int j = 0; j < kTilesN; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) block.values[j][v] = 0.f;
        for (int piece = 0; piece < plan.pieces; ++piece) {
            const float *partial =
                partial_of_lane(args.partials + static_cast<int64_t>(piece * plan.tail + index) * kPartialFloats, wave,
                                lane) +
                i * kTilesN * 4 * 256;
#pragma unroll
            for (int j = 0; j < kTilesN; ++j)
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    const f32x4_t value = *reinterpret_cast<const f32x4_t *>(partial + (j * 4 + g) * 256);
#pragma unroll
                    for (int c = 0; c < 4; ++c) block.values[j][4 * g + c] += value[c];
                }
        }
        return block;
    };
    store_result(args, work, summed_block, lds, wave, lane, (wave / kWavesN) * kWaveRows, kTilesM);
}

// ---- host side -----------------------------------------------------------------------------------------
// Kernels that use more dynamic LDS than the default limit need the attribute set once per device; `configured` is the
// kernel's own bit mask of devices done (setting it twice from racing threads is harmless).
static int allow_lds(const void *kernel, int bytes, std::atomic<uint64_t> &configured) {
    int device = 0;
    if (hipGetDevice(&device) != hipSuccess) return fail(FM_ERR_LAUNCH, "hipGetDevice failed");
    const uint64_t bit = uint64_t(1) << (device & 63);
    if (device < 64 && (configured.load(std::memory_order_relaxed) & bit)) return FM_OK;
    hipError_t error = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
    if (error != hipSuccess) return fail(FM_ERR_LAUNCH, "hipFuncSetAttribute: %s", hipGetErrorString(error));
    if (device < 64) configured.fetch_or(bit, std::memory_order_relaxed);
    return FM_OK;
}

template <typename T, bool kLhsK, bool kRhsK, bool kMasked, int kFusion = kFusionNone>
static int launch_instance(const GemmArgs &args, hipStream_t stream) {
    auto kernel = grouped_gemm_mfma_kernel<T, kLhsK, kRhsK, kMasked, kFusion>;
    static std::atomic<uint64_t> configured{0};
    if (int status = allow_lds(reinterpret_cast<const void *>(kernel), kLdsBytes, configured)) return status;
    // With a workspace, one wavefront per id first writes the id's tile record (and, when the last round may be
    // split, the plan of the split).
    if (args.tile_table != nullptr)
        grouped_gemm_plan_kernel<<<(args.num_ids + 3) / 4, 256, 0, stream>>>(args, static_cast<TileRecord *>(args.tile_table));
    // One workgroup per CU walks the ids (see the kernel).
    kernel<<<min(args.num_ids, kRound), kMfmaThreads, kLdsBytes, stream>>>(args);
    if (args.partials != nullptr) {
        static std::atomic<uint64_t> reduce_configured{0};
        if (int status = allow_lds(reinterpret_cast<const void *>(grouped_gemm_reduce_kernel), kReduceLdsBytes,
                                   reduce_configured))
            return status;
        grouped_gemm_reduce_kernel<<<kRound * kWaves, 64, kReduceLdsBytes, stream>>>(args);
    }
    return FM_OK;
}

template <typename T>
static int launch_layout(const GemmArgs &args, hipStream_t stream) {
    const bool lhs_k = args.lhs_stride_inner == 1, rhs_k = args.rhs_stride_inner == 1;
    if (args.fusion == kFusionGatedForward) return launch_instance<T, true, true, false, kFusionGatedForward>(args, stream);
    if (args.fusion == kFusionGatedBackward) return launch_instance<T, true, true, false, kFusionGatedBackward>(args, stream);
    // Only the row-sparse product with a map has a ragged reduction range.
    const bool masked = args.mode == kInputRowSparse && args.expert_ends != nullptr;
#define FM_LAUNCH(LHS, RHS) \
    return masked ? launch_instance<T, LHS, RHS, true>(args, stream) : launch_instance<T, LHS, RHS, false>(args, stream)
    if (lhs_k && rhs_k) FM_LAUNCH(true, true);
    if (lhs_k) FM_LAUNCH(true, false);
    if (rhs_k) FM_LAUNCH(false, true);
    FM_LAUNCH(false, false);
#undef FM_LAUNCH
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
    // Per-lane byte offsets inside an operand tile are 32-bit.
    if (max(max(args.lhs_stride_row, args.lhs_stride_inner), max(args.rhs_stride_inner, args.rhs_stride_col)) >=
        (int64_t(1) << 21))
        return false;
    // The tile is stored as vectors of 4 elements.
    if (!aligned16(args.out) || args.out_stride_row % 8 != 0) return false;
    return true;
}

// The fused epilogues exist for one layout: both operands K-contiguous, output-sparse mode, T in and out, whole
// column tiles (the activation width a multiple of 128 for the forward, of 8 for the backward).
bool mfma_gemm_fusion_eligible(const GemmArgs &args, int dtype) {
    if (!mfma_gemm_eligible(args, dtype) || args.mode != kOutputSparse || args.out_dtype != dtype || args.accumulate)
        return false;
    if (args.lhs_stride_inner != 1 || args.rhs_stride_inner != 1) return false;
    if (!aligned16(args.fused_out) || !aligned16(args.fused_in) || args.fused_stride % 8 != 0 || args.half % 8 != 0)
        return false;
    if (args.fusion == kFusionGatedForward) {
        // The up rows of a tile are addressed with 32-bit byte offsets from its gate rows.
        if (args.half % (kTile / 2) != 0 || (args.half + kTile) * args.rhs_stride_col * 2 >= (int64_t(1) << 32)) return false;
    }
    return true;
}

// ---- workspace: the tile table and the pieces of split reductions ----------------------------------------
// Whether a product is one whose last round is split is decided from its dimensions alone (few rounds of long tiles);
// the caller then brings kMaxPartials tile-sized fp32 slots, followed by one tile record per workgroup id. Given the
// dimensions, whether the split happens depends on nothing but the presence of the workspace, which is the caller's
// choice; the table changes no result, only where a workgroup finds its tile.
static void count_tiles(GemmArgs &args) {
    if (args.mode == kInputRowSparse) {
        args.tiles_m = static_cast<int>((args.sparse_size + kTile - 1) / kTile) * args.num_experts;
    } else {
        // Upper bound of sum_e ceil(rows_e / 256); the surplus ids have no tile.
        args.tiles_m = static_cast<int>((args.rows + kTile - 1) / kTile + (args.num_experts > 1 ? args.num_experts : 0));
    }
    args.tiles_n = static_cast<int>((args.cols + kTile - 1) / kTile);
    if (args.fusion == kFusionGatedForward) args.tiles_n = static_cast<int>(args.half / (kTile / 2));
}

static bool too_many_tiles(const GemmArgs &args) {
    return static_cast<int64_t>(args.tiles_m) * args.tiles_n >= (int64_t(1) << 31) - 2 * kRound - kMaxPartials;
}

static bool splits_last_round(const GemmArgs &args) {
    constexpr int kMaxRoundsToSplit = 16;
    return args.fusion == kFusionNone && args.mode != kInputRowSparse && args.inner / kBK >= 2 * kMinPieceSlices &&
           static_cast<int64_t>(args.tiles_m) * args.tiles_n <= kMaxRoundsToSplit * kRound;
}

// Whole rounds of one chunk per XCD; when the last round is split its pieces come after the whole tiles, at most
// kMaxPartials of them.
static int count_ids(const GemmArgs &args, bool split) {
    return (args.tiles_m * args.tiles_n + kRound - 1) / kRound * kRound + (split ? kMaxPartials : 0);
}

constexpr size_t kPartialBytes = sizeof(float) * kPartialFloats * kMaxPartials;
// The header, then one record per id.
static size_t table_bytes(int num_ids) {
    return (sizeof(TableHeader) + static_cast<size_t>(num_ids) * sizeof(TileRecord) + 255) / 256 * 256;
}

size_t mfma_gemm_workspace_size(GemmArgs args) {
    if (args.rows <= 0 || args.cols <= 0 || args.inner <= 0) return 0;
    // Dimensions that `mfma_gemm_eligible` refuses whatever the strides: such a product runs on the generic kernel,
    // which takes no workspace.
    if (args.inner % kBK != 0 || args.cols % 8 != 0 || (args.mode == kInputRowSparse && args.sparse_size % 8 != 0)) return 0;
    count_tiles(args);
    if (too_many_tiles(args)) return 0;
    const bool split = splits_last_round(args);
    return (split ? kPartialBytes : 0) + table_bytes(count_ids(args, split));
}

int mfma_gemm_launch(GemmArgs args, int dtype, void *workspace, size_t workspace_size, hipStream_t stream) {
    count_tiles(args);
    if (too_many_tiles(args)) return fail(FM_ERR_UNSUPPORTED, "grouped gemm: too many tiles");
    args.partials = nullptr;
    args.tile_table = nullptr;
    const bool split = workspace != nullptr && splits_last_round(args);
    args.num_ids = count_ids(args, split);
    if (workspace != nullptr) {
        const size_t needed = (split ? kPartialBytes : 0) + table_bytes(args.num_ids);
        if (workspace_size < needed || reinterpret_cast<uintptr_t>(workspace) % 64 != 0)
            return fail(FM_ERR_INVALID_ARGUMENT,
                        "grouped gemm: workspace of %zu bytes (64-byte aligned) needed, got %zu at %p", needed,
                        workspace_size, workspace);
        if (split) args.partials = static_cast<float *>(workspace);
        args.tile_table = static_cast<char *>(workspace) + (split ? kPartialBytes : 0) + sizeof(TableHeader);
        // A launch of at most one round that does not split: every workgroup finds its one tile itself (a scan of the
        // expert map, a few thousand cycles) sooner than a kernel launched in front of it could tell it.
        if (!split && args.num_ids <= kRound) args.tile_table = nullptr;
    }
    return dtype == FM_DTYPE_BF16 ? launch_layout<bf16_t>(args, stream) : launch_layout<f16_t>(args, stream);
}

}  // namespace fm
