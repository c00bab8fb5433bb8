// Routing: build the sparse map (expert histogram -> padded expert offsets -> stable row of every
// (token, slot) pair) with integer arithmetic only, so the result is bit-exact and run-to-run identical.
//
// Three small launches over the flattened `top_experts` (M = tokens * experts_per_token entries):
//   1. sparse_map_histogram_kernel: one workgroup per 1024 entries. Each wavefront finds, with
//      ceil(log2 E) ballots, the set of lanes that hold the same expert ("match-any"); the lowest lane of each
//      set adds the set size to an LDS histogram. The workgroup writes its E counts to the workspace.
//   2. sparse_map_layout_kernel: one workgroup. Thread e turns column e of the per-workgroup counts into an
//      exclusive prefix (in place) and gets count[e]; an LDS scan of the padded counts gives expert_ends,
//      expert_pad_begins and the first row of every expert.
//   3. sparse_map_rows_kernel: same partition as (1). rank inside the wavefront = popcount of the match set
//      below the lane; rank inside the workgroup adds an LDS prefix over the 16 wavefronts; the global stable
//      rank adds the exclusive prefix from (2). row = begin[e] + rank.
// Ranks follow the flattened index order, i.e. the order of a stable sort by expert
// (reference: fast_llm/functional/triton/sparse_copy.py:249-254).
#include "fm_common.h"
#include "fm_router_layout.h"

#include <mutex>

namespace fm {

constexpr int kMapBlock = 1024;  // entries (= threads) per workgroup
constexpr int kMapWaves = kMapBlock / 64;
constexpr int kMapMaxExperts = 1024;

__device__ __forceinline__ int log2_ceil(int value) {
    int bits = 0;
    while ((1 << bits) < value) ++bits;
    return bits;
}

// Lanes of this wavefront whose (valid) expert equals this lane's. Undefined for invalid lanes.
__device__ __forceinline__ uint64_t match_expert(int expert, bool valid, int num_bits) {
    uint64_t same = __ballot(valid);
    for (int bit = 0; bit < num_bits; ++bit) {
        const bool set = (expert >> bit) & 1;
        const uint64_t with_bit = __ballot(valid && set);
        same &= set ? with_bit : ~with_bit;
    }
    return same;
}

__global__ __launch_bounds__(kMapBlock) void sparse_map_histogram_kernel(const int64_t *__restrict__ top_experts,
                                                                         int64_t num_entries, int num_experts,
                                                                         int32_t *__restrict__ block_counts) {
    extern __shared__ int32_t lds_counts[];  // [num_experts]
    for (int e = threadIdx.x; e < num_experts; e += kMapBlock) lds_counts[e] = 0;
    __syncthreads();

    const int64_t entry = static_cast<int64_t>(blockIdx.x) * kMapBlock + threadIdx.x;
    int64_t expert64 = entry < num_entries ? top_experts[entry] : -1;
    const bool valid = expert64 >= 0 && expert64 < num_experts;
    const int expert = valid ? static_cast<int>(expert64) : 0;
    const uint64_t same = match_expert(expert, valid, log2_ceil(num_experts));
    const int lane = threadIdx.x & 63;
    if (valid && (same & ((1ull << lane) - 1)) == 0) atomicAdd(&lds_counts[expert], __popcll(same));
    __syncthreads();

    int32_t *out = block_counts + static_cast<int64_t>(blockIdx.x) * num_experts;
    for (int e = threadIdx.x; e < num_experts; e += kMapBlock) out[e] = lds_counts[e];
}

// Second half of the layout kernels: thread e holds count[e]; writes expert_ends, expert_pad_begins and the first row
// of every expert (inclusive scan of the padded counts over experts: wavefront scan, then the wavefront totals).
__device__ __forceinline__ void write_expert_layout(int64_t count, int num_experts, int64_t pad_to_multiple,
                                                    int index_dtype, void *__restrict__ expert_ends,
                                                    void *__restrict__ expert_pad_begins,
                                                    int32_t *__restrict__ expert_begins) {
    __shared__ int64_t lds_wave_totals[kMapWaves];
    const int e = threadIdx.x;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int64_t padded = (count + pad_to_multiple - 1) / pad_to_multiple * pad_to_multiple;
    int64_t inclusive = padded;
#pragma unroll
    for (int offset = 1; offset < 64; offset <<= 1) {
        const int64_t other = __shfl_up(inclusive, offset, 64);
        if (lane >= offset) inclusive += other;
    }
    if (lane == 63) lds_wave_totals[wave] = inclusive;
    __syncthreads();
    int64_t base = 0;
    for (int w = 0; w < wave; ++w) base += lds_wave_totals[w];
    inclusive += base;

    if (e < num_experts) {
        const int64_t begin = inclusive - padded;
        store_index(expert_ends, index_dtype, e, inclusive);
        store_index(expert_pad_begins, index_dtype, e, begin + count);
        expert_begins[e] = static_cast<int32_t>(begin);
    }
}

__global__ __launch_bounds__(kMapBlock) void sparse_map_layout_kernel(int32_t *__restrict__ block_counts,
                                                                      int num_blocks, int num_experts,
                                                                      int64_t pad_to_multiple, int index_dtype,
                                                                      void *__restrict__ expert_ends,
                                                                      void *__restrict__ expert_pad_begins,
                                                                      int32_t *__restrict__ expert_begins) {
    const int e = threadIdx.x;
    // Exclusive prefix over workgroups of this expert's counts, in place.
    int64_t count = 0;
    if (e < num_experts) {
        // 16 counts are requested before the first is used: one memory latency per 16 workgroups, not per workgroup
        // (a load after a store to the same array is not moved ahead of it by the compiler).
        constexpr int kBatch = 16;
        int32_t running = 0;
        for (int b0 = 0; b0 < num_blocks; b0 += kBatch) {
            int32_t *slot = block_counts + static_cast<int64_t>(b0) * num_experts + e;
            int32_t here[kBatch];
#pragma unroll
            for (int i = 0; i < kBatch; ++i)
                here[i] = b0 + i < num_blocks ? slot[static_cast<int64_t>(i) * num_experts] : 0;
#pragma unroll
            for (int i = 0; i < kBatch; ++i) {
                if (b0 + i < num_blocks) slot[static_cast<int64_t>(i) * num_experts] = running;
                running += here[i];
            }
        }
        count = running;
    }
    write_expert_layout(count, num_experts, pad_to_multiple, index_dtype, expert_ends, expert_pad_begins, expert_begins);
}

// The same from what the router's forward kernel left in its workspace: per workgroup of that kernel (a fixed range
// of `tokens_per_block` tokens) and routed expert, the number of tokens of the range that selected the expert, as a
// float (exact: at most 2^24). Shared experts follow the routed ones and are selected by every token.
__global__ __launch_bounds__(kMapBlock) void sparse_map_layout_from_router_kernel(
    const float *__restrict__ router_partials, int router_stats, int num_blocks, int64_t num_tokens,
    int64_t tokens_per_block, int routed_experts, int num_experts, int64_t pad_to_multiple, int index_dtype,
    void *__restrict__ expert_ends, void *__restrict__ expert_pad_begins, int32_t *__restrict__ block_prefix,
    int32_t *__restrict__ expert_begins) {
    const int e = threadIdx.x;
    int64_t count = 0;
    if (e < num_experts) {
        constexpr int kBatch = 16;  // counts requested together, as in sparse_map_layout_kernel
        int32_t running = 0;
        for (int b0 = 0; b0 < num_blocks; b0 += kBatch) {
            int32_t here[kBatch];
#pragma unroll
            for (int i = 0; i < kBatch; ++i) {
                const int b = b0 + i;
                if (b >= num_blocks) {
                    here[i] = 0;
                } else if (e < routed_experts) {
                    here[i] = static_cast<int32_t>(router_partials[static_cast<int64_t>(b) * router_stats + routed_experts + e]);
                } else {
                    const int64_t begin = b * tokens_per_block;
                    here[i] = static_cast<int32_t>(max(int64_t(0), min(begin + tokens_per_block, num_tokens) - begin));
                }
            }
#pragma unroll
            for (int i = 0; i < kBatch; ++i) {
                if (b0 + i < num_blocks) block_prefix[static_cast<int64_t>(b0 + i) * num_experts + e] = running;
                running += here[i];
            }
        }
        count = running;
    }
    write_expert_layout(count, num_experts, pad_to_multiple, index_dtype, expert_ends, expert_pad_begins, expert_begins);
}

// Workgroup b ranks the entries [b * entries_per_block, (b + 1) * entries_per_block) of the flattened `top_experts`,
// 1024 at a time, given the number of earlier entries per expert (`block_prefix[b]`).
__global__ __launch_bounds__(kMapBlock) void sparse_map_rows_kernel(const int64_t *__restrict__ top_experts,
                                                                    int64_t num_entries, int64_t entries_per_block,
                                                                    int num_experts,
                                                                    const int32_t *__restrict__ block_prefix,
                                                                    const int32_t *__restrict__ expert_begins,
                                                                    int index_dtype, void *__restrict__ sparse_rows) {
    static_assert(kMapMaxExperts <= kMapBlock, "thread e keeps the running count of expert e in a register");
    extern __shared__ int32_t lds_wave_counts[];  // [kMapWaves][num_experts] counts per wavefront: 64 KiB at 1024 experts
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int num_bits = log2_ceil(num_experts);
    const int64_t first = static_cast<int64_t>(blockIdx.x) * entries_per_block;
    const int64_t last = min(first + entries_per_block, num_entries);
    // Rows handed out so far to expert threadIdx.x (there are at most as many experts as threads).
    const int own_expert = threadIdx.x;
    int32_t running = 0;
    if (own_expert < num_experts)
        running = expert_begins[own_expert] + block_prefix[static_cast<int64_t>(blockIdx.x) * num_experts + own_expert];

    for (int64_t chunk = first; chunk < last; chunk += kMapBlock) {
        for (int i = threadIdx.x; i < kMapWaves * num_experts; i += kMapBlock) lds_wave_counts[i] = 0;
        __syncthreads();

        const int64_t entry = chunk + threadIdx.x;
        int64_t expert64 = entry < last ? top_experts[entry] : -1;
        const bool valid = expert64 >= 0 && expert64 < num_experts;
        const int expert = valid ? static_cast<int>(expert64) : 0;
        const uint64_t same = match_expert(expert, valid, num_bits);
        const int rank_in_wave = __popcll(same & ((1ull << lane) - 1));
        if (valid && rank_in_wave == 0) lds_wave_counts[wave * num_experts + expert] = __popcll(same);
        __syncthreads();

        // Exclusive prefix over the wavefronts of the workgroup, per expert, in place, on top of the running count.
        if (own_expert < num_experts) {
#pragma unroll
            for (int w = 0; w < kMapWaves; ++w) {
                const int32_t here = lds_wave_counts[w * num_experts + own_expert];
                lds_wave_counts[w * num_experts + own_expert] = running;
                running += here;
            }
        }
        __syncthreads();

        if (entry < last) {
            int64_t row = -1;
            if (valid) row = static_cast<int64_t>(lds_wave_counts[wave * num_experts + expert]) + rank_in_wave;
            store_index(sparse_rows, index_dtype, entry, row);
        }
        __syncthreads();
    }
}

static inline int64_t map_num_blocks(int64_t num_entries) { return (num_entries + kMapBlock - 1) / kMapBlock; }

}  // namespace fm

extern "C" size_t fm_sparse_map_workspace_size(int64_t num_rows_dense, int64_t num_experts_per_token,
                                               int64_t num_experts) {
    if (num_rows_dense < 0 || num_experts_per_token < 0 || num_experts < 0) return 0;
    const int64_t blocks = fm::map_num_blocks(num_rows_dense * num_experts_per_token);
    const size_t bytes = static_cast<size_t>((blocks + 1) * num_experts) * sizeof(int32_t);
    return (bytes + 255) / 256 * 256 + 256;
}

namespace fm {

// Validation and the three launches; `workspace` holds fm_sparse_map_workspace_size(...) bytes.
static int run_sparse_map(const char *name, const int64_t *top_experts, int64_t num_rows_dense,
                          int64_t num_experts_per_token, int64_t num_experts, int64_t pad_to_multiple, int index_dtype,
                          void *sparse_rows, void *expert_ends, void *expert_pad_begins, void *workspace,
                          hipStream_t stream) {
    const int64_t num_entries = num_rows_dense * num_experts_per_token;
    const int blocks = static_cast<int>(map_num_blocks(num_entries));
    const int experts = static_cast<int>(num_experts);
    int32_t *block_counts = static_cast<int32_t *>(workspace);
    int32_t *expert_begins = block_counts + static_cast<int64_t>(blocks) * experts;

    if (blocks > 0) {
        sparse_map_histogram_kernel<<<blocks, kMapBlock, experts * sizeof(int32_t), stream>>>(
            top_experts, num_entries, experts, block_counts);
    }
    sparse_map_layout_kernel<<<1, kMapBlock, 0, stream>>>(block_counts, blocks, experts, pad_to_multiple, index_dtype,
                                                          expert_ends, expert_pad_begins, expert_begins);
    if (blocks > 0) {
        sparse_map_rows_kernel<<<blocks, kMapBlock, kMapWaves * experts * sizeof(int32_t), stream>>>(
            top_experts, num_entries, kMapBlock, experts, block_counts, expert_begins, index_dtype, sparse_rows);
    }
    return check_launch(name);
}

static int check_sparse_map_arguments(const char *name, const int64_t *top_experts, int64_t num_rows_dense,
                                      int64_t num_experts_per_token, int64_t num_experts, int64_t pad_to_multiple,
                                      int index_dtype, void *sparse_rows, void *expert_ends, void *expert_pad_begins) {
    FM_REQUIRE(num_rows_dense >= 0 && num_experts_per_token >= 0, "%s: negative shape", name);
    FM_REQUIRE(num_experts >= 1 && num_experts <= kMapMaxExperts, "%s: num_experts=%lld outside [1, %d]", name,
               (long long)num_experts, kMapMaxExperts);
    FM_REQUIRE(pad_to_multiple >= 1, "%s: pad_to_multiple=%lld < 1", name, (long long)pad_to_multiple);
    FM_REQUIRE(valid_index_dtype(index_dtype), "%s: bad index_dtype %d", name, index_dtype);
    const int64_t num_entries = num_rows_dense * num_experts_per_token;
    const int64_t max_rows = num_entries + num_experts * pad_to_multiple;
    FM_REQUIRE(max_rows < (int64_t(1) << 31), "%s: %lld padded rows overflow int32", name, (long long)max_rows);
    FM_REQUIRE(index_dtype != FM_INDEX_I16 || max_rows <= 32767 + pad_to_multiple,
               "%s: %lld padded rows do not fit int16", name, (long long)max_rows);
    FM_REQUIRE(expert_ends && expert_pad_begins, "%s: null output", name);
    FM_REQUIRE(num_entries == 0 || (top_experts && sparse_rows), "%s: null top_experts/sparse_rows", name);
    return FM_OK;
}

}  // namespace fm

extern "C" int fm_sparse_map(const int64_t *top_experts, int64_t num_rows_dense, int64_t num_experts_per_token,
                             int64_t num_experts, int64_t pad_to_multiple, int index_dtype, void *sparse_rows,
                             void *expert_ends, void *expert_pad_begins, void *workspace, size_t workspace_size,
                             void *stream) {
    using namespace fm;
    if (int status = check_sparse_map_arguments("fm_sparse_map", top_experts, num_rows_dense, num_experts_per_token,
                                                num_experts, pad_to_multiple, index_dtype, sparse_rows, expert_ends,
                                                expert_pad_begins))
        return status;
    FM_REQUIRE(workspace, "fm_sparse_map: null workspace");
    FM_REQUIRE(workspace_size >= fm_sparse_map_workspace_size(num_rows_dense, num_experts_per_token, num_experts),
               "fm_sparse_map: workspace of %zu bytes is too small", workspace_size);
    FM_REQUIRE(aligned16(workspace), "fm_sparse_map: workspace must be 16-byte aligned");
    return run_sparse_map("fm_sparse_map", top_experts, num_rows_dense, num_experts_per_token, num_experts,
                          pad_to_multiple, index_dtype, sparse_rows, expert_ends, expert_pad_begins, workspace,
                          static_cast<hipStream_t>(stream));
}

// ---- the map from the router's own counts ------------------------------------------------------------------
extern "C" size_t fm_sparse_map_from_router_workspace_size(int64_t num_tokens, int64_t num_experts) {
    if (num_tokens < 0 || num_experts < 0) return 0;
    const size_t bytes = static_cast<size_t>(fm::router_blocks(num_tokens) + 1) * num_experts * sizeof(int32_t);
    return (bytes + 255) / 256 * 256 + 256;
}

extern "C" int fm_sparse_map_from_router(const int64_t *top_experts, const void *router_workspace,
                                         size_t router_workspace_size, int64_t num_tokens, int64_t num_experts,
                                         int64_t experts_per_token, int64_t shared_experts, int64_t pad_to_multiple,
                                         int index_dtype, void *sparse_rows, void *expert_ends,
                                         void *expert_pad_begins, void *workspace, size_t workspace_size,
                                         void *stream_) {
    using namespace fm;
    const char *name = "fm_sparse_map_from_router";
    FM_REQUIRE(shared_experts >= 0 && experts_per_token > 0 && num_experts > shared_experts,
               "%s: %lld experts of which %lld shared, %lld per token", name, (long long)num_experts,
               (long long)shared_experts, (long long)experts_per_token);
    const int64_t slots = shared_experts + experts_per_token, routed = num_experts - shared_experts;
    if (int status = check_sparse_map_arguments(name, top_experts, num_tokens, slots, num_experts, pad_to_multiple,
                                                index_dtype, sparse_rows, expert_ends, expert_pad_begins))
        return status;
    FM_REQUIRE(num_tokens > 0, "%s: no tokens (the router does not run on none either)", name);
    const int blocks = router_blocks(num_tokens);
    const int stats = RouterStats::size(static_cast<int>(routed));
    FM_REQUIRE(router_workspace && router_workspace_size >= sizeof(float) * blocks * stats,
               "%s: the router workspace must be the %zu bytes fm_router_forward filled, got %zu", name,
               sizeof(float) * blocks * stats, router_workspace_size);
    FM_REQUIRE(workspace && aligned16(workspace) &&
                   workspace_size >= fm_sparse_map_from_router_workspace_size(num_tokens, num_experts),
               "%s: workspace of %zu bytes is null, misaligned or too small", name, workspace_size);
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    const int experts = static_cast<int>(num_experts);
    const int64_t tokens_per_block = router_tokens_per_block(num_tokens);
    int32_t *block_prefix = static_cast<int32_t *>(workspace);
    int32_t *expert_begins = block_prefix + static_cast<int64_t>(blocks) * experts;
    sparse_map_layout_from_router_kernel<<<1, kMapBlock, 0, stream>>>(
        static_cast<const float *>(router_workspace), stats, blocks, num_tokens, tokens_per_block,
        static_cast<int>(routed), experts, pad_to_multiple, index_dtype, expert_ends, expert_pad_begins, block_prefix,
        expert_begins);
    sparse_map_rows_kernel<<<blocks, kMapBlock, kMapWaves * experts * sizeof(int32_t), stream>>>(
        top_experts, num_tokens * slots, tokens_per_block * slots, experts, block_prefix, expert_begins, index_dtype,
        sparse_rows);
    return check_launch(name);
}

// ---- the same map without any allocation ----------------------------------------------------------------
// The per-workgroup counts live in a fixed array in device memory that is part of the loaded code object: every GPU
// the library runs on holds its own copy, at its own address, until the process ends.
namespace fm {

constexpr size_t kStaticScratchBytes = FM_SPARSE_MAP_STATIC_SCRATCH_BYTES;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

constexpr int kMaxDevices = 64;

// Device address of this device's copy of `scratch`, looked up once per device with that device current. In host
// code the array's name is not a device address; only the pointer returned here may go to kernels.
// `stream` (may be null: the current device's default stream) must belong to the current device: the kernels run where
// the stream lives, and each device has its own copy of the array.
static int static_scratch_of_current_device(hipStream_t stream, void **pointer) {
    static std::mutex mutex;
    static void *addresses[kMaxDevices] = {};
    int device = -1;
    hipError_t error = hipGetDevice(&device);
    if (error != hipSuccess) return fail(FM_ERR_LAUNCH, "fm_sparse_map_static: hipGetDevice: %s", hipGetErrorString(error));
    int stream_device = device;
    if (stream != nullptr && hipStreamGetDevice(stream, &stream_device) == hipSuccess && stream_device != device)
        return fail(FM_ERR_INVALID_ARGUMENT,
                    "fm_sparse_map_static: the stream belongs to device %d but device %d is current; make the stream's "
                    "device current before the call",
                    stream_device, device);
    if (device < 0 || device >= kMaxDevices)
        return fail(FM_ERR_UNSUPPORTED, "fm_sparse_map_static: device %d outside [0, %d)", device, kMaxDevices);
    std::lock_guard<std::mutex> lock(mutex);
    if (addresses[device] == nullptr) {
        void *address = nullptr;
        error = hipGetSymbolAddress(&address, HIP_SYMBOL(scratch));
        if (error != hipSuccess || address == nullptr)
            return fail(FM_ERR_LAUNCH, "fm_sparse_map_static: hipGetSymbolAddress: %s", hipGetErrorString(error));
        addresses[device] = address;
    }
    *pointer = addresses[device];
    return FM_OK;
}

}  // namespace fm

extern "C" size_t fm_sparse_map_static_scratch_size(void) { return fm::kStaticScratchBytes; }

extern "C" int fm_sparse_map_static(const int64_t *top_experts, int64_t num_rows_dense, int64_t num_experts_per_token,
                                    int64_t num_experts, int64_t pad_to_multiple, int index_dtype, void *sparse_rows,
                                    void *expert_ends, void *expert_pad_begins, void *stream) {
    using namespace fm;
    if (int status = check_sparse_map_arguments("fm_sparse_map_static", top_experts, num_rows_dense,
                                                num_experts_per_token, num_experts, pad_to_multiple, index_dtype,
                                                sparse_rows, expert_ends, expert_pad_begins))
        return status;
    const size_t needed = fm_sparse_map_workspace_size(num_rows_dense, num_experts_per_token, num_experts);
    if (needed > kStaticScratchBytes)
        return fail(FM_ERR_UNSUPPORTED,
                    "fm_sparse_map_static: %lld x %lld entries over %lld experts need %zu bytes of scratch, the fixed "
                    "array holds %zu; use fm_sparse_map with a workspace",
                    (long long)num_rows_dense, (long long)num_experts_per_token, (long long)num_experts, needed,
                    kStaticScratchBytes);
    void *workspace = nullptr;
    if (int status = static_scratch_of_current_device(static_cast<hipStream_t>(stream), &workspace)) return status;
    // Nothing to clear: the histogram kernel writes every count the other two kernels read.
    return run_sparse_map("fm_sparse_map_static", top_experts, num_rows_dense, num_experts_per_token, num_experts,
                          pad_to_multiple, index_dtype, sparse_rows, expert_ends, expert_pad_begins, workspace,
                          static_cast<hipStream_t>(stream));
}
