// Bandwidth-bound gather/scatter between the dense token layout [T, H] and the expert-sorted sparse layout
// [R, H]: dispatch (dense -> sparse), combine (sparse -> dense), the score gradient of the combine, and the
// fused backward of the combine.
//
// One workgroup per token row. Every lane moves 16-byte vectors (8 bf16 / 4 fp32), consecutive lanes touch
// consecutive vectors, so each wavefront access is one contiguous 1 KiB segment of a row. The k row indices
// and scores of a token are wave-uniform and live in scalar registers. Rows whose index is negative (the sparse
// map marks out-of-range experts that way) or not below the sparse buffer's row count are skipped.
//
// Arithmetic contract (reference: fast_llm/functional/triton/sparse_copy.py:27-49, 69-90, 111-148):
// products and sums in fp32, scores converted to fp32 on load, one rounding at the store, combine adds the
// slots in the order j = 0 .. k-1.
#include "fm_common.h"

namespace fm {

constexpr int kCopyThreads = 256;
// Gathered sparse rows are read once. While the sparse buffer fits the 256 MiB Infinity Cache, the rows the previous
// kernel wrote are still there and ordinary loads find them (measured inside a training step at 142 MB: streaming loads
// 2 % slower in the combine, 13 % in its backward); beyond that size streaming loads are faster (604 MB: 7 % and 3 %).
constexpr int64_t kStreamGatherBytes = int64_t(256) << 20;

struct CopyArgs {
    const void *sparse_rows;
    const void *scores;  // may be null
    int64_t num_columns;
    int64_t num_rows_sparse;  // sparse rows outside [0, num_rows_sparse) are skipped
    int experts_per_token;
    int index_dtype;
    int scores_dtype;
    bool stream_gather;  // sparse rows are read with streaming loads (the sparse buffer is larger than the Infinity Cache)
};

__device__ __forceinline__ float load_score(const void *scores, int scores_dtype, int64_t i) {
    if (scores_dtype == FM_DTYPE_F32) return static_cast<const float *>(scores)[i];
    if (scores_dtype == FM_DTYPE_BF16) return to_float(static_cast<const bf16_t *>(scores)[i]);
    return to_float(static_cast<const f16_t *>(scores)[i]);
}

// ---- dispatch ------------------------------------------------------------------------------------------
// One workgroup per token. kChunks > 0: the row has at most kChunks vectors per lane, all loaded before the first
// store (more bytes in flight per CU); kChunks = 0: any row length, one vector per lane at a time.
template <typename T, bool kVector, int kChunks>
__global__ __launch_bounds__(kCopyThreads) void copy_dense_to_sparse_kernel(const T *__restrict__ input,
                                                                            T *__restrict__ output, CopyArgs args) {
    constexpr int N = kVector ? Vec16<T>::N : 1;
    constexpr int kPasses = kChunks > 0 ? kChunks : 1;
    const int64_t columns = args.num_columns;
    const int k = args.experts_per_token;
    const int64_t stride = static_cast<int64_t>(blockDim.x) * N;
    const int64_t token = blockIdx.x;
    for (int64_t c0 = static_cast<int64_t>(threadIdx.x) * N; c0 < columns; c0 += stride * kPasses) {
        Vec16<T> value[kPasses];
        const T *in_row = input + token * columns;
#pragma unroll
        for (int q = 0; q < kPasses; ++q) {
            const int64_t c = c0 + q * stride;
            if (c < columns) {
                if constexpr (kVector) value[q] = load16(in_row + c);
                else value[q].v[0] = in_row[c];
            }
        }
        for (int j = 0; j < k; ++j) {
            const int64_t row = load_index(args.sparse_rows, args.index_dtype, token * k + j);
            if (row < 0 || row >= args.num_rows_sparse) continue;
            const bool scaled_copy = args.scores != nullptr;
            const float score = scaled_copy ? load_score(args.scores, args.scores_dtype, token * k + j) : 1.f;
#pragma unroll
            for (int q = 0; q < kPasses; ++q) {
                const int64_t c = c0 + q * stride;
                if (c >= columns) continue;
                Vec16<T> scaled = value[q];
                if (scaled_copy) {
#pragma unroll
                    for (int i = 0; i < N; ++i) scaled.v[i] = from_float<T>(to_float(value[q].v[i]) * score);
                }
                if constexpr (kVector) store16(output + row * columns + c, scaled);
                else output[row * columns + c] = scaled.v[0];
            }
        }
        if (kChunks > 0) break;
    }
}

// ---- combine -------------------------------------------------------------------------------------------
// Slots are taken two at a time: all loads of a pair (and of all the lane's vectors) are issued before the first
// addition; the additions keep the slot order j = 0 .. k - 1.
template <typename T, bool kVector, int kChunks, bool kStreamGather = false>
__global__ __launch_bounds__(kCopyThreads) void copy_sparse_to_dense_kernel(const T *__restrict__ input,
                                                                            T *__restrict__ output, CopyArgs args) {
    constexpr int N = kVector ? Vec16<T>::N : 1;
    constexpr int kPasses = kChunks > 0 ? kChunks : 1;
    constexpr int kGroup = 2;
    const int64_t columns = args.num_columns;
    const int k = args.experts_per_token;
    const int64_t stride = static_cast<int64_t>(blockDim.x) * N;
    const int64_t token = blockIdx.x;
    for (int64_t c0 = static_cast<int64_t>(threadIdx.x) * N; c0 < columns; c0 += stride * kPasses) {
        float sum[kPasses][N];
#pragma unroll
        for (int q = 0; q < kPasses; ++q)
#pragma unroll
            for (int i = 0; i < N; ++i) sum[q][i] = 0.f;
        for (int j0 = 0; j0 < k; j0 += kGroup) {
            Vec16<T> value[kGroup][kPasses];
            float score[kGroup];
            bool present[kGroup];
#pragma unroll
            for (int u = 0; u < kGroup; ++u) {
                const int j = j0 + u;
                const int64_t row = j < k ? load_index(args.sparse_rows, args.index_dtype, token * k + j) : -1;
                present[u] = row >= 0 && row < args.num_rows_sparse;
                score[u] = 1.f;
                if (present[u]) {
                    if (args.scores != nullptr) score[u] = load_score(args.scores, args.scores_dtype, token * k + j);
#pragma unroll
                    for (int q = 0; q < kPasses; ++q) {
                        const int64_t c = c0 + q * stride;
                        if (c < columns) {
                            if constexpr (kVector)
                                value[u][q] = kStreamGather ? load16_stream(input + row * columns + c)
                                                            : load16(input + row * columns + c);
                            else value[u][q].v[0] = input[row * columns + c];
                        }
                    }
                }
            }
#pragma unroll
            for (int u = 0; u < kGroup; ++u) {
                if (!present[u]) continue;
#pragma unroll
                for (int q = 0; q < kPasses; ++q) {
                    if (args.scores != nullptr) {
#pragma unroll
                        for (int i = 0; i < N; ++i) sum[q][i] += to_float(value[u][q].v[i]) * score[u];
                    } else {
#pragma unroll
                        for (int i = 0; i < N; ++i) sum[q][i] += to_float(value[u][q].v[i]);
                    }
                }
            }
        }
#pragma unroll
        for (int q = 0; q < kPasses; ++q) {
            const int64_t c = c0 + q * stride;
            if (c >= columns) continue;
            Vec16<T> result;
#pragma unroll
            for (int i = 0; i < N; ++i) result.v[i] = from_float<T>(sum[q][i]);
            if constexpr (kVector) store16(output + token * columns + c, result);
            else output[token * columns + c] = result.v[0];
        }
        if (kChunks > 0) break;
    }
}

// ---- score gradient, optionally fused with the scaled dispatch of grad_output ---------------------------
// grad_scores[t, j] = <input[row(t, j), :], grad_output[t, :]>; when kFused also
// grad_input[row(t, j), :] = grad_output[t, :] * scores[t, j].
// kChunks vectors of grad_output per lane are kept in registers across the k slots.
// kAhead: the rows of slot j + 1 are requested before slot j is reduced (pays from three slots per token on).
template <typename T, typename OutT, bool kVector, bool kFused, int kChunks, bool kStreamGather = false,
          bool kAhead = false>
__global__ __launch_bounds__(kCopyThreads) void grad_score_kernel(const T *__restrict__ input,
                                                                  const T *__restrict__ grad_output,
                                                                  T *__restrict__ grad_input,
                                                                  OutT *__restrict__ grad_scores, CopyArgs args) {
    constexpr int N = kVector ? Vec16<T>::N : 1;
    __shared__ float lds_partial[kCopyThreads / 64];
    const int64_t token = blockIdx.x;
    const int64_t columns = args.num_columns;
    const int k = args.experts_per_token;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, waves = blockDim.x >> 6;
    const T *grad_row = grad_output + token * columns;

    Vec16<T> grad[kChunks > 0 ? kChunks : 1];
    if constexpr (kChunks > 0) {
#pragma unroll
        for (int q = 0; q < kChunks; ++q) {
            const int64_t c = (static_cast<int64_t>(q) * blockDim.x + threadIdx.x) * N;
            if (c < columns) {
                if constexpr (kVector) grad[q] = load16(grad_row + c);
                else grad[q].v[0] = grad_row[c];
            }
        }
    }

    // The reduction of a slot's products over the workgroup, and the store of the result.
    auto finish_slot = [&](int j, float partial) {
        partial = wave_sum(partial);
        if (lane == 0) lds_partial[wave] = partial;
        __syncthreads();
        if (threadIdx.x == 0) {
            float total = 0.f;
            for (int w = 0; w < waves; ++w) total += lds_partial[w];
            grad_scores[token * k + j] = from_float<OutT>(total);
        }
        __syncthreads();
    };
    auto products = [&](const Vec16<T> &value, const Vec16<T> &g, float score, T *out, float &partial) {
#pragma unroll
        for (int i = 0; i < N; ++i) partial += to_float(value.v[i]) * to_float(g.v[i]);
        if constexpr (kFused) {
            Vec16<T> scaled;
#pragma unroll
            for (int i = 0; i < N; ++i) scaled.v[i] = from_float<T>(to_float(g.v[i]) * score);
            if constexpr (kVector) store16_stream(out, scaled);
            else out[0] = scaled.v[0];
        }
    };

    if constexpr (kChunks > 0 && kAhead) {
        // The lane's vectors of slot j + 1 are requested before slot j is reduced (two barriers and an LDS round trip
        // per slot): a slot's memory latency overlaps the previous slot's reduction.
        struct Slot {
            int64_t row;
            float score;
            Vec16<T> value[kChunks];
        };
        auto request = [&](int j, Slot &slot) {
            slot.row = load_index(args.sparse_rows, args.index_dtype, token * k + j);
            slot.score = 0.f;
            if constexpr (kFused) slot.score = load_score(args.scores, args.scores_dtype, token * k + j);
            if (slot.row < 0 || slot.row >= args.num_rows_sparse) {
                slot.row = -1;
                return;
            }
            const T *in_row = input + slot.row * columns;
#pragma unroll
            for (int q = 0; q < kChunks; ++q) {
                const int64_t c = (static_cast<int64_t>(q) * blockDim.x + threadIdx.x) * N;
                if (c < columns) {
                    if constexpr (kVector) slot.value[q] = kStreamGather ? load16_stream(in_row + c) : load16(in_row + c);
                    else slot.value[q].v[0] = in_row[c];
                }
            }
        };
        auto process = [&](int j, const Slot &slot) {
            float partial = 0.f;
            if (slot.row >= 0) {
                T *out_row = kFused ? grad_input + slot.row * columns : nullptr;
#pragma unroll
                for (int q = 0; q < kChunks; ++q) {
                    const int64_t c = (static_cast<int64_t>(q) * blockDim.x + threadIdx.x) * N;
                    if (c < columns) products(slot.value[q], grad[q], slot.score, out_row + c, partial);
                }
            }
            finish_slot(j, partial);
        };
        Slot even, odd;
        request(0, even);
        for (int j = 0; j < k; j += 2) {
            if (j + 1 < k) request(j + 1, odd);
            process(j, even);
            if (j + 2 < k) request(j + 2, even);
            if (j + 1 < k) process(j + 1, odd);
        }
    } else {
        for (int j = 0; j < k; ++j) {
            const int64_t row = load_index(args.sparse_rows, args.index_dtype, token * k + j);
            float score = 0.f;
            if constexpr (kFused) score = load_score(args.scores, args.scores_dtype, token * k + j);
            float partial = 0.f;
            if (row >= 0 && row < args.num_rows_sparse) {
                const T *in_row = input + row * columns;
                T *out_row = kFused ? grad_input + row * columns : nullptr;
                auto column = [&](const Vec16<T> &g, int64_t c) {
                    Vec16<T> value;
                    if constexpr (kVector) value = kStreamGather ? load16_stream(in_row + c) : load16(in_row + c);
                    else value.v[0] = in_row[c];
                    products(value, g, score, out_row + c, partial);
                };
                if constexpr (kChunks > 0) {
#pragma unroll
                    for (int q = 0; q < kChunks; ++q) {
                        const int64_t c = (static_cast<int64_t>(q) * blockDim.x + threadIdx.x) * N;
                        if (c < columns) column(grad[q], c);
                    }
                } else {
                    for (int64_t c = static_cast<int64_t>(threadIdx.x) * N; c < columns;
                         c += static_cast<int64_t>(blockDim.x) * N) {
                        Vec16<T> g;
                        if constexpr (kVector) g = load16(grad_row + c);
                        else g.v[0] = grad_row[c];
                        column(g, c);
                    }
                }
            }
            finish_slot(j, partial);
        }
    }
}

// Lanes that share a row when each is to move `per_lane` vectors of `vector` elements.
static int copy_threads(int64_t num_columns, int vector, int per_lane = 1) {
    const int64_t chunks = ((num_columns + vector - 1) / vector + per_lane - 1) / per_lane;
    int64_t threads = (chunks + 63) / 64 * 64;
    if (threads > kCopyThreads) threads = kCopyThreads;
    if (threads < 64) threads = 64;
    return static_cast<int>(threads);
}

#define FM_DEFINE_COPY_LAUNCHER(NAME, KERNEL)                                                                        \
    template <typename T>                                                                                            \
    static void NAME(const T *in, T *out, int64_t rows, const CopyArgs &args, bool vectorised, int chunks,          \
                     int threads, hipStream_t stream) {                                                              \
        if (!vectorised) KERNEL<T, false, 0><<<rows, threads, 0, stream>>>(in, out, args);                           \
        else if (chunks <= 1) KERNEL<T, true, 1><<<rows, threads, 0, stream>>>(in, out, args);                       \
        else if (chunks <= 2) KERNEL<T, true, 2><<<rows, threads, 0, stream>>>(in, out, args);                       \
        else if (chunks <= 4) KERNEL<T, true, 4><<<rows, threads, 0, stream>>>(in, out, args);                       \
        else if (chunks <= 8) KERNEL<T, true, 8><<<rows, threads, 0, stream>>>(in, out, args);                       \
        else KERNEL<T, true, 0><<<rows, threads, 0, stream>>>(in, out, args);                                        \
    }
FM_DEFINE_COPY_LAUNCHER(launch_dispatch, copy_dense_to_sparse_kernel)
#undef FM_DEFINE_COPY_LAUNCHER

template <typename T>
static void launch_combine(const T *in, T *out, int64_t rows, const CopyArgs &args, bool vectorised, int chunks,
                           int threads, hipStream_t stream) {
#define FM_LAUNCH_COMBINE(VEC, CHUNKS)                                                                       \
    do {                                                                                                     \
        if (args.stream_gather)                                                                              \
            copy_sparse_to_dense_kernel<T, VEC, CHUNKS, true><<<rows, threads, 0, stream>>>(in, out, args);  \
        else                                                                                                 \
            copy_sparse_to_dense_kernel<T, VEC, CHUNKS, false><<<rows, threads, 0, stream>>>(in, out, args); \
    } while (0)
    if (!vectorised) copy_sparse_to_dense_kernel<T, false, 0><<<rows, threads, 0, stream>>>(in, out, args);
    else if (chunks <= 1) FM_LAUNCH_COMBINE(true, 1);
    else if (chunks <= 2) FM_LAUNCH_COMBINE(true, 2);
    else if (chunks <= 4) FM_LAUNCH_COMBINE(true, 4);
    else if (chunks <= 8) FM_LAUNCH_COMBINE(true, 8);
    else FM_LAUNCH_COMBINE(true, 0);
#undef FM_LAUNCH_COMBINE
}

// Vectors of `vector` elements a lane handles when `threads` lanes share a row.
static int chunks_per_lane(int64_t num_columns, int vector, int threads) {
    const int64_t per_pass = static_cast<int64_t>(vector) * threads;
    return static_cast<int>(min((num_columns + per_pass - 1) / per_pass, static_cast<int64_t>(1 << 20)));
}

static int validate_copy(const char *name, const void *a, const void *b, const void *sparse_rows, int64_t rows,
                         int64_t columns, int64_t k, int64_t rows_sparse, int dtype, int scores_dtype,
                         int index_dtype) {
    FM_REQUIRE(rows >= 0 && columns >= 0 && k >= 0 && rows_sparse >= 0, "%s: negative shape", name);
    FM_REQUIRE(rows < (int64_t(1) << 31), "%s: too many rows", name);
    FM_REQUIRE(valid_dtype(dtype) && valid_dtype(scores_dtype), "%s: bad dtype", name);
    FM_REQUIRE(valid_index_dtype(index_dtype), "%s: bad index_dtype %d", name, index_dtype);
    FM_REQUIRE(rows == 0 || columns == 0 || (a && b), "%s: null tensor", name);
    FM_REQUIRE(rows == 0 || k == 0 || sparse_rows, "%s: null sparse_rows", name);
    return FM_OK;
}

}  // namespace fm

using namespace fm;

extern "C" int fm_copy_dense_to_sparse(const void *input, const void *scores, const void *sparse_rows, void *output,
                                       int64_t num_rows_dense, int64_t num_columns, int64_t num_experts_per_token,
                                       int64_t num_rows_sparse, int dtype, int scores_dtype, int index_dtype,
                                       void *stream_) {
    const char *name = "fm_copy_dense_to_sparse";
    if (int status = validate_copy(name, input, output, sparse_rows, num_rows_dense, num_columns,
                                   num_experts_per_token, num_rows_sparse, dtype, scores_dtype, index_dtype))
        return status;
    if (num_rows_dense == 0 || num_columns == 0 || num_experts_per_token == 0) return FM_OK;
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    CopyArgs args{sparse_rows, scores, num_columns, num_rows_sparse, static_cast<int>(num_experts_per_token), index_dtype, scores_dtype,
                  num_rows_sparse * num_columns * dtype_size(dtype) > kStreamGatherBytes};
    const int vector = 16 / dtype_size(dtype);
    const bool vectorised = num_columns % vector == 0 && aligned16(input) && aligned16(output);
    // Two vectors per lane (measured on MI355X, inside a training step: rows of 4 KiB go 7 % faster with 128 lanes x 2
    // than with 256 x 1; 8 KiB rows take 256 x 2 either way; four or more per lane, or 512 lanes per row, are slower).
    const int threads = copy_threads(num_columns, vectorised ? vector : 1, 2);
    const int chunks = chunks_per_lane(num_columns, vectorised ? vector : 1, threads);
    FM_DISPATCH_DTYPE(dtype, T, {
        launch_dispatch<T>(static_cast<const T *>(input), static_cast<T *>(output), num_rows_dense, args, vectorised, chunks,
                    threads, stream);
    });
    return check_launch(name);
}

extern "C" int fm_copy_sparse_to_dense(const void *input, const void *scores, const void *sparse_rows, void *output,
                                       int64_t num_rows_dense, int64_t num_columns, int64_t num_experts_per_token,
                                       int64_t num_rows_sparse, int dtype, int scores_dtype, int index_dtype,
                                       void *stream_) {
    const char *name = "fm_copy_sparse_to_dense";
    if (int status = validate_copy(name, num_experts_per_token ? input : output, output, sparse_rows, num_rows_dense,
                                   num_columns, num_experts_per_token, num_rows_sparse, dtype, scores_dtype,
                                   index_dtype))
        return status;
    if (num_rows_dense == 0 || num_columns == 0) return FM_OK;
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    CopyArgs args{sparse_rows, scores, num_columns, num_rows_sparse, static_cast<int>(num_experts_per_token), index_dtype, scores_dtype,
                  num_rows_sparse * num_columns * dtype_size(dtype) > kStreamGatherBytes};
    const int vector = 16 / dtype_size(dtype);
    const bool vectorised = num_columns % vector == 0 && aligned16(input) && aligned16(output);
    const int threads = copy_threads(num_columns, vectorised ? vector : 1, 2);
    const int chunks = chunks_per_lane(num_columns, vectorised ? vector : 1, threads);
    FM_DISPATCH_DTYPE(dtype, T, {
        launch_combine<T>(static_cast<const T *>(input), static_cast<T *>(output), num_rows_dense, args, vectorised, chunks,
                    threads, stream);
    });
    return check_launch(name);
}

namespace fm {

template <typename T, typename OutT, bool kFused>
static void launch_grad_score(const void *input, const void *grad_output, void *grad_input, void *grad_scores,
                              int64_t rows, const CopyArgs &args, bool vectorised, int threads, hipStream_t stream) {
    const T *in = static_cast<const T *>(input);
    const T *go = static_cast<const T *>(grad_output);
    T *gi = static_cast<T *>(grad_input);
    OutT *gs = static_cast<OutT *>(grad_scores);
    const int vector = vectorised ? Vec16<T>::N : 1;
    const int64_t chunks = (args.num_columns + static_cast<int64_t>(vector) * threads - 1) /
                           (static_cast<int64_t>(vector) * threads);
#define FM_LAUNCH_GS_STREAM(VEC, CHUNKS, STREAM)                                                                   \
    do {                                                                                                            \
        if (args.experts_per_token > 2 && CHUNKS > 0)                                                               \
            grad_score_kernel<T, OutT, VEC, kFused, CHUNKS, STREAM, true><<<rows, threads, 0, stream>>>(in, go, gi, gs, args); \
        else                                                                                                        \
            grad_score_kernel<T, OutT, VEC, kFused, CHUNKS, STREAM, false><<<rows, threads, 0, stream>>>(in, go, gi, gs, args); \
    } while (0)
#define FM_LAUNCH_GS(VEC, CHUNKS)                                       \
    do {                                                                \
        if (args.stream_gather) FM_LAUNCH_GS_STREAM(VEC, CHUNKS, true); \
        else FM_LAUNCH_GS_STREAM(VEC, CHUNKS, false);                   \
    } while (0)
    if (vectorised) {
        if (chunks <= 1) FM_LAUNCH_GS(true, 1);
        else if (chunks <= 2) FM_LAUNCH_GS(true, 2);
        else if (chunks <= 4) FM_LAUNCH_GS(true, 4);
        else FM_LAUNCH_GS(true, 0);
    } else {
        FM_LAUNCH_GS(false, 0);
    }
#undef FM_LAUNCH_GS
#undef FM_LAUNCH_GS_STREAM
}

template <bool kFused>
static int grad_score_entry(const char *name, const void *input, const void *grad_output, const void *scores,
                            const void *sparse_rows, void *grad_input, void *grad_scores, int64_t num_rows_dense,
                            int64_t num_columns, int64_t num_experts_per_token, int64_t num_rows_sparse, int dtype,
                            int scores_dtype, int out_dtype, int index_dtype, void *stream_) {
    if (int status = validate_copy(name, input, grad_output, sparse_rows, num_rows_dense, num_columns,
                                   num_experts_per_token, num_rows_sparse, dtype, scores_dtype, index_dtype))
        return status;
    FM_REQUIRE(valid_dtype(out_dtype), "%s: bad out_dtype %d", name, out_dtype);
    if (num_rows_dense == 0 || num_experts_per_token == 0) return FM_OK;
    FM_REQUIRE(grad_scores, "%s: null grad_scores", name);
    if (kFused) FM_REQUIRE(scores && (grad_input || num_columns == 0), "%s: null scores or grad_input", name);
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    CopyArgs args{sparse_rows, scores, num_columns, num_rows_sparse, static_cast<int>(num_experts_per_token), index_dtype, scores_dtype,
                  num_rows_sparse * num_columns * dtype_size(dtype) > kStreamGatherBytes};
    const int vector = 16 / dtype_size(dtype);
    const bool vectorised = num_columns % vector == 0 && aligned16(input) && aligned16(grad_output) &&
                            (!kFused || aligned16(grad_input));
    const int threads = copy_threads(num_columns, vectorised ? vector : 1);
    FM_DISPATCH_DTYPE(dtype, T, {
        FM_DISPATCH_DTYPE(out_dtype, OutT, {
            launch_grad_score<T, OutT, kFused>(input, grad_output, grad_input, grad_scores, num_rows_dense, args,
                                               vectorised, threads, stream);
        });
    });
    return check_launch(name);
}

}  // namespace fm

extern "C" int fm_copy_sparse_to_dense_grad_score(const void *input, const void *grad_output, const void *sparse_rows,
                                                  void *grad_scores, int64_t num_rows_dense, int64_t num_columns,
                                                  int64_t num_experts_per_token, int64_t num_rows_sparse, int dtype,
                                                  int out_dtype, int index_dtype, void *stream) {
    return grad_score_entry<false>("fm_copy_sparse_to_dense_grad_score", input, grad_output, nullptr, sparse_rows,
                                   nullptr, grad_scores, num_rows_dense, num_columns, num_experts_per_token,
                                   num_rows_sparse, dtype, FM_DTYPE_F32, out_dtype, index_dtype, stream);
}

extern "C" int fm_copy_sparse_to_dense_backward(const void *input, const void *grad_output, const void *scores,
                                                const void *sparse_rows, void *grad_input, void *grad_scores,
                                                int64_t num_rows_dense, int64_t num_columns,
                                                int64_t num_experts_per_token, int64_t num_rows_sparse, int dtype,
                                                int scores_dtype, int out_dtype, int index_dtype, void *stream) {
    return grad_score_entry<true>("fm_copy_sparse_to_dense_backward", input, grad_output, scores, sparse_rows,
                                  grad_input, grad_scores, num_rows_dense, num_columns, num_experts_per_token,
                                  num_rows_sparse, dtype, scores_dtype, out_dtype, index_dtype, stream);
}
