// MLP activation between the two grouped GEMMs: forward (optionally gated) and backward with optional
// recomputation of the forward output. Pure streaming kernels: every lane handles a few 16-byte vectors per
// operand (all loaded before the first store), math in fp32, one rounding per stored element.
//
// Formulas follow fast_llm/functional/triton/mlp.py:49-67 (forward) and :100-128 (backward), including the
// overflow-safe form of silu' = sigma^2 + (1 + x) / (2 + e^-x + e^x).
#include "fm_activation_math.h"

namespace fm {

constexpr int kActThreads = 256;
constexpr int kActRows = 4;  // rows per workgroup: that many independent vectors per operand in flight per lane

// Rows at and past `*row_limit` (an entry of a sparse map's `expert_ends`, or null: none) are neither read nor
// written: in the static worst-case layout they are rows no expert owns.
struct ActivationShape {
    int64_t columns;  // of the output
    int64_t rows;
    uint32_t blocks_per_row;
    const void *row_limit;
    int index_dtype;
};

__device__ __forceinline__ int64_t rows_in_use(const ActivationShape &shape) {
    if (shape.row_limit == nullptr) return shape.rows;
    return min(shape.rows, load_index(shape.row_limit, shape.index_dtype, 0));
}

// A workgroup handles kActRows consecutive rows x 256 vectors of columns; consecutive workgroups walk along the rows,
// then to the next group of rows. All loads of a lane are issued before its first store.
template <typename T, int kActivation, bool kGated, bool kVector>
__global__ __launch_bounds__(kActThreads) void activation_forward_kernel(const T *__restrict__ input,
                                                                         T *__restrict__ output,
                                                                         ActivationShape shape) {
    constexpr int N = kVector ? Vec16<T>::N : 1;
    const int64_t columns = shape.columns;
    const int64_t row0 = static_cast<int64_t>(blockIdx.x / shape.blocks_per_row) * kActRows;
    const int64_t c = (static_cast<int64_t>(blockIdx.x % shape.blocks_per_row) * kActThreads + threadIdx.x) * N;
    const int64_t rows = rows_in_use(shape);
    if (c >= columns || row0 >= rows) return;
    Vec16<T> x[kActRows], other[kActRows];
#pragma unroll
    for (int r = 0; r < kActRows; ++r) {
        if (row0 + r >= rows) break;
        const T *in = input + (row0 + r) * columns * (kGated ? 2 : 1) + c;
        if constexpr (kVector) {
            x[r] = load16_stream(in);
            if constexpr (kGated) other[r] = load16_stream(in + columns);
        } else {
            x[r].v[0] = in[0];
            if constexpr (kGated) other[r].v[0] = in[columns];
        }
    }
#pragma unroll
    for (int r = 0; r < kActRows; ++r) {
        if (row0 + r >= rows) break;
        Vec16<T> result;
#pragma unroll
        for (int i = 0; i < N; ++i) {
            float out = activation_forward<kActivation>(to_float(x[r].v[i]));
            if constexpr (kGated) out *= to_float(other[r].v[i]);
            result.v[i] = from_float<T>(out);
        }
        if constexpr (kVector) store16_stream(output + (row0 + r) * columns + c, result);
        else output[(row0 + r) * columns + c] = result.v[0];
    }
}

constexpr int kActBackwardRows = 2;

template <typename T, int kActivation, bool kGated, bool kVector>
__global__ __launch_bounds__(kActThreads) void activation_backward_kernel(const T *__restrict__ grad_output,
                                                                          T *__restrict__ grad_input,
                                                                          const T *__restrict__ input,
                                                                          T *__restrict__ output,
                                                                          ActivationShape shape) {
    constexpr int N = kVector ? Vec16<T>::N : 1;
    const int64_t columns = shape.columns;
    const int64_t row0 = static_cast<int64_t>(blockIdx.x / shape.blocks_per_row) * kActBackwardRows;
    const int64_t c = (static_cast<int64_t>(blockIdx.x % shape.blocks_per_row) * kActThreads + threadIdx.x) * N;
    const int64_t rows = rows_in_use(shape);
    if (c >= columns || row0 >= rows) return;
    Vec16<T> x[kActBackwardRows], other[kActBackwardRows], go[kActBackwardRows];
#pragma unroll
    for (int r = 0; r < kActBackwardRows; ++r) {
        if (row0 + r >= rows) break;
        const int64_t in_offset = (row0 + r) * columns * (kGated ? 2 : 1) + c;
        const int64_t out_offset = (row0 + r) * columns + c;
        if constexpr (kVector) {
            x[r] = load16_stream(input + in_offset);
            go[r] = load16_stream(grad_output + out_offset);
            if constexpr (kGated) other[r] = load16_stream(input + in_offset + columns);
        } else {
            x[r].v[0] = input[in_offset];
            go[r].v[0] = grad_output[out_offset];
            if constexpr (kGated) other[r].v[0] = input[in_offset + columns];
        }
    }
#pragma unroll
    for (int r = 0; r < kActBackwardRows; ++r) {
        if (row0 + r >= rows) break;
        const int64_t in_offset = (row0 + r) * columns * (kGated ? 2 : 1) + c;
        const int64_t out_offset = (row0 + r) * columns + c;
        Vec16<T> grad_x, grad_other, recomputed;
#pragma unroll
        for (int i = 0; i < N; ++i) {
            float out;
            const float grad = activation_backward<kActivation>(to_float(x[r].v[i]), out);
            const float g = to_float(go[r].v[i]);
            if constexpr (kGated) {
                const float up = to_float(other[r].v[i]);
                grad_x.v[i] = from_float<T>(grad * up * g);
                grad_other.v[i] = from_float<T>(out * g);
                out = out * up;
            } else {
                grad_x.v[i] = from_float<T>(grad * g);
            }
            recomputed.v[i] = from_float<T>(out);
        }
        if constexpr (kVector) {
            store16_stream(grad_input + in_offset, grad_x);
            if constexpr (kGated) store16_stream(grad_input + in_offset + columns, grad_other);
            if (output != nullptr) store16_stream(output + out_offset, recomputed);
        } else {
            grad_input[in_offset] = grad_x.v[0];
            if constexpr (kGated) grad_input[in_offset + columns] = grad_other.v[0];
            if (output != nullptr) output[out_offset] = recomputed.v[0];
        }
    }
}

template <typename T, int kActivation, bool kGated>
static void launch_activation(bool forward, const void *grad_output, void *grad_input, const void *input, void *output,
                              ActivationShape shape, hipStream_t stream) {
    constexpr int vector = Vec16<T>::N;
    const bool vectorised = shape.columns % vector == 0 && aligned16(input) && aligned16(output) &&
                            aligned16(grad_output) && aligned16(grad_input);
    const int per_block = kActThreads * (vectorised ? vector : 1);
    shape.blocks_per_row = static_cast<uint32_t>((shape.columns + per_block - 1) / per_block);
    const int rows_per_block = forward ? kActRows : kActBackwardRows;
    const uint32_t grid =
        static_cast<uint32_t>((shape.rows + rows_per_block - 1) / rows_per_block) * shape.blocks_per_row;
    const T *in = static_cast<const T *>(input);
    T *out = static_cast<T *>(output);
    if (forward) {
        if (vectorised) activation_forward_kernel<T, kActivation, kGated, true><<<grid, kActThreads, 0, stream>>>(in, out, shape);
        else activation_forward_kernel<T, kActivation, kGated, false><<<grid, kActThreads, 0, stream>>>(in, out, shape);
    } else {
        const T *go = static_cast<const T *>(grad_output);
        T *gi = static_cast<T *>(grad_input);
        if (vectorised) activation_backward_kernel<T, kActivation, kGated, true><<<grid, kActThreads, 0, stream>>>(go, gi, in, out, shape);
        else activation_backward_kernel<T, kActivation, kGated, false><<<grid, kActThreads, 0, stream>>>(go, gi, in, out, shape);
    }
}

template <typename T>
static void dispatch_activation(int activation, bool gated, bool forward, const void *grad_output, void *grad_input,
                                const void *input, void *output, const ActivationShape &shape, hipStream_t stream) {
#define FM_ACT_CASE(ACT)                                                                                              \
    case ACT:                                                                                                         \
        if (gated) launch_activation<T, ACT, true>(forward, grad_output, grad_input, input, output, shape, stream);  \
        else launch_activation<T, ACT, false>(forward, grad_output, grad_input, input, output, shape, stream);       \
        break;
    switch (activation) {
        FM_ACT_CASE(FM_ACT_GELU)
        FM_ACT_CASE(FM_ACT_SILU)
        FM_ACT_CASE(FM_ACT_RELU)
        FM_ACT_CASE(FM_ACT_SQUARED_RELU)
        default:
        FM_ACT_CASE(FM_ACT_IDENTITY)
    }
#undef FM_ACT_CASE
}

static int activation_entry(const char *name, bool forward, const void *grad_output, void *grad_input,
                            const void *input, void *output, int64_t rows, int64_t columns, int gated, int activation,
                            int dtype, const void *row_limit, int index_dtype, void *stream) {
    FM_REQUIRE(rows >= 0 && columns >= 0, "%s: negative shape", name);
    FM_REQUIRE(rows < (int64_t(1) << 31) && columns < (int64_t(1) << 40) && rows * ((columns + 255) / 256) < (int64_t(1) << 31),
               "%s: shape too large", name);
    FM_REQUIRE(valid_dtype(dtype), "%s: bad dtype %d", name, dtype);
    FM_REQUIRE(activation >= FM_ACT_GELU && activation <= FM_ACT_IDENTITY, "%s: bad activation %d", name, activation);
    FM_REQUIRE(row_limit == nullptr || valid_index_dtype(index_dtype), "%s: bad index_dtype %d", name, index_dtype);
    if (rows == 0 || columns == 0) return FM_OK;
    FM_REQUIRE(input && (forward ? output != nullptr : (grad_output && grad_input)), "%s: null tensor", name);
    const ActivationShape shape{columns, rows, 0, row_limit, index_dtype};
    FM_DISPATCH_DTYPE(dtype, T, {
        dispatch_activation<T>(activation, gated != 0, forward, grad_output, grad_input, input, output, shape,
                               static_cast<hipStream_t>(stream));
    });
    return check_launch(name);
}

}  // namespace fm

extern "C" int fm_mlp_activation_forward(const void *input, void *output, int64_t num_rows, int64_t num_columns,
                                         int gated, int activation, int dtype, const void *row_limit, int index_dtype,
                                         void *stream) {
    return fm::activation_entry("fm_mlp_activation_forward", true, nullptr, nullptr, input, output, num_rows,
                                num_columns, gated, activation, dtype, row_limit, index_dtype, stream);
}

extern "C" int fm_mlp_activation_backward(const void *grad_output, void *grad_input, const void *input, void *output,
                                          int64_t num_rows, int64_t num_columns, int gated, int activation, int dtype,
                                          const void *row_limit, int index_dtype, void *stream) {
    return fm::activation_entry("fm_mlp_activation_backward", false, grad_output, grad_input, input, output, num_rows,
                                num_columns, gated, activation, dtype, row_limit, index_dtype, stream);
}
