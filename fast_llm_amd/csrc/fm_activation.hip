// MLP activation between the two grouped GEMMs: forward (optionally gated) and backward with optional
// recomputation of the forward output. Pure streaming kernels: every lane handles one 16-byte vector per
// operand, math in fp32, one rounding per stored element.
//
// Formulas follow fast_llm/functional/triton/mlp.py:49-67 (forward) and :100-128 (backward), including the
// overflow-safe form of silu' = sigma^2 + (1 + x) / (2 + e^-x + e^x).
#include "fm_activation_math.h"

namespace fm {

constexpr int kActThreads = 256;

template <typename T, int kActivation, bool kGated, bool kVector>
__global__ __launch_bounds__(kActThreads) void activation_forward_kernel(const T *__restrict__ input,
                                                                         T *__restrict__ output, int64_t columns,
                                                                         uint32_t blocks_per_row) {
    constexpr int N = kVector ? Vec16<T>::N : 1;
    // Consecutive workgroups walk along a row, then to the next row: concurrent accesses stay in a few open pages.
    const int64_t row = blockIdx.x / blocks_per_row;
    const int64_t c = (static_cast<int64_t>(blockIdx.x % blocks_per_row) * kActThreads + threadIdx.x) * N;
    if (c >= columns) return;
    const T *in = input + row * columns * (kGated ? 2 : 1) + c;
    Vec16<T> x, other, result;
    if constexpr (kVector) {
        x = load16_stream(in);
        if constexpr (kGated) other = load16_stream(in + columns);
    } else {
        x.v[0] = in[0];
        if constexpr (kGated) other.v[0] = in[columns];
    }
#pragma unroll
    for (int i = 0; i < N; ++i) {
        float out = activation_forward<kActivation>(to_float(x.v[i]));
        if constexpr (kGated) out *= to_float(other.v[i]);
        result.v[i] = from_float<T>(out);
    }
    if constexpr (kVector) store16_stream(output + row * columns + c, result);
    else output[row * columns + c] = result.v[0];
}

template <typename T, int kActivation, bool kGated, bool kVector>
__global__ __launch_bounds__(kActThreads) void activation_backward_kernel(const T *__restrict__ grad_output,
                                                                          T *__restrict__ grad_input,
                                                                          const T *__restrict__ input,
                                                                          T *__restrict__ output, int64_t columns,
                                                                         uint32_t blocks_per_row) {
    constexpr int N = kVector ? Vec16<T>::N : 1;
    const int64_t row = blockIdx.x / blocks_per_row;
    const int64_t c = (static_cast<int64_t>(blockIdx.x % blocks_per_row) * kActThreads + threadIdx.x) * N;
    if (c >= columns) return;
    const int64_t in_offset = row * columns * (kGated ? 2 : 1) + c;
    const int64_t out_offset = row * columns + c;
    Vec16<T> x, other, go, grad_x, grad_other, recomputed;
    if constexpr (kVector) {
        x = load16_stream(input + in_offset);
        go = load16_stream(grad_output + out_offset);
        if constexpr (kGated) other = load16_stream(input + in_offset + columns);
    } else {
        x.v[0] = input[in_offset];
        go.v[0] = grad_output[out_offset];
        if constexpr (kGated) other.v[0] = input[in_offset + columns];
    }
#pragma unroll
    for (int i = 0; i < N; ++i) {
        float out;
        const float grad = activation_backward<kActivation>(to_float(x.v[i]), out);
        const float g = to_float(go.v[i]);
        if constexpr (kGated) {
            const float up = to_float(other.v[i]);
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

template <typename T, int kActivation, bool kGated>
static void launch_activation(bool forward, const void *grad_output, void *grad_input, const void *input, void *output,
                              int64_t rows, int64_t columns, hipStream_t stream) {
    constexpr int vector = Vec16<T>::N;
    const bool vectorised = columns % vector == 0 && aligned16(input) && aligned16(output) && aligned16(grad_output) &&
                            aligned16(grad_input);
    const int per_block = kActThreads * (vectorised ? vector : 1);
    const uint32_t blocks_per_row = static_cast<uint32_t>((columns + per_block - 1) / per_block);
    const uint32_t grid = static_cast<uint32_t>(rows) * blocks_per_row;
    const T *in = static_cast<const T *>(input);
    T *out = static_cast<T *>(output);
    if (forward) {
        if (vectorised) activation_forward_kernel<T, kActivation, kGated, true><<<grid, kActThreads, 0, stream>>>(in, out, columns, blocks_per_row);
        else activation_forward_kernel<T, kActivation, kGated, false><<<grid, kActThreads, 0, stream>>>(in, out, columns, blocks_per_row);
    } else {
        const T *go = static_cast<const T *>(grad_output);
        T *gi = static_cast<T *>(grad_input);
        if (vectorised) activation_backward_kernel<T, kActivation, kGated, true><<<grid, kActThreads, 0, stream>>>(go, gi, in, out, columns, blocks_per_row);
        else activation_backward_kernel<T, kActivation, kGated, false><<<grid, kActThreads, 0, stream>>>(go, gi, in, out, columns, blocks_per_row);
    }
}

template <typename T>
static void dispatch_activation(int activation, bool gated, bool forward, const void *grad_output, void *grad_input,
                                const void *input, void *output, int64_t rows, int64_t columns, hipStream_t stream) {
#define FM_ACT_CASE(ACT)                                                                                              \
    case ACT:                                                                                                         \
        if (gated) launch_activation<T, ACT, true>(forward, grad_output, grad_input, input, output, rows, columns, stream); \
        else launch_activation<T, ACT, false>(forward, grad_output, grad_input, input, output, rows, columns, stream);      \
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
                            int dtype, void *stream) {
    FM_REQUIRE(rows >= 0 && columns >= 0, "%s: negative shape", name);
    FM_REQUIRE(rows < (int64_t(1) << 31) && columns < (int64_t(1) << 40) && rows * ((columns + 255) / 256) < (int64_t(1) << 31),
               "%s: shape too large", name);
    FM_REQUIRE(valid_dtype(dtype), "%s: bad dtype %d", name, dtype);
    FM_REQUIRE(activation >= FM_ACT_GELU && activation <= FM_ACT_IDENTITY, "%s: bad activation %d", name, activation);
    if (rows == 0 || columns == 0) return FM_OK;
    FM_REQUIRE(input && (forward ? output != nullptr : (grad_output && grad_input)), "%s: null tensor", name);
    FM_DISPATCH_DTYPE(dtype, T, {
        dispatch_activation<T>(activation, gated != 0, forward, grad_output, grad_input, input, output, rows, columns,
                               static_cast<hipStream_t>(stream));
    });
    return check_launch(name);
}

}  // namespace fm

extern "C" int fm_mlp_activation_forward(const void *input, void *output, int64_t num_rows, int64_t num_columns,
                                         int gated, int activation, int dtype, void *stream) {
    return fm::activation_entry("fm_mlp_activation_forward", true, nullptr, nullptr, input, output, num_rows,
                                num_columns, gated, activation, dtype, stream);
}

extern "C" int fm_mlp_activation_backward(const void *grad_output, void *grad_input, const void *input, void *output,
                                          int64_t num_rows, int64_t num_columns, int gated, int activation, int dtype,
                                          void *stream) {
    return fm::activation_entry("fm_mlp_activation_backward", false, grad_output, grad_input, input, output, num_rows,
                                num_columns, gated, activation, dtype, stream);
}
