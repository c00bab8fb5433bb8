// Activation formulas shared by the streaming activation kernels and the fused grouped-GEMM epilogues, so that a
// fused result is bit-identical to the unfused one. They follow fast_llm/functional/triton/mlp.py:49-67 (forward)
// and :100-128 (backward), including the overflow-safe form of silu' = sigma^2 + (1 + x) / (2 + e^-x + e^x).
#pragma once

#include "fm_common.h"

namespace fm {

// Hardware exponential and reciprocal (v_exp_f32, v_rcp_f32; about 1 ulp each). With the libm versions a gated-SiLU
// lane spends ~40 instructions per element and the kernels become VALU-bound instead of HBM-bound.
__device__ __forceinline__ float fast_exp(float x) { return __expf(x); }
__device__ __forceinline__ float fast_rcp(float x) { return __builtin_amdgcn_rcpf(x); }

// Returns act'(x) and writes act(x) to `out`.
template <int kActivation>
__device__ __forceinline__ float activation_backward(float x, float &out) {
    if constexpr (kActivation == FM_ACT_GELU) {
        const float tanh_input = 0.79788456f * x * (1.f + 0.044715f * x * x);
        const float tanh_value = 1.f - 2.f * fast_rcp(1.f + fast_exp(2.f * tanh_input));
        out = x * 0.5f * (1.f + tanh_value);
        return 0.5f * x * ((1.f - tanh_value * tanh_value) * (0.79788456f + 0.1070322243f * x * x)) +
               0.5f * (1.f + tanh_value);
    } else if constexpr (kActivation == FM_ACT_SILU) {
        const float exp_neg = fast_exp(-x);
        const float sigma = fast_rcp(1.f + exp_neg);
        out = x * sigma;
        return sigma * sigma + (1.f + x) * fast_rcp(2.f + exp_neg + fast_rcp(exp_neg));
    } else if constexpr (kActivation == FM_ACT_RELU) {
        out = x > 0.f ? x : 0.f;
        return x > 0.f ? 1.f : 0.f;
    } else if constexpr (kActivation == FM_ACT_SQUARED_RELU) {
        const float relu = x > 0.f ? x : 0.f;
        out = relu * relu;
        return 2.f * relu;
    } else {
        out = x;
        return 1.f;
    }
}

// The forward value is taken from the same expression the backward kernel uses when it recomputes the output,
// so a recomputed activation is bit-identical to the stored one.
template <int kActivation>
__device__ __forceinline__ float activation_forward(float x) {
    float out;
    (void)activation_backward<kActivation>(x, out);
    return out;
}

// Runs the statement with `kActivation` a compile-time constant equal to the run-time tag `activation`.
#define FM_DISPATCH_ACTIVATION(activation, kActivation, ...)                                   \
    switch (activation) {                                                                      \
        case FM_ACT_GELU: { constexpr int kActivation = FM_ACT_GELU; __VA_ARGS__; break; }     \
        case FM_ACT_SILU: { constexpr int kActivation = FM_ACT_SILU; __VA_ARGS__; break; }     \
        case FM_ACT_RELU: { constexpr int kActivation = FM_ACT_RELU; __VA_ARGS__; break; }     \
        case FM_ACT_SQUARED_RELU: { constexpr int kActivation = FM_ACT_SQUARED_RELU; __VA_ARGS__; break; } \
        default: { constexpr int kActivation = FM_ACT_IDENTITY; __VA_ARGS__; break; }          \
    }

}  // namespace fm
