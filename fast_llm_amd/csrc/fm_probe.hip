// Measurement probes, not on the MoE path: what the matrix cores and the HBM of the device sustain, so that kernel
// figures can be set against a measured ceiling next to the published peak.
//   fm_probe_mfma: a register-only loop of back-to-back v_mfma_f32_32x32x16_bf16 (the instruction of the grouped
//     products), 4 x 4 accumulators per wavefront fed from 8 + 8 operand fragments that hold zeros or normal(0, sigma)
//     bf16 values. The chip lowers its clock under power, and operand toggling costs power: the rate on random data
//     is the ceiling a product on real activations can reach, the rate on zeros is the published peak.
//   fm_probe_copy: a plain streaming copy (16-byte vectors, one read and one write per byte).
#include "fm_common.h"

namespace fm {

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 probe_bf16x8_t;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float probe_f32x16_t;

constexpr int kProbeMfmasPerIteration = 32;

__device__ __forceinline__ uint32_t probe_hash(uint32_t x) {
    x ^= x >> 16;
    x *= 0x7feb352du;
    x ^= x >> 15;
    x *= 0x846ca68bu;
    x ^= x >> 16;
    return x;
}

// Box-Muller on two hashed uniforms.
__device__ __forceinline__ float probe_normal(uint32_t seed) {
    const float u1 = (probe_hash(seed) >> 8) * (1.0f / 16777216.0f) + 1e-7f;
    const float u2 = (probe_hash(seed ^ 0x9e3779b9u) >> 8) * (1.0f / 16777216.0f);
    return sqrtf(-2.f * logf(u1)) * cosf(6.2831853f * u2);
}

__global__ __launch_bounds__(256, 1) void probe_mfma_kernel(float *sink, int64_t iterations, int random_operands,
                                                            float sigma) {
    probe_bf16x8_t a[8], b[8];
#pragma unroll
    for (int f = 0; f < 8; ++f)
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const uint32_t seed = ((blockIdx.x * 256 + threadIdx.x) * 8 + f) * 16 + i;
            a[f][i] = random_operands ? static_cast<__bf16>(sigma * probe_normal(seed)) : static_cast<__bf16>(0.f);
            b[f][i] = random_operands ? static_cast<__bf16>(sigma * probe_normal(seed + 8)) : static_cast<__bf16>(0.f);
        }
    probe_f32x16_t acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;
    for (int64_t iteration = 0; iteration < iterations; ++iteration) {
#pragma unroll
        for (int half = 0; half < 2; ++half)
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[half * 4 + i], b[half * 4 + j], acc[i][j], 0, 0, 0);
    }
    float sum = 0.f;
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) sum += acc[i][j][v];
    sink[blockIdx.x * blockDim.x + threadIdx.x] = sum;
}

__global__ __launch_bounds__(256) void probe_copy_kernel(const RawVec16 *__restrict__ source,
                                                         RawVec16 *__restrict__ target, int64_t vectors) {
    const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < vectors; i += stride)
        __builtin_nontemporal_store(__builtin_nontemporal_load(source + i), target + i);
}

}  // namespace fm

extern "C" int fm_probe_mfma(void *sink, int64_t workgroups, int64_t iterations, int random_operands, float sigma,
                             void *stream) {
    using namespace fm;
    FM_REQUIRE(sink && workgroups > 0 && workgroups < (1 << 20) && iterations >= 0, "fm_probe_mfma: bad argument");
    probe_mfma_kernel<<<static_cast<int>(workgroups), 256, 0, static_cast<hipStream_t>(stream)>>>(
        static_cast<float *>(sink), iterations, random_operands, sigma);
    return check_launch("fm_probe_mfma");
}

extern "C" int64_t fm_probe_mfma_flops(int64_t workgroups, int64_t iterations) {
    return workgroups * 4 * iterations * fm::kProbeMfmasPerIteration * (2LL * 32 * 32 * 16);
}

extern "C" int fm_probe_copy(const void *source, void *target, int64_t bytes, int64_t workgroups, void *stream) {
    using namespace fm;
    FM_REQUIRE(bytes >= 0 && bytes % 16 == 0 && workgroups > 0 && workgroups < (int64_t(1) << 31),
               "fm_probe_copy: bytes must be a non-negative multiple of 16");
    if (bytes == 0) return FM_OK;
    FM_REQUIRE(source && target && aligned16(source) && aligned16(target), "fm_probe_copy: null or misaligned buffer");
    probe_copy_kernel<<<static_cast<int>(workgroups), 256, 0, static_cast<hipStream_t>(stream)>>>(
        static_cast<const RawVec16 *>(source), static_cast<RawVec16 *>(target), bytes / 16);
    return check_launch("fm_probe_copy");
}
