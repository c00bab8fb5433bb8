// Measurement probes of bench.py, built into their own small library (libbench_probes.so, beside this file): what the
// matrix cores, the HBM and the L2 of the device at hand sustain, so that kernel figures can be set against a measured
// ceiling next to the published peak. Not part of the kernel library and not on the MoE path. Every entry point
// returns 0, -1 for a bad argument or -3 when the runtime rejected the launch.
//   probe_mfma: a register-only loop of back-to-back v_mfma_f32_32x32x16_bf16 (the instruction of the grouped
//     products), 4 x 4 accumulators per wavefront fed from 8 + 8 operand fragments that hold zeros or normal(0, sigma)
//     bf16 values. The chip lowers its clock under power, and operand toggling costs power: the rate on random data
//     is the ceiling a product on real activations can reach, the rate on zeros is the published peak.
//   probe_copy: a plain streaming copy (16-byte vectors, one read and one write per byte).
//   probe_l2: every workgroup streams a small region that stays in its XCD's L2 straight into LDS, 64 KiB per
//     iteration (what a 256 x 256 x 64 bf16 GEMM slice needs), with the GEMM's load instruction. A workgroup tile of
//     256 x 256 needs 1/128 byte per FLOP from L2, i.e. 32 bytes per cycle and CU at the matrix peak of 4096
//     FLOP/cycle/CU: the rate measured here says how far below the matrix peak the L2 caps such a product.
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace {

typedef __attribute__((__vector_size__(4 * sizeof(uint32_t)))) uint32_t RawVec16;
constexpr int kOk = 0, kBadArgument = -1, kLaunchFailed = -3;
inline bool aligned16(const void *pointer) { return (reinterpret_cast<uintptr_t>(pointer) & 15) == 0; }
inline int launched() { return hipGetLastError() == hipSuccess ? kOk : kLaunchFailed; }


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

__global__ __launch_bounds__(256, 1) void probe_mfma_kernel(float *sink, int64_t *cycles, int64_t iterations,
                                                            int random_operands, float sigma) {
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
    const int64_t start = clock64();
    for (int64_t iteration = 0; iteration < iterations; ++iteration) {
#pragma unroll
        for (int half = 0; half < 2; ++half)
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[half * 4 + i], b[half * 4 + j], acc[i][j], 0, 0, 0);
    }
    // Shader clock cycles of the loop (the counter runs at the shader clock): cycles / elapsed time is the clock the
    // device held under this load.
    if (cycles != nullptr && threadIdx.x == 0) cycles[blockIdx.x] = clock64() - start;
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

// One workgroup per CU (the dynamic LDS leaves room for one). Workgroups b, b + 8, b + 16, ... run on the same XCD;
// groups of `shared_by` of them stream the same region of `region_bytes`, 64 KiB per iteration, wrapping around.
// kInFlight: iterations a wavefront may have on their way besides the one it is issuing (16 loads each).
template <int kInFlight>
__global__ __launch_bounds__(256, 1) void probe_l2_kernel(const char *base, int64_t region_bytes, int shared_by,
                                                          int64_t iterations, int64_t *cycles) {
    extern __shared__ __attribute__((aligned(1024))) char probe_lds_generic[];
    __attribute__((address_space(3))) char *lds = (__attribute__((address_space(3))) char *)(probe_lds_generic);
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int xcd = blockIdx.x % 8, local = blockIdx.x / 8;
    const int groups_per_xcd = (gridDim.x / 8 + shared_by - 1) / shared_by;
    const char *region = base + static_cast<int64_t>(xcd * groups_per_xcd + local / shared_by) * region_bytes;
    // Members of a group start at different offsets so that they do not walk in lock step.
    const uint32_t mask = static_cast<uint32_t>(region_bytes - 1);  // region_bytes is a power of two
    uint32_t offset = static_cast<uint32_t>(local % shared_by) * 65536u & mask;
    __syncthreads();
    const int64_t start = clock64();
    for (int64_t iteration = 0; iteration < iterations; ++iteration) {
#pragma unroll
        for (int j = 0; j < 16; ++j) {
            const char *pointer = region + (((offset + (wave * 16 + j) * 1024u) & mask) + lane * 16);
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)pointer,
                                             (__attribute__((address_space(3))) void *)(lds + (iteration & 1) * 65536 +
                                                                                        (wave * 16 + j) * 1024),
                                             16, 0, 0);
        }
        offset = (offset + 65536u) & mask;
        asm volatile("s_waitcnt vmcnt(%0)" ::"n"(16 * kInFlight) : "memory");
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (threadIdx.x == 0) cycles[blockIdx.x] = clock64() - start;
}

}  // namespace

// `workgroups` workgroups (a multiple of 8, one per CU) of 4 wavefronts each stream 64 KiB per iteration from global
// memory straight into LDS with 16-byte loads, `iterations` times. Workgroups on one XCD form groups of `shared_by`
// that read the same region of `region_bytes` (a power of two, 64 KiB or more) over and over, so a small region stays
// in that XCD's L2. A wavefront keeps up to `in_flight` (1 to 3) iterations of 16 loads on their way while it issues
// the next. `source` holds (workgroups / 8 / shared_by rounded up) * 8 regions; `cycles` receives one int64 per
// workgroup: the shader clock cycles its loop took.
extern "C" int probe_l2(const void *source, int64_t region_bytes, int64_t shared_by, int64_t workgroups,
                        int64_t iterations, int64_t in_flight, void *cycles, void *stream) {
    if (!(source && cycles && aligned16(source))) return kBadArgument;
    if (!(region_bytes >= 65536 && region_bytes <= (int64_t(1) << 30) && (region_bytes & (region_bytes - 1)) == 0 &&
          shared_by > 0 && workgroups > 0 && workgroups % 8 == 0 && workgroups < (1 << 20) && iterations >= 0 &&
          in_flight >= 1 && in_flight <= 3))
        return kBadArgument;
    constexpr int kLdsBytes = 2 * 65536;
    auto kernel = in_flight == 1 ? probe_l2_kernel<1> : in_flight == 2 ? probe_l2_kernel<2> : probe_l2_kernel<3>;
    if (hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                            kLdsBytes) != hipSuccess)
        return kLaunchFailed;
    kernel<<<static_cast<int>(workgroups), 256, kLdsBytes, static_cast<hipStream_t>(stream)>>>(
        static_cast<const char *>(source), region_bytes, static_cast<int>(shared_by), iterations,
        static_cast<int64_t *>(cycles));
    return launched();
}

// `workgroups` workgroups of 4 wavefronts each issue `iterations` x 32 back-to-back v_mfma_f32_32x32x16_bf16 from
// registers; operands are zeros (random_operands = 0) or normal(0, sigma) values. `sink` receives 256 floats per
// workgroup, `cycles` (may be null) one int64 per workgroup: the shader clock cycles of its loop. The work done is
// probe_mfma_flops(workgroups, iterations).
extern "C" int probe_mfma(void *sink, void *cycles, int64_t workgroups, int64_t iterations, int random_operands,
                          float sigma, void *stream) {
    if (!(sink && workgroups > 0 && workgroups < (1 << 20) && iterations >= 0)) return kBadArgument;
    probe_mfma_kernel<<<static_cast<int>(workgroups), 256, 0, static_cast<hipStream_t>(stream)>>>(
        static_cast<float *>(sink), static_cast<int64_t *>(cycles), iterations, random_operands, sigma);
    return launched();
}

extern "C" int64_t probe_mfma_flops(int64_t workgroups, int64_t iterations) {
    return workgroups * 4 * iterations * kProbeMfmasPerIteration * (2LL * 32 * 32 * 16);
}

// target[0 .. bytes) = source[0 .. bytes) with 16-byte streaming loads and stores from `workgroups` workgroups of 256
// lanes (grid stride). `bytes` a multiple of 16, both pointers 16-byte aligned.
extern "C" int probe_copy(const void *source, void *target, int64_t bytes, int64_t workgroups, void *stream) {
    if (!(bytes >= 0 && bytes % 16 == 0 && workgroups > 0 && workgroups < (int64_t(1) << 31))) return kBadArgument;
    if (bytes == 0) return kOk;
    if (!(source && target && aligned16(source) && aligned16(target))) return kBadArgument;
    probe_copy_kernel<<<static_cast<int>(workgroups), 256, 0, static_cast<hipStream_t>(stream)>>>(
        static_cast<const RawVec16 *>(source), static_cast<RawVec16 *>(target), bytes / 16);
    return launched();
}
