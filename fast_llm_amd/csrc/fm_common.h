// Shared helpers of the gfx950 kernel library: dtype tags, error reporting, index loads, vector types.
#pragma once

#include <hip/hip_runtime.h>
#include <stdarg.h>
#include <stdint.h>
#include <stdio.h>

#include "../../include/fastmoe_hip.h"

namespace fm {

using bf16_t = __bf16;
using f16_t = _Float16;

// ---- error state (per host thread) -------------------------------------------------------------------
char *error_buffer();  // defined in fm_api.hip; 512 bytes, thread local

inline int fail(int status, const char *format, ...) {
    va_list args;
    va_start(args, format);
    vsnprintf(error_buffer(), 512, format, args);
    va_end(args);
    return status;
}

inline int check_launch(const char *what) {
    hipError_t error = hipGetLastError();
    if (error != hipSuccess) return fail(FM_ERR_LAUNCH, "%s: %s", what, hipGetErrorString(error));
    return FM_OK;
}

#define FM_REQUIRE(condition, ...) \
    do {                           \
        if (!(condition)) return ::fm::fail(FM_ERR_INVALID_ARGUMENT, __VA_ARGS__); \
    } while (0)

inline bool valid_dtype(int dtype) { return dtype == FM_DTYPE_F32 || dtype == FM_DTYPE_BF16 || dtype == FM_DTYPE_F16; }
inline bool valid_index_dtype(int dtype) { return dtype == FM_INDEX_I16 || dtype == FM_INDEX_I32 || dtype == FM_INDEX_I64; }
inline int dtype_size(int dtype) { return dtype == FM_DTYPE_F32 ? 4 : 2; }
inline bool aligned16(const void *pointer) { return (reinterpret_cast<uintptr_t>(pointer) & 15) == 0; }

// ---- device helpers ----------------------------------------------------------------------------------
template <typename T>
__device__ __forceinline__ float to_float(T value) { return static_cast<float>(value); }
template <typename T>
__device__ __forceinline__ T from_float(float value) { return static_cast<T>(value); }

// Load entry `i` of an index array whose element type is only known at run time.
__device__ __forceinline__ int64_t load_index(const void *pointer, int index_dtype, int64_t i) {
    if (index_dtype == FM_INDEX_I16) return static_cast<const int16_t *>(pointer)[i];
    if (index_dtype == FM_INDEX_I32) return static_cast<const int32_t *>(pointer)[i];
    return static_cast<const int64_t *>(pointer)[i];
}

__device__ __forceinline__ void store_index(void *pointer, int index_dtype, int64_t i, int64_t value) {
    if (index_dtype == FM_INDEX_I16) static_cast<int16_t *>(pointer)[i] = static_cast<int16_t>(value);
    else if (index_dtype == FM_INDEX_I32) static_cast<int32_t *>(pointer)[i] = static_cast<int32_t>(value);
    else static_cast<int64_t *>(pointer)[i] = value;
}

// 16-byte vector of T (4 floats or 8 half-precision values): the unit of every coalesced HBM access.
template <typename T>
struct alignas(16) Vec16 {
    static constexpr int N = 16 / sizeof(T);
    T v[N];
};

template <typename T>
__device__ __forceinline__ Vec16<T> load16(const T *pointer) {
    return *reinterpret_cast<const Vec16<T> *>(pointer);
}
template <typename T>
__device__ __forceinline__ void store16(T *pointer, const Vec16<T> &value) {
    *reinterpret_cast<Vec16<T> *>(pointer) = value;
}

// Streaming variants: the data is touched once by this kernel and is larger than the caches.
typedef __attribute__((__vector_size__(4 * sizeof(uint32_t)))) uint32_t RawVec16;
template <typename T>
__device__ __forceinline__ Vec16<T> load16_stream(const T *pointer) {
    const RawVec16 raw = __builtin_nontemporal_load(reinterpret_cast<const RawVec16 *>(pointer));
    return __builtin_bit_cast(Vec16<T>, raw);
}
template <typename T>
__device__ __forceinline__ void store16_stream(T *pointer, const Vec16<T> &value) {
    __builtin_nontemporal_store(__builtin_bit_cast(RawVec16, value), reinterpret_cast<RawVec16 *>(pointer));
}

__device__ __forceinline__ float wave_sum(float value) {
#pragma unroll
    for (int offset = 32; offset > 0; offset >>= 1) value += __shfl_xor(value, offset, 64);
    return value;
}

// Dispatch a run-time dtype tag to a template parameter.
#define FM_DISPATCH_DTYPE(dtype, T, ...)                                    \
    switch (dtype) {                                                        \
        case FM_DTYPE_F32: { using T = float; __VA_ARGS__; break; }        \
        case FM_DTYPE_BF16: { using T = ::fm::bf16_t; __VA_ARGS__; break; } \
        default: { using T = ::fm::f16_t; __VA_ARGS__; break; }             \
    }

}  // namespace fm
