// Top-k routing: for every token the k largest router logits, in descending order, their expert indices, and the
// softmax over just those k logits in fp32 (reference: MixtureOfExpertMLP._topk_routing,
// fast_llm/layers/decoder/mlp/mixture_of_experts.py:243-244, i.e. torch.topk followed by torch.softmax(dtype=fp32));
// and the backward of that pair with respect to the logits.
//
// One wavefront per token: lane l keeps the logits of experts l, l + 64, ... in registers (at most kMaxPerLane), and
// k rounds of a wave-wide arg-max (ties go to the lower expert index) pick the experts. Latency-bound: the whole
// input is tokens * experts values.
#include "fm_common.h"

namespace fm {

constexpr int kRoutingThreads = 256;  // 4 tokens per workgroup
constexpr int kMaxPerLane = 16;       // experts <= 1024
constexpr int kMaxTopK = 64;

struct Candidate {
    float value;
    int index;
};

// The larger value wins; equal values: the lower index. NaN never wins against a number.
__device__ __forceinline__ Candidate better(Candidate a, Candidate b) {
    const bool take_b = b.value > a.value || (b.value == a.value && b.index < a.index) || (a.value != a.value && b.value == b.value);
    return take_b ? b : a;
}

template <typename T>
__global__ __launch_bounds__(kRoutingThreads) void topk_routing_kernel(const T *__restrict__ logits,
                                                                      int64_t *__restrict__ top_experts,
                                                                      float *__restrict__ scores, int64_t tokens,
                                                                      int experts, int k) {
    const int lane = threadIdx.x & 63;
    const int64_t token = static_cast<int64_t>(blockIdx.x) * (kRoutingThreads / 64) + (threadIdx.x >> 6);
    if (token >= tokens) return;
    const T *row = logits + token * experts;
    float values[kMaxPerLane];
#pragma unroll
    for (int q = 0; q < kMaxPerLane; ++q) {
        const int e = q * 64 + lane;
        values[q] = e < experts ? to_float(row[e]) : -INFINITY;
    }
    float top_value = 0.f, sum = 0.f, my_value = 0.f;
    for (int j = 0; j < k; ++j) {
        Candidate best{-INFINITY, 0x7fffffff};
#pragma unroll
        for (int q = 0; q < kMaxPerLane; ++q) {
            const int e = q * 64 + lane;
            if (e < experts) best = better(best, Candidate{values[q], e});
        }
#pragma unroll
        for (int offset = 32; offset > 0; offset >>= 1) {
            Candidate other{__shfl_xor(best.value, offset, 64), __shfl_xor(best.index, offset, 64)};
            best = better(best, other);
        }
        // Every lane now holds the winner; its owner retires it.
#pragma unroll
        for (int q = 0; q < kMaxPerLane; ++q)
            if (q * 64 + lane == best.index) values[q] = -INFINITY;
        if (j == 0) top_value = best.value;
        const float shifted = __expf(best.value - top_value);
        sum += shifted;
        if (lane == j) {  // lane j keeps slot j (k <= 64)
            my_value = shifted;
            top_experts[token * k + j] = best.index;
        }
    }
    if (lane < k) scores[token * k + lane] = my_value / sum;
}

// grad_logits[t, e] = scores[t, j] * (grad_scores[t, j] - sum_i scores[t, i] * grad_scores[t, i]) where e is the j-th
// selected expert of token t, and 0 for every expert that was not selected.
template <typename T>
__global__ __launch_bounds__(kRoutingThreads) void topk_routing_backward_kernel(
    const float *__restrict__ grad_scores, const float *__restrict__ scores, const int64_t *__restrict__ top_experts,
    T *__restrict__ grad_logits, int64_t tokens, int experts, int k) {
    const int lane = threadIdx.x & 63;
    const int64_t token = static_cast<int64_t>(blockIdx.x) * (kRoutingThreads / 64) + (threadIdx.x >> 6);
    if (token >= tokens) return;
    const float score = lane < k ? scores[token * k + lane] : 0.f;
    const float grad = lane < k ? grad_scores[token * k + lane] : 0.f;
    const float dot = wave_sum(score * grad);
    const float grad_logit = score * (grad - dot);
    const int expert = lane < k ? static_cast<int>(top_experts[token * k + lane]) : -1;
    T *row = grad_logits + token * experts;
    // Every element of the row is written once, by the lane that owns it: the value of the slot that selected it, or 0.
    for (int base = 0; base < experts; base += 64) {
        const int e = base + lane;
        float value = 0.f;
        for (int j = 0; j < k; ++j) {
            const int selected = __shfl(expert, j, 64);
            const float selected_grad = __shfl(grad_logit, j, 64);
            if (selected == e) value = selected_grad;
        }
        if (e < experts) row[e] = from_float<T>(value);
    }
}

}  // namespace fm

using namespace fm;

extern "C" int fm_topk_routing(const void *logits, void *top_experts, void *scores, int64_t num_tokens,
                               int64_t num_experts, int64_t experts_per_token, int dtype, void *stream_) {
    const char *name = "fm_topk_routing";
    FM_REQUIRE(valid_dtype(dtype), "%s: bad dtype %d", name, dtype);
    FM_REQUIRE(num_tokens >= 0 && num_experts > 0 && num_experts <= 64 * kMaxPerLane, "%s: %lld experts (1..%d)", name,
               static_cast<long long>(num_experts), 64 * kMaxPerLane);
    FM_REQUIRE(experts_per_token > 0 && experts_per_token <= num_experts && experts_per_token <= kMaxTopK,
               "%s: experts_per_token %lld", name, static_cast<long long>(experts_per_token));
    if (num_tokens == 0) return FM_OK;
    FM_REQUIRE(logits && top_experts && scores, "%s: null tensor", name);
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    const int64_t blocks = (num_tokens + kRoutingThreads / 64 - 1) / (kRoutingThreads / 64);
    FM_REQUIRE(blocks < (int64_t(1) << 31), "%s: too many tokens", name);
    FM_DISPATCH_DTYPE(dtype, T, {
        topk_routing_kernel<T><<<blocks, kRoutingThreads, 0, stream>>>(
            static_cast<const T *>(logits), static_cast<int64_t *>(top_experts), static_cast<float *>(scores),
            num_tokens, static_cast<int>(num_experts), static_cast<int>(experts_per_token));
    });
    return check_launch(name);
}

extern "C" int fm_topk_routing_backward(const void *grad_scores, const void *scores, const void *top_experts,
                                        void *grad_logits, int64_t num_tokens, int64_t num_experts,
                                        int64_t experts_per_token, int dtype, void *stream_) {
    const char *name = "fm_topk_routing_backward";
    FM_REQUIRE(valid_dtype(dtype), "%s: bad dtype %d", name, dtype);
    FM_REQUIRE(num_tokens >= 0 && num_experts > 0, "%s: bad shape", name);
    FM_REQUIRE(experts_per_token > 0 && experts_per_token <= num_experts && experts_per_token <= kMaxTopK,
               "%s: experts_per_token %lld", name, static_cast<long long>(experts_per_token));
    if (num_tokens == 0) return FM_OK;
    FM_REQUIRE(grad_scores && scores && top_experts && grad_logits, "%s: null tensor", name);
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    const int64_t blocks = (num_tokens + kRoutingThreads / 64 - 1) / (kRoutingThreads / 64);
    FM_REQUIRE(blocks < (int64_t(1) << 31), "%s: too many tokens", name);
    FM_DISPATCH_DTYPE(dtype, T, {
        topk_routing_backward_kernel<T><<<blocks, kRoutingThreads, 0, stream>>>(
            static_cast<const float *>(grad_scores), static_cast<const float *>(scores),
            static_cast<const int64_t *>(top_experts), static_cast<T *>(grad_logits), num_tokens,
            static_cast<int>(num_experts), static_cast<int>(experts_per_token));
    });
    return check_launch(name);
}
