// Top-k routing: for every token the k largest router logits, in descending order, their expert indices, and the
// softmax over just those k logits in fp32 (reference: MixtureOfExpertMLP._topk_routing,
// fast_llm/layers/decoder/mlp/mixture_of_experts.py:243-244, i.e. torch.topk followed by torch.softmax(dtype=fp32));
// and the backward of that pair with respect to the logits.
//
// One wavefront per token: lane l keeps the logits of experts l, l + 64, ... in registers (at most kMaxPerLane), and
// k rounds of a wave-wide arg-max (ties go to the lower expert index) pick the experts. Latency-bound: the whole
// input is tokens * experts values.
#include "fm_common.h"
#include "fm_router_layout.h"

namespace fm {

constexpr int kRoutingThreads = 256;  // 4 tokens per workgroup
constexpr int kMaxPerLane = 16;       // experts <= 1024
constexpr int kMaxTopK = 64;

struct Candidate {
    float value;
    int index;
};

// The larger value wins; equal values: the lower index. NaN counts as larger than every number, as in torch.topk
// (the reference's routing, fast_llm/layers/decoder/mlp/mixture_of_experts.py:243): a token with a NaN logit selects
// that expert and gets NaN scores, so a broken router shows in the loss instead of silently losing a slot.
__device__ __forceinline__ Candidate better(Candidate a, Candidate b) {
    const bool a_nan = a.value != a.value, b_nan = b.value != b.value;
    const bool same = a_nan == b_nan && (a_nan || a.value == b.value);
    const bool take_b = (b_nan && !a_nan) || (!a_nan && !b_nan && b.value > a.value) || (same && b.index < a.index);
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


// ---- the router front end: routing, auxiliary losses and shared experts in one pass ---------------------------
// Everything MixtureOfExpertMLP does between the router's logits and the sparse map (reference:
// fast_llm/layers/decoder/mlp/mixture_of_experts.py:146-171, 237-278) from one read of the logits:
//   * z-loss mean_t(logsumexp(logits_t)^2) on the logits as they come (:147-154, layers/language_model/loss/z_loss.py:88-92);
//   * jitter: the logits are multiplied by `noise` (drawn by the caller) and rounded to their type (:157-159, 234-235);
//   * top-k experts and the fp32 softmax over their logits (:243-244);
//   * the load-balancing loss sum_e mean_t(softmax(logits)[t, e]) * mean_t(selected[t, e]) (:245-254);
//   * shared experts, prepended to every token's slots with score 1 (:264-278).
// A workgroup walks a fixed range of tokens, one wavefront per token, and keeps the per-expert sums of its tokens in
// registers; the sums of all workgroups are then added in a fixed order by a second kernel, so results do not depend
// on scheduling.
constexpr int kRouterWaves = kRoutingThreads / 64;

__device__ __forceinline__ float wave_max(float value) {
#pragma unroll
    for (int offset = 32; offset > 0; offset >>= 1) value = fmaxf(value, __shfl_xor(value, offset, 64));
    return value;
}

// log(sum_e exp(values[e])) over the experts of a token (values of absent experts are -inf).
__device__ __forceinline__ float wave_logsumexp(const float (&values)[kMaxPerLane], int experts) {
    float maximum = -INFINITY;
#pragma unroll
    for (int q = 0; q < kMaxPerLane; ++q)
        if (q * 64 < experts) maximum = fmaxf(maximum, values[q]);
    maximum = wave_max(maximum);
    float sum = 0.f;
#pragma unroll
    for (int q = 0; q < kMaxPerLane; ++q)
        if (q * 64 < experts) sum += __expf(values[q] - maximum);
    return maximum + logf(wave_sum(sum));
}

// The logits of a token as the router sees them: raw, and after the jitter (rounded to T like the reference's
// `logits * noise`).
template <typename T>
__device__ __forceinline__ void load_router_row(const T *logits, const T *noise, int64_t token, int experts, int lane,
                                                float (&raw)[kMaxPerLane], float (&routed)[kMaxPerLane],
                                                float (&factor)[kMaxPerLane]) {
#pragma unroll
    for (int q = 0; q < kMaxPerLane; ++q) {
        const int e = q * 64 + lane;
        raw[q] = routed[q] = -INFINITY;
        factor[q] = 1.f;
        if (e < experts) {
            raw[q] = routed[q] = to_float(logits[token * experts + e]);
            if (noise != nullptr) {
                factor[q] = to_float(noise[token * experts + e]);
                routed[q] = to_float(from_float<T>(raw[q] * factor[q]));
            }
        }
    }
}

template <typename T>
__global__ __launch_bounds__(kRoutingThreads) void router_forward_kernel(
    const T *__restrict__ logits, const T *__restrict__ noise, int64_t *__restrict__ top_experts,
    float *__restrict__ scores, float *__restrict__ lse, float *__restrict__ partials, int64_t tokens,
    int64_t per_block, int experts, int k, int shared) {
    extern __shared__ float block_sums[];  // [waves][stats]
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int64_t begin = blockIdx.x * per_block, end = min(begin + per_block, tokens);
    const int slots = shared + k;
    float probability_sum[kMaxPerLane], count[kMaxPerLane], z_sum = 0.f;
#pragma unroll
    for (int q = 0; q < kMaxPerLane; ++q) probability_sum[q] = count[q] = 0.f;

    for (int64_t token = begin + wave; token < end; token += kRouterWaves) {
        float raw[kMaxPerLane], values[kMaxPerLane], factor[kMaxPerLane];
        load_router_row(logits, noise, token, experts, lane, raw, values, factor);
        const float lse_routed = wave_logsumexp(values, experts);
        const float lse_raw = noise != nullptr ? wave_logsumexp(raw, experts) : lse_routed;
        if (lane == 0) {
            lse[2 * token] = lse_routed;
            lse[2 * token + 1] = lse_raw;
        }
        z_sum += lse_raw * lse_raw;
#pragma unroll
        for (int q = 0; q < kMaxPerLane; ++q)
            if (q * 64 + lane < experts) probability_sum[q] += __expf(values[q] - lse_routed);

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
#pragma unroll
            for (int q = 0; q < kMaxPerLane; ++q)
                if (q * 64 + lane == best.index) {
                    values[q] = -INFINITY;
                    count[q] += 1.f;
                }
            if (j == 0) top_value = best.value;
            const float shifted = __expf(best.value - top_value);
            sum += shifted;
            if (lane == j) {
                my_value = shifted;
                top_experts[token * slots + shared + j] = best.index;
            }
        }
        if (lane < k) scores[token * slots + shared + lane] = my_value / sum;
        if (lane < shared) {
            top_experts[token * slots + lane] = experts + lane;
            scores[token * slots + lane] = 1.f;
        }
    }

    // Sums of the workgroup's tokens: the four wavefronts' registers, added in wavefront order.
    const int stats = RouterStats::size(experts);
    float *mine = block_sums + wave * stats;
#pragma unroll
    for (int q = 0; q < kMaxPerLane; ++q) {
        const int e = q * 64 + lane;
        if (e < experts) {
            mine[RouterStats::probability_sum(e)] = probability_sum[q];
            mine[RouterStats::count(experts, e)] = count[q];
        }
    }
    if (lane == 0) mine[RouterStats::z_sum(experts)] = z_sum;
    __syncthreads();
    for (int c = threadIdx.x; c < stats; c += kRoutingThreads) {
        float total = 0.f;
        for (int w = 0; w < kRouterWaves; ++w) total += block_sums[w * stats + c];
        partials[static_cast<int64_t>(blockIdx.x) * stats + c] = total;
    }
}

// statistics[c] = sum over the workgroups of the forward kernel, in workgroup order.
__global__ __launch_bounds__(kRoutingThreads) void router_reduce_kernel(const float *__restrict__ partials,
                                                                       float *__restrict__ statistics, int blocks,
                                                                       int stats) {
    const int c = blockIdx.x * kRoutingThreads + threadIdx.x;
    if (c >= stats) return;
    double total = 0.0;  // up to 1024 terms of similar size: fp32 would lose about 1e-5 of the sum
    for (int b = 0; b < blocks; ++b) total += partials[static_cast<int64_t>(b) * stats + c];
    statistics[c] = static_cast<float>(total);
}

// losses[0] = load-balancing loss, losses[1] = z-loss. One workgroup.
__global__ __launch_bounds__(kRoutingThreads) void router_losses_kernel(const float *__restrict__ statistics,
                                                                       float *__restrict__ losses, int64_t tokens,
                                                                       int experts) {
    __shared__ float wave_totals[kRouterWaves];
    float total = 0.f;
    for (int e = threadIdx.x; e < experts; e += kRoutingThreads)
        total += statistics[RouterStats::probability_sum(e)] * statistics[RouterStats::count(experts, e)];
    total = wave_sum(total);
    if ((threadIdx.x & 63) == 0) wave_totals[threadIdx.x >> 6] = total;
    __syncthreads();
    if (threadIdx.x == 0) {
        float sum = 0.f;
        for (int w = 0; w < kRouterWaves; ++w) sum += wave_totals[w];
        const float count = static_cast<float>(tokens);
        losses[0] = sum / count / count;
        losses[1] = statistics[RouterStats::z_sum(experts)] / count;
    }
}

// Gradient of the raw logits: through the top-k softmax (as topk_routing_backward_kernel), plus, scaled by the constant
// gradients the reference attaches to its auxiliary losses (functional/utils.py:63-71),
//   load balancing:  aux_scale * p[t, e] * (count[e] - sum_i p[t, i] * count[i]),  p = softmax of the routed logits
//   z-loss:          z_scale * lse_raw[t] * softmax(raw logits)[t, e]
// with aux_scale = aux_grad / tokens^2 and z_scale = 2 * z_grad / tokens; the routed part is multiplied by the jitter.
template <typename T>
__global__ __launch_bounds__(kRoutingThreads) void router_backward_kernel(
    const float *__restrict__ grad_scores, const float *__restrict__ scores, const int64_t *__restrict__ top_experts,
    const T *__restrict__ logits, const T *__restrict__ noise, const float *__restrict__ lse,
    const float *__restrict__ statistics, T *__restrict__ grad_logits, float aux_scale, float z_scale, int64_t tokens,
    int experts, int k, int shared) {
    const int lane = threadIdx.x & 63;
    const int64_t token = static_cast<int64_t>(blockIdx.x) * kRouterWaves + (threadIdx.x >> 6);
    if (token >= tokens) return;
    const int slots = shared + k;
    float raw[kMaxPerLane], routed[kMaxPerLane], factor[kMaxPerLane], grad[kMaxPerLane];
    load_router_row(logits, noise, token, experts, lane, raw, routed, factor);
    const float lse_routed = lse[2 * token], lse_raw = lse[2 * token + 1];

    // Load balancing.
    float weighted = 0.f;
#pragma unroll
    for (int q = 0; q < kMaxPerLane; ++q) {
        const int e = q * 64 + lane;
        grad[q] = 0.f;
        if (e < experts && aux_scale != 0.f) {
            const float probability = __expf(routed[q] - lse_routed);
            const float selected = statistics[RouterStats::count(experts, e)];
            grad[q] = probability * selected;  // finished below
            weighted += grad[q];
        }
    }
    if (aux_scale != 0.f) {
        weighted = wave_sum(weighted);
#pragma unroll
        for (int q = 0; q < kMaxPerLane; ++q) {
            const int e = q * 64 + lane;
            if (e < experts) grad[q] = aux_scale * (grad[q] - __expf(routed[q] - lse_routed) * weighted);
        }
    }
    // Top-k softmax.
    const float score = lane < k ? scores[token * slots + shared + lane] : 0.f;
    const float grad_score = lane < k ? grad_scores[token * slots + shared + lane] : 0.f;
    const float dot = wave_sum(score * grad_score);
    const float grad_selected = score * (grad_score - dot);
    const int expert = lane < k ? static_cast<int>(top_experts[token * slots + shared + lane]) : -1;
    for (int j = 0; j < k; ++j) {
        const int selected = __shfl(expert, j, 64);
        const float value = __shfl(grad_selected, j, 64);
#pragma unroll
        for (int q = 0; q < kMaxPerLane; ++q)
            if (q * 64 + lane == selected) grad[q] += value;
    }
    // Back through the jitter; z-loss.
#pragma unroll
    for (int q = 0; q < kMaxPerLane; ++q) {
        const int e = q * 64 + lane;
        if (e < experts) {
            float value = grad[q] * factor[q];
            if (z_scale != 0.f) value += z_scale * lse_raw * __expf(raw[q] - lse_raw);
            grad_logits[token * experts + e] = from_float<T>(value);
        }
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

extern "C" size_t fm_router_workspace_size(int64_t num_tokens, int64_t num_experts) {
    if (num_tokens <= 0 || num_experts <= 0) return 0;
    return sizeof(float) * static_cast<size_t>(router_blocks(num_tokens)) * RouterStats::size(static_cast<int>(num_experts));
}

static int check_router_shape(const char *name, int64_t num_tokens, int64_t num_experts, int64_t experts_per_token,
                              int64_t shared_experts, int dtype) {
    FM_REQUIRE(valid_dtype(dtype), "%s: bad dtype %d", name, dtype);
    FM_REQUIRE(num_tokens >= 0 && num_experts > 0 && num_experts <= 64 * kMaxPerLane, "%s: %lld experts (1..%d)", name,
               static_cast<long long>(num_experts), 64 * kMaxPerLane);
    FM_REQUIRE(experts_per_token > 0 && experts_per_token <= num_experts && shared_experts >= 0 &&
                   experts_per_token + shared_experts <= kMaxTopK,
               "%s: experts_per_token %lld, shared_experts %lld", name, static_cast<long long>(experts_per_token),
               static_cast<long long>(shared_experts));
    FM_REQUIRE((num_tokens + kRouterWaves - 1) / kRouterWaves < (int64_t(1) << 31), "%s: too many tokens", name);
    return FM_OK;
}

extern "C" int fm_router_forward(const void *logits, const void *noise, void *top_experts, void *scores, void *lse,
                                 void *statistics, void *losses, void *workspace, size_t workspace_size,
                                 int64_t num_tokens, int64_t num_experts, int64_t experts_per_token,
                                 int64_t shared_experts, int dtype, void *stream_) {
    const char *name = "fm_router_forward";
    if (int status = check_router_shape(name, num_tokens, num_experts, experts_per_token, shared_experts, dtype))
        return status;
    FM_REQUIRE(num_tokens > 0, "%s: no tokens", name);
    FM_REQUIRE(logits && top_experts && scores && lse && statistics && losses && workspace, "%s: null tensor", name);
    FM_REQUIRE(workspace_size >= fm_router_workspace_size(num_tokens, num_experts), "%s: workspace of %zu bytes, need %zu",
               name, workspace_size, fm_router_workspace_size(num_tokens, num_experts));
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    const int experts = static_cast<int>(num_experts), stats = RouterStats::size(experts);
    const int blocks = router_blocks(num_tokens);
    FM_DISPATCH_DTYPE(dtype, T, {
        router_forward_kernel<T><<<blocks, kRoutingThreads, sizeof(float) * kRouterWaves * stats, stream>>>(
            static_cast<const T *>(logits), static_cast<const T *>(noise), static_cast<int64_t *>(top_experts),
            static_cast<float *>(scores), static_cast<float *>(lse), static_cast<float *>(workspace), num_tokens,
            router_tokens_per_block(num_tokens), experts, static_cast<int>(experts_per_token),
            static_cast<int>(shared_experts));
    });
    router_reduce_kernel<<<(stats + kRoutingThreads - 1) / kRoutingThreads, kRoutingThreads, 0, stream>>>(
        static_cast<const float *>(workspace), static_cast<float *>(statistics), blocks, stats);
    router_losses_kernel<<<1, kRoutingThreads, 0, stream>>>(static_cast<const float *>(statistics),
                                                           static_cast<float *>(losses), num_tokens, experts);
    return check_launch(name);
}

extern "C" int fm_router_backward(const void *grad_scores, const void *scores, const void *top_experts,
                                  const void *logits, const void *noise, const void *lse, const void *statistics,
                                  void *grad_logits, double auxiliary_loss_grad, double z_loss_grad,
                                  int64_t num_tokens, int64_t num_experts, int64_t experts_per_token,
                                  int64_t shared_experts, int dtype, void *stream_) {
    const char *name = "fm_router_backward";
    if (int status = check_router_shape(name, num_tokens, num_experts, experts_per_token, shared_experts, dtype))
        return status;
    if (num_tokens == 0) return FM_OK;
    FM_REQUIRE(grad_scores && scores && top_experts && logits && lse && statistics && grad_logits, "%s: null tensor",
               name);
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    const double count = static_cast<double>(num_tokens);
    const float aux_scale = static_cast<float>(auxiliary_loss_grad / count / count);
    const float z_scale = static_cast<float>(2.0 * z_loss_grad / count);
    const int64_t blocks = (num_tokens + kRouterWaves - 1) / kRouterWaves;
    FM_DISPATCH_DTYPE(dtype, T, {
        router_backward_kernel<T><<<blocks, kRoutingThreads, 0, stream>>>(
            static_cast<const float *>(grad_scores), static_cast<const float *>(scores),
            static_cast<const int64_t *>(top_experts), static_cast<const T *>(logits), static_cast<const T *>(noise),
            static_cast<const float *>(lse), static_cast<const float *>(statistics), static_cast<T *>(grad_logits),
            aux_scale, z_scale, num_tokens, static_cast<int>(num_experts), static_cast<int>(experts_per_token),
            static_cast<int>(shared_experts));
    });
    return check_launch(name);
}
