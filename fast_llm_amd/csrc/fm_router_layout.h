// What the router's forward kernel leaves in its workspace, shared with the sparse-map kernels that consume it.
#pragma once

#include <stdint.h>

namespace fm {

// Per workgroup of the router's forward kernel: 2 * experts + 1 floats.
struct RouterStats {
    static __host__ __device__ int probability_sum(int e) { return e; }
    static __host__ __device__ int count(int experts, int e) { return experts + e; }
    static __host__ __device__ int z_sum(int experts) { return 2 * experts; }
    static __host__ __device__ int size(int experts) { return 2 * experts + 1; }
};

constexpr int kMaxRouterBlocks = 1024;
constexpr int kRouterTokensPerBlock = 16;

// Workgroups of the router's forward kernel; workgroup b handles the tokens
// [b * router_tokens_per_block, (b + 1) * router_tokens_per_block).
inline int router_blocks(int64_t tokens) {
    const int64_t blocks = (tokens + kRouterTokensPerBlock - 1) / kRouterTokensPerBlock;
    return static_cast<int>(blocks < kMaxRouterBlocks ? blocks : kMaxRouterBlocks);
}
inline int64_t router_tokens_per_block(int64_t tokens) {
    const int blocks = router_blocks(tokens);
    return blocks > 0 ? (tokens + blocks - 1) / blocks : 0;
}

}  // namespace fm
