// MoE routing: stable sort of the flat (token, route) list by expert.  Produces both directions of
// the permutation and the tokens per expert, which is what the gather + dynamic quantisation
// (dyn_quant.hip), the grouped matmul (group sizes) and the un-permute (unpermute.hip) consume.
//
// Follows the sort stage of moe_init_routing_quant_v2
// (examples/aux_ops/moe_init_routing_quant_v2/moe_init_routing_quant_v2.h:70-110: sort by expert,
// MoeV2SrcToDstOp inverts the permutation, MoeV2ExpertTokenOut counts) and its CPU stand-in
// (examples/utils/gen_data_moe.py:48-57: torch.argsort(stable=True) + bincount).  Keys are small
// integers, so the sort is a counting sort in three launches: per-chunk histograms, one scan over
// (expert, chunk), and a placement pass in which one wave walks its chunk in order.
#include <algorithm>

#include "common.h"

namespace cch {

constexpr int ROUTE_CHUNK = 1024;       // rows per workgroup
constexpr int ROUTE_MAX_EXPERTS = 1024;

// hist[e * nchunks + c] = rows of chunk c routed to expert e; dst_to_src of the chunk's positions
// is preset to -1 (positions past the routed rows keep it).
__global__ __launch_bounds__(256) void route_histogram_kernel(const int32_t *__restrict__ expert_idx, int rows, int experts,
                                                              int nchunks, int32_t *__restrict__ hist,
                                                              int32_t *__restrict__ dst_to_src)
{
    __shared__ int32_t h[ROUTE_MAX_EXPERTS];
    for (int e = threadIdx.x; e < experts; e += 256) h[e] = 0;
    __syncthreads();
    const int base = blockIdx.x * ROUTE_CHUNK;
    for (int i = threadIdx.x; i < ROUTE_CHUNK; i += 256) {
        const int r = base + i;
        if (r < rows) {
            const int e = expert_idx[r];
            if (e >= 0 && e < experts) atomicAdd(&h[e], 1);
            dst_to_src[r] = -1;
        }
    }
    __syncthreads();
    for (int e = threadIdx.x; e < experts; e += 256) hist[(size_t)e * nchunks + blockIdx.x] = h[e];
}

// In-place exclusive scan of hist in (expert, chunk) order: hist[e * nchunks + c] becomes the first
// sorted position of expert e's rows of chunk c.  One workgroup; also writes the per-expert token
// counts (or their running sum).
__global__ __launch_bounds__(1024) void route_scan_kernel(int32_t *__restrict__ hist, int experts, int nchunks,
                                                          int32_t *__restrict__ expert_tokens, int cumsum)
{
    __shared__ int32_t part[1024];
    __shared__ int32_t carry;
    const int n = experts * nchunks;
    if (threadIdx.x == 0) carry = 0;
    __syncthreads();
    for (int base = 0; base < n; base += 1024) {
        const int i = base + threadIdx.x;
        const int v = i < n ? hist[i] : 0;
        part[threadIdx.x] = v;
        __syncthreads();
        // Hillis-Steele inclusive scan over the 1024 entries
        for (int off = 1; off < 1024; off <<= 1) {
            const int add = threadIdx.x >= off ? part[threadIdx.x - off] : 0;
            __syncthreads();
            part[threadIdx.x] += add;
            __syncthreads();
        }
        const int incl = part[threadIdx.x], c0 = carry;
        if (i < n) hist[i] = c0 + incl - v;
        __syncthreads();
        if (threadIdx.x == 1023) carry = c0 + incl;
        __syncthreads();
    }
    // tokens per expert from the scanned starts
    const int total = carry;
    for (int e = threadIdx.x; e < experts; e += 1024) {
        const int start = hist[(size_t)e * nchunks];
        const int end = e + 1 < experts ? hist[(size_t)(e + 1) * nchunks] : total;
        expert_tokens[e] = cumsum ? end : end - start;
    }
}

// One wave per chunk walks its rows in order, 64 at a time.  Inside a group of 64 the rank of a
// row among the rows of the same expert comes from a ballot per distinct expert value; the
// running position of every expert lives in LDS.
__global__ __launch_bounds__(64) void route_place_kernel(const int32_t *__restrict__ expert_idx, int rows, int experts, int nchunks,
                                                         const int32_t *__restrict__ starts, int32_t *__restrict__ dst_to_src,
                                                         int32_t *__restrict__ src_to_dst)
{
    __shared__ int32_t next[ROUTE_MAX_EXPERTS];
    const int lane = threadIdx.x;
    for (int e = lane; e < experts; e += 64) next[e] = starts[(size_t)e * nchunks + blockIdx.x];
    __syncthreads();
    const int base = blockIdx.x * ROUTE_CHUNK;
    for (int i = 0; i < ROUTE_CHUNK; i += 64) {
        const int r = base + i + lane;
        const int e = r < rows ? expert_idx[r] : -1;
        const bool routed = e >= 0 && e < experts;
        int pos = -1;
        uint64_t remaining = __ballot(routed);
        while (remaining) {   // wave-uniform: one round per distinct expert among the 64 rows
            const int leader = __ffsll((long long)remaining) - 1;
            const int v = __builtin_amdgcn_readlane(e, leader);
            const uint64_t same = __ballot(routed && e == v);
            const int first = next[v];
            if (routed && e == v) pos = first + __popcll(same & ((1ull << lane) - 1ull));
            __syncthreads();   // every lane has read next[v] before the leader moves it on
            if (lane == leader) next[v] = first + __popcll(same);
            __syncthreads();
            remaining &= ~same;
        }
        if (r < rows) {
            src_to_dst[r] = pos;
            if (pos >= 0) dst_to_src[pos] = r;
        }
    }
}

}  // namespace cch

extern "C" int64_t cch_moe_init_routing_workspace_bytes(int64_t rows, int num_experts)
{
    if (rows < 0 || num_experts < 1) return 0;
    const int64_t nchunks = (rows + cch::ROUTE_CHUNK - 1) / cch::ROUTE_CHUNK;
    return std::max<int64_t>(nchunks, 1) * num_experts * (int64_t)sizeof(int32_t);
}

extern "C" int cch_moe_init_routing(const int32_t *expert_idx, int64_t rows, int num_experts, int32_t *dst_to_src,
                                    int32_t *src_to_dst, int32_t *expert_tokens, int cumsum, void *workspace,
                                    int64_t workspace_bytes, void *stream)
{
    using namespace cch;
    CCH_REQUIRE(rows >= 0 && rows < ((int64_t)1 << 30), "cch_moe_init_routing: rows=%lld", (long long)rows);
    CCH_REQUIRE(num_experts >= 1 && num_experts <= ROUTE_MAX_EXPERTS, "cch_moe_init_routing: num_experts=%d outside 1..%d",
                num_experts, ROUTE_MAX_EXPERTS);
    CCH_REQUIRE(expert_tokens != nullptr, "cch_moe_init_routing: null expert_tokens");
    hipStream_t s = static_cast<hipStream_t>(stream);
    const int64_t nchunks = std::max<int64_t>((rows + ROUTE_CHUNK - 1) / ROUTE_CHUNK, 1);
    CCH_REQUIRE(nchunks * num_experts < ((int64_t)1 << 31), "cch_moe_init_routing: rows x experts too large");
    CCH_REQUIRE(workspace != nullptr && workspace_bytes >= cch_moe_init_routing_workspace_bytes(rows, num_experts),
                "cch_moe_init_routing: workspace of %lld bytes, need %lld", (long long)workspace_bytes,
                (long long)cch_moe_init_routing_workspace_bytes(rows, num_experts));
    CCH_REQUIRE(rows == 0 || (expert_idx && dst_to_src && src_to_dst), "cch_moe_init_routing: null pointer");
    int32_t *hist = static_cast<int32_t *>(workspace);
    hipLaunchKernelGGL(route_histogram_kernel, dim3((unsigned)nchunks), dim3(256), 0, s, expert_idx, (int)rows, num_experts,
                       (int)nchunks, hist, dst_to_src);
    hipLaunchKernelGGL(route_scan_kernel, dim3(1), dim3(1024), 0, s, hist, num_experts, (int)nchunks, expert_tokens, cumsum);
    if (rows > 0)
        hipLaunchKernelGGL(route_place_kernel, dim3((unsigned)nchunks), dim3(64), 0, s, expert_idx, (int)rows, num_experts,
                           (int)nchunks, hist, dst_to_src, src_to_dst);
    return launch_status("route kernels");
}
