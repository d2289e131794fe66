// MoE routing: stable sort of the flat (token, route) list by expert.  Produces both directions of
// the permutation and the tokens per expert, which is what the gather + dynamic quantisation
// (dyn_quant.hip), the grouped matmul (group sizes) and the un-permute (unpermute.hip) consume.
//
// Follows the sort stage of moe_init_routing_quant_v2
// (examples/aux_ops/moe_init_routing_quant_v2/moe_init_routing_quant_v2.h:70-110: sort by expert,
// MoeV2SrcToDstOp inverts the permutation, MoeV2ExpertTokenOut counts) and its CPU stand-in
// (examples/utils/gen_data_moe.py:48-57: torch.argsort(stable=True) + bincount).  Keys are small
// integers, so the sort is a counting sort in three launches: per-chunk histograms, one scan over
// (expert, chunk), and a placement pass in which four waves walk their quarters of a chunk in order.
#include <algorithm>
#include <atomic>

#include "common.h"

namespace cch {

constexpr int ROUTE_CHUNK = 1024;       // rows per workgroup
constexpr int ROUTE_MAX_EXPERTS = 1024;
// cch_set_option("routing_three_launches", 1): the general path also where one workgroup would do (for tests)
std::atomic<int> g_route_three_launches{0};

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
// sorted position of expert e's rows of chunk c.  One workgroup of 16 waves: a wave sums the
// (contiguous) row of an expert, the per-expert totals are scanned across the workgroup, and the
// wave then scans its rows 64 chunks at a time from the expert's start.  Also writes the
// per-expert token counts (or their running sum).
__global__ __launch_bounds__(1024) void route_scan_kernel(int32_t *__restrict__ hist, int experts, int nchunks,
                                                          int32_t *__restrict__ expert_tokens, int cumsum)
{
    __shared__ int32_t part[1024];   // per-expert totals, then their inclusive scan (experts <= 1024)
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    part[threadIdx.x] = 0;
    __syncthreads();
    for (int e = wave; e < experts; e += 16) {
        int sum = 0;
        for (int c = lane; c < nchunks; c += 64) sum += hist[(size_t)e * nchunks + c];
#pragma unroll
        for (int off = 32; off >= 1; off >>= 1) sum += __shfl_xor(sum, off, 64);
        if (lane == 0) part[e] = sum;
    }
    __syncthreads();
    const int own = part[threadIdx.x];
    // Hillis-Steele inclusive scan over the 1024 totals
    for (int off = 1; off < 1024; off <<= 1) {
        const int add = threadIdx.x >= off ? part[threadIdx.x - off] : 0;
        __syncthreads();
        part[threadIdx.x] += add;
        __syncthreads();
    }
    if ((int)threadIdx.x < experts) expert_tokens[threadIdx.x] = cumsum ? part[threadIdx.x] : own;
    for (int e = wave; e < experts; e += 16) {
        int run = e > 0 ? part[e - 1] : 0;   // first position of expert e
        for (int c0 = 0; c0 < nchunks; c0 += 64) {
            const int c = c0 + lane;
            const int v = c < nchunks ? hist[(size_t)e * nchunks + c] : 0;
            int incl = v;
#pragma unroll
            for (int off = 1; off < 64; off <<= 1) {
                const int up = __shfl_up(incl, off, 64);
                if (lane >= off) incl += up;
            }
            if (c < nchunks) hist[(size_t)e * nchunks + c] = run + incl - v;
            run += __shfl(incl, 63, 64);
        }
    }
}

// Lanes of the wave that hold the same key as this lane (keys below 2^bits; lanes with
// routed == false match nobody): one ballot per key bit.
__device__ __forceinline__ uint64_t same_key_lanes(int key, bool routed, int bits)
{
    uint64_t m = __ballot(routed);
    for (int b = 0; b < bits; b++) {
        const uint64_t set = __ballot(routed && ((key >> b) & 1));
        m &= ((key >> b) & 1) ? set : ~set;
    }
    return routed ? m : 0;
}

// Four waves per chunk, 256 consecutive rows each, 64 at a time.  Inside a group of 64 the rank
// of a row among the rows of the same expert is a population count over the lanes that hold the
// same key; a wave first counts its rows per expert, the counts of the waves before it (and the
// chunk's scanned start) give its first position per expert, and a second walk over the same
// rows hands the positions out in order.  A wave's LDS accesses execute in program order, so
// "all lanes read the counter, then the first lane of each key moves it on" needs no barrier.
constexpr int ROUTE_WAVES = 4;
constexpr int ROUTE_GROUPS = ROUTE_CHUNK / 64 / ROUTE_WAVES;   // groups of 64 rows per wave
__global__ __launch_bounds__(64 * ROUTE_WAVES) void route_place_kernel(const int32_t *__restrict__ expert_idx, int rows, int experts,
                                                                      int nchunks, int bits, const int32_t *__restrict__ starts,
                                                                      int32_t *__restrict__ dst_to_src,
                                                                      int32_t *__restrict__ src_to_dst)
{
    __shared__ int32_t cnt[ROUTE_WAVES][ROUTE_MAX_EXPERTS];
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    for (int e = threadIdx.x; e < experts; e += 64 * ROUTE_WAVES) {
#pragma unroll
        for (int v = 0; v < ROUTE_WAVES; v++) cnt[v][e] = 0;
    }
    __syncthreads();
    const int base = blockIdx.x * ROUTE_CHUNK + w * (ROUTE_GROUPS * 64);
    const uint64_t below = (1ull << lane) - 1ull;
    int key[ROUTE_GROUPS];
    uint64_t same[ROUTE_GROUPS];
#pragma unroll
    for (int g = 0; g < ROUTE_GROUPS; g++) {
        const int r = base + g * 64 + lane;
        const int e = r < rows ? expert_idx[r] : -1;
        const bool routed = e >= 0 && e < experts;
        key[g] = routed ? e : -1;
        same[g] = same_key_lanes(e, routed, bits);
        if (routed && (same[g] & below) == 0) cnt[w][e] += __popcll(same[g]);   // first lane of its key
    }
    __syncthreads();
    // counts -> first positions: the chunk's start per expert, then the waves in order
    for (int e = threadIdx.x; e < experts; e += 64 * ROUTE_WAVES) {
        int run = starts[(size_t)e * nchunks + blockIdx.x];
#pragma unroll
        for (int v = 0; v < ROUTE_WAVES; v++) {
            const int c = cnt[v][e];
            cnt[v][e] = run;
            run += c;
        }
    }
    __syncthreads();
#pragma unroll
    for (int g = 0; g < ROUTE_GROUPS; g++) {
        const int r = base + g * 64 + lane;
        const bool routed = key[g] >= 0;
        int pos = -1;
        if (routed) pos = cnt[w][key[g]] + __popcll(same[g] & below);
        if (routed && (same[g] & below) == 0) cnt[w][key[g]] += __popcll(same[g]);
        if (r < rows) {
            src_to_dst[r] = pos;
            if (pos >= 0) dst_to_src[pos] = r;
        }
    }
}

// Few rows and experts (a decode step's routes): the whole sort in one workgroup and one launch.  Sixteen waves
// walk their sixteenths of the rows in order, 64 at a time, exactly like the waves of the placement pass above;
// the per-wave counts per expert meet in LDS, thread e scans expert e's counts over the waves, the experts'
// totals are scanned across the workgroup, and a second walk over the rows (keys and lane sets kept in registers)
// hands the positions out.  No workspace.
constexpr int ONE_WAVES = 16, ONE_MAX_GROUPS = 8, ONE_MAX_EXPERTS = 256;
constexpr int ONE_MAX_ROWS = ONE_WAVES * ONE_MAX_GROUPS * 64;   // 8192
__global__ __launch_bounds__(64 * ONE_WAVES) void route_one_workgroup_kernel(const int32_t *__restrict__ expert_idx, int rows, int experts,
                                                                            int bits, int groups, int32_t *__restrict__ dst_to_src,
                                                                            int32_t *__restrict__ src_to_dst,
                                                                            int32_t *__restrict__ expert_tokens, int cumsum)
{
    __shared__ int32_t cnt[ONE_WAVES][ONE_MAX_EXPERTS];
    __shared__ int32_t part[ONE_MAX_EXPERTS];
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    for (int e = threadIdx.x; e < ONE_WAVES * ONE_MAX_EXPERTS; e += 64 * ONE_WAVES) (&cnt[0][0])[e] = 0;
    __syncthreads();
    const int base = w * groups * 64;   // `groups` groups of 64 rows per wave
    const uint64_t below = (1ull << lane) - 1ull;
    int key[ONE_MAX_GROUPS];
    uint64_t same[ONE_MAX_GROUPS];
#pragma unroll
    for (int g = 0; g < ONE_MAX_GROUPS; g++) {
        key[g] = -1;
        same[g] = 0;
        if (g < groups) {
            const int r = base + g * 64 + lane;
            const int e = r < rows ? expert_idx[r] : -1;
            const bool routed = e >= 0 && e < experts;
            key[g] = routed ? e : -1;
            same[g] = same_key_lanes(e, routed, bits);
            if (routed && (same[g] & below) == 0) cnt[w][e] += __popcll(same[g]);   // first lane of its key
        }
    }
    __syncthreads();
    // thread e: expert e's counts over the waves -> exclusive running sums, total into part[e]
    int total = 0;
    if ((int)threadIdx.x < ONE_MAX_EXPERTS) {
        const int e = threadIdx.x;
#pragma unroll
        for (int v = 0; v < ONE_WAVES; v++) {
            const int c = cnt[v][e];
            cnt[v][e] = total;
            total += c;
        }
        part[e] = total;
    }
    __syncthreads();
    // inclusive scan of the experts' totals (Hillis-Steele over 256 entries)
    for (int off = 1; off < ONE_MAX_EXPERTS; off <<= 1) {
        int add = 0;
        if ((int)threadIdx.x < ONE_MAX_EXPERTS && (int)threadIdx.x >= off) add = part[threadIdx.x - off];
        __syncthreads();
        if ((int)threadIdx.x < ONE_MAX_EXPERTS) part[threadIdx.x] += add;
        __syncthreads();
    }
    if ((int)threadIdx.x < experts) expert_tokens[threadIdx.x] = cumsum ? part[threadIdx.x] : total;
    const int routed_rows = part[ONE_MAX_EXPERTS - 1];
    // sorted positions past the routed rows hold no row
    for (int i = routed_rows + (int)threadIdx.x; i < rows; i += 64 * ONE_WAVES) dst_to_src[i] = -1;
#pragma unroll
    for (int g = 0; g < ONE_MAX_GROUPS; g++) {
        if (g < groups) {
            const int r = base + g * 64 + lane;
            const bool routed = key[g] >= 0;
            int pos = -1;
            if (routed) pos = (key[g] > 0 ? part[key[g] - 1] : 0) + cnt[w][key[g]] + __popcll(same[g] & below);
            if (routed && (same[g] & below) == 0) cnt[w][key[g]] += __popcll(same[g]);
            if (r < rows) {
                src_to_dst[r] = pos;
                if (pos >= 0) dst_to_src[pos] = r;
            }
        }
    }
}

// Checks shared by the two entry points; fills nchunks.
static int route_check(const char *who, const int32_t *expert_idx, int64_t rows, int num_experts, const int32_t *dst_to_src,
                       const int32_t *src_to_dst, const int32_t *expert_tokens, int64_t *nchunks)
{
    CCH_REQUIRE(rows >= 0 && rows < ((int64_t)1 << 30), "%s: rows=%lld", who, (long long)rows);
    CCH_REQUIRE(num_experts >= 1 && num_experts <= ROUTE_MAX_EXPERTS, "%s: num_experts=%d outside 1..%d", who, num_experts,
                ROUTE_MAX_EXPERTS);
    CCH_REQUIRE(expert_tokens != nullptr, "%s: null expert_tokens", who);
    *nchunks = std::max<int64_t>((rows + ROUTE_CHUNK - 1) / ROUTE_CHUNK, 1);
    CCH_REQUIRE(*nchunks * num_experts < ((int64_t)1 << 31), "%s: rows x experts too large", who);
    CCH_REQUIRE(rows == 0 || (expert_idx && dst_to_src && src_to_dst), "%s: null pointer", who);
    return CCH_OK;
}

// The three launches; hist holds nchunks * num_experts entries, every one of which the histogram
// pass writes before the scan reads it (nothing has to start at zero).
static bool route_fits_one_workgroup(int64_t rows, int num_experts) { return rows > 0 && rows <= ONE_MAX_ROWS && num_experts <= ONE_MAX_EXPERTS; }

static int route_launch(const int32_t *expert_idx, int64_t rows, int num_experts, int64_t nchunks, int32_t *dst_to_src,
                        int32_t *src_to_dst, int32_t *expert_tokens, int cumsum, int32_t *hist, hipStream_t s)
{
    if (route_fits_one_workgroup(rows, num_experts) && !g_route_three_launches.load(std::memory_order_relaxed)) {
        int bits = 0;
        while ((1 << bits) < num_experts) bits++;
        const int groups = (int)((rows + 64 * ONE_WAVES - 1) / (64 * ONE_WAVES));
        hipLaunchKernelGGL(route_one_workgroup_kernel, dim3(1), dim3(64 * ONE_WAVES), 0, s, expert_idx, (int)rows, num_experts, bits, groups,
                           dst_to_src, src_to_dst, expert_tokens, cumsum);
        return launch_status("route kernel");
    }
    hipLaunchKernelGGL(route_histogram_kernel, dim3((unsigned)nchunks), dim3(256), 0, s, expert_idx, (int)rows, num_experts,
                       (int)nchunks, hist, dst_to_src);
    hipLaunchKernelGGL(route_scan_kernel, dim3(1), dim3(1024), 0, s, hist, num_experts, (int)nchunks, expert_tokens, cumsum);
    int bits = 0;
    while ((1 << bits) < num_experts) bits++;
    if (rows > 0)
        hipLaunchKernelGGL(route_place_kernel, dim3((unsigned)nchunks), dim3(64 * ROUTE_WAVES), 0, s, expert_idx, (int)rows,
                           num_experts, (int)nchunks, bits, hist, dst_to_src, src_to_dst);
    return launch_status("route kernels");
}

// Histogram area of cch_moe_init_routing_noalloc: part of the library's device image, so every GPU
// the library runs on holds its own copy (1 MiB) from load to process end.  The name is only a
// host-side handle; the device address is looked up once per device and kept in g_scratch_ptr.
constexpr int64_t ROUTE_STATIC_ENTRIES = CCH_ROUTING_NOALLOC_MAX_ENTRIES;
static __device__ __align__(256) int32_t scratch[ROUTE_STATIC_ENTRIES];
constexpr int ROUTE_MAX_DEVICES = 64;
static std::atomic<int32_t *> g_scratch_ptr[ROUTE_MAX_DEVICES];

// Device address of `scratch` on the current device (looked up on first use, or by cch_init).
int routing_scratch_setup(int32_t **out)
{
    int dev = 0;
    CCH_HIP(hipGetDevice(&dev));
    CCH_REQUIRE(dev >= 0 && dev < ROUTE_MAX_DEVICES, "routing scratch: device %d outside 0..%d", dev, ROUTE_MAX_DEVICES - 1);
    int32_t *ptr = g_scratch_ptr[dev].load(std::memory_order_acquire);
    if (ptr == nullptr) {
        void *sym = nullptr;
        CCH_HIP(hipGetSymbolAddress(&sym, HIP_SYMBOL(scratch)));
        if (sym == nullptr) return fail(CCH_EHIP, "routing scratch: hipGetSymbolAddress gave a null address on device %d", dev);
        ptr = static_cast<int32_t *>(sym);
        g_scratch_ptr[dev].store(ptr, std::memory_order_release);   // two threads racing here store the same address
    }
    if (out) *out = ptr;
    return CCH_OK;
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
    int64_t nchunks = 0;
    int rc = route_check("cch_moe_init_routing", expert_idx, rows, num_experts, dst_to_src, src_to_dst, expert_tokens, &nchunks);
    if (rc) return rc;
    CCH_REQUIRE(workspace != nullptr && workspace_bytes >= cch_moe_init_routing_workspace_bytes(rows, num_experts),
                "cch_moe_init_routing: workspace of %lld bytes, need %lld", (long long)workspace_bytes,
                (long long)cch_moe_init_routing_workspace_bytes(rows, num_experts));
    return route_launch(expert_idx, rows, num_experts, nchunks, dst_to_src, src_to_dst, expert_tokens, cumsum,
                        static_cast<int32_t *>(workspace), static_cast<hipStream_t>(stream));
}

extern "C" int cch_moe_init_routing_noalloc(const int32_t *expert_idx, int64_t rows, int num_experts, int32_t *dst_to_src,
                                            int32_t *src_to_dst, int32_t *expert_tokens, int cumsum, void *stream)
{
    using namespace cch;
    int64_t nchunks = 0;
    int rc = route_check("cch_moe_init_routing_noalloc", expert_idx, rows, num_experts, dst_to_src, src_to_dst, expert_tokens,
                         &nchunks);
    if (rc) return rc;
    CCH_REQUIRE(nchunks * num_experts <= ROUTE_STATIC_ENTRIES,
                "cch_moe_init_routing_noalloc: ceil(rows/%d) * num_experts = %lld exceeds the built-in area of %lld entries; "
                "use cch_moe_init_routing with a workspace", ROUTE_CHUNK, (long long)(nchunks * num_experts),
                (long long)ROUTE_STATIC_ENTRIES);
    int32_t *hist = nullptr;
    rc = routing_scratch_setup(&hist);
    if (rc) return rc;
    return route_launch(expert_idx, rows, num_experts, nchunks, dst_to_src, src_to_dst, expert_tokens, cumsum, hist,
                        static_cast<hipStream_t>(stream));
}
