// MoE token un-permute (combine side): every output token is the probability-weighted sum of its
// top-K rows of the expert outputs.  Streaming, HBM-bound gather-reduce: a lane owns 8 consecutive
// columns (one 16-byte load per routed row), all of a token's routed rows are requested before the
// first is used, the sum is kept in fp32 and leaves as one 16-byte store.
//
// Follows KernelMoeTokenUnpermute (examples/aux_ops/moe_token_unpermute/moe_token_unpermute.h:
// 235-279 CalPartOutToken, :298-343 CalFirstToken / CalToken, :345-355 CopyOut): the first route
// initialises the sum (x * p, or zero when its index is out of range), every further route in
// range adds its separately rounded product, and the result is rounded to nearest even.
#include <algorithm>

#include "common.h"

namespace cch {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));

constexpr int UNP_THREADS = 256;
constexpr int UNP_MAX_TOPK = 8;
constexpr int UNP_BLOCKS_PER_CU = 8;

// VEC: hidden % 8 == 0 and 16-byte aligned rows; otherwise element-wise accesses.
template <bool PROBS, bool VEC>
__global__ __launch_bounds__(UNP_THREADS) void moe_token_unpermute_kernel(
    const uint16_t *__restrict__ permuted, const int32_t *__restrict__ sorted_indices, const float *__restrict__ probs,
    uint16_t *__restrict__ out, int rows, int hidden, int topk, int wpt, int total_ws)
{
    // each product is rounded before it is added: no fused multiply-add in this function
#pragma clang fp contract(off)
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane((int)(blockIdx.x * (UNP_THREADS / 64) + (threadIdx.x >> 6)));
    const int stride = (int)gridDim.x * (UNP_THREADS / 64);
    for (int ws = wave; ws < total_ws; ws += stride) {
        const int t = ws / wpt;                            // token (wave-uniform)
        const int c0 = ((ws - t * wpt) * 64 + lane) * 8;   // first column of this lane
        int idx[UNP_MAX_TOPK];
        float p[UNP_MAX_TOPK];
        uint32_t w[UNP_MAX_TOPK][4];
#pragma unroll
        for (int j = 0; j < UNP_MAX_TOPK; j++) {
            idx[j] = -1;
            p[j] = 0.0f;
            if (j < topk) {
                idx[j] = sorted_indices[(size_t)t * topk + j];
                if (PROBS) p[j] = probs[(size_t)t * topk + j];
                if (idx[j] >= rows) idx[j] = -1;
            }
            w[j][0] = w[j][1] = w[j][2] = w[j][3] = 0;
            if (idx[j] >= 0 && c0 < hidden) {
                const uint16_t *src = permuted + (size_t)idx[j] * hidden + c0;
                if (VEC) {
                    const u32x4 v = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(src));
                    w[j][0] = v[0]; w[j][1] = v[1]; w[j][2] = v[2]; w[j][3] = v[3];
                } else {
#pragma unroll
                    for (int i = 0; i < 8; i++)
                        if (c0 + i < hidden) w[j][i >> 1] |= (uint32_t)src[i] << ((i & 1) * 16);
                }
            }
        }
        float acc[8];
#pragma unroll
        for (int i = 0; i < 8; i++) acc[i] = 0.0f;
#pragma unroll
        for (int j = 0; j < UNP_MAX_TOPK; j++) {
            if (idx[j] < 0) continue;  // wave-uniform
#pragma unroll
            for (int i = 0; i < 8; i++) {
                const float x = __uint_as_float((i & 1) ? (w[j][i >> 1] & 0xFFFF0000u) : (w[j][i >> 1] << 16));
                const float v = PROBS ? x * p[j] : x;
                acc[i] = j == 0 ? v : acc[i] + v;   // the first route assigns, the others add
            }
        }
        if (c0 < hidden) {
            uint32_t o[4];
#pragma unroll
            for (int i = 0; i < 4; i++)
                o[i] = __builtin_bit_cast(uint32_t, __builtin_convertvector((f32x2){acc[2 * i], acc[2 * i + 1]}, bf16x2));
            uint16_t *dst = out + (size_t)t * hidden + c0;
            if (VEC) {
                __builtin_nontemporal_store((u32x4){o[0], o[1], o[2], o[3]}, reinterpret_cast<u32x4 *>(dst));
            } else {
#pragma unroll
                for (int i = 0; i < 8; i++)
                    if (c0 + i < hidden) dst[i] = (uint16_t)(o[i >> 1] >> ((i & 1) * 16));
            }
        }
    }
}

}  // namespace cch

extern "C" int cch_moe_token_unpermute(const void *permuted_tokens, const int32_t *sorted_indices, const float *probs, void *out,
                                       int64_t rows, int64_t tokens, int64_t hidden, int top_k, void *stream)
{
    using namespace cch;
    CCH_REQUIRE(rows >= 0 && tokens >= 0 && hidden >= 0, "cch_moe_token_unpermute: negative shape rows=%lld tokens=%lld hidden=%lld",
                (long long)rows, (long long)tokens, (long long)hidden);
    CCH_REQUIRE(top_k >= 1 && top_k <= UNP_MAX_TOPK, "cch_moe_token_unpermute: top_k=%d outside 1..%d", top_k, UNP_MAX_TOPK);
    CCH_REQUIRE(rows < ((int64_t)1 << 31) && hidden < ((int64_t)1 << 30), "cch_moe_token_unpermute: shape too large");
    if (tokens == 0 || hidden == 0) return CCH_OK;
    CCH_REQUIRE(sorted_indices && out && (permuted_tokens || rows == 0), "cch_moe_token_unpermute: null pointer");
    const int64_t wpt = (hidden + 511) / 512;   // wave-steps per token
    CCH_REQUIRE(tokens * wpt < ((int64_t)1 << 31), "cch_moe_token_unpermute: tokens=%lld x hidden=%lld too large for one launch",
                (long long)tokens, (long long)hidden);
    int dev = 0, cus = 0;
    CCH_HIP(hipGetDevice(&dev));
    CCH_HIP(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev));
    const int64_t total_ws = tokens * wpt;
    const unsigned grid = (unsigned)std::max<int64_t>(
        1, std::min<int64_t>((total_ws + UNP_THREADS / 64 - 1) / (UNP_THREADS / 64), (int64_t)cus * UNP_BLOCKS_PER_CU));
    const bool vec = hidden % 8 == 0 && aligned(permuted_tokens, 16) && aligned(out, 16);
    hipStream_t s = static_cast<hipStream_t>(stream);
    const uint16_t *src = static_cast<const uint16_t *>(permuted_tokens);
    uint16_t *dst = static_cast<uint16_t *>(out);
#define CCH_UNP_LAUNCH(P, V)                                                                                              \
    hipLaunchKernelGGL((moe_token_unpermute_kernel<P, V>), dim3(grid), dim3(UNP_THREADS), 0, s, src, sorted_indices, probs, \
                       dst, (int)rows, (int)hidden, top_k, (int)wpt, (int)total_ws)
    if (probs) {
        if (vec) CCH_UNP_LAUNCH(true, true);
        else CCH_UNP_LAUNCH(true, false);
    } else {
        if (vec) CCH_UNP_LAUNCH(false, true);
        else CCH_UNP_LAUNCH(false, false);
    }
#undef CCH_UNP_LAUNCH
    return launch_status("moe_token_unpermute_kernel");
}
