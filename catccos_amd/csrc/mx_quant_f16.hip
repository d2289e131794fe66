// MX block quantiser for IEEE half input: the `half` instantiation of the reference's quantiser
// (MxQuantTraits<half>, include/catccos/epilogue/block/block_epilogue_dynamic_mx_quant.hpp:57-71;
// CommBlockMxQuant::ComputeMxQuant, include/catccos/comm/block/comm_block_mx_quant.hpp:414-663),
// which widens the input to fp32, takes the shared exponent from the fp32 exponent field of the
// block maximum and multiplies by the power-of-two reciprocal in fp32 before the saturating
// round-to-nearest-even cast.  Here: one lane holds 8 consecutive elements (one 16-byte load),
// four neighbouring lanes one 32-element block; the maximum is taken on the |half| bit patterns
// (monotonic in the value), widened once per block; round-to-nearest-even payloads come from the
// fused packed-half conversions of gfx950, the table rounding rule and E1M2 from the integer-exact
// encoder the bf16 quantiser uses for them.  HBM-bound streaming: 2 B read and 1 B (FP8) or 0.5 B (FP4)
// + 1/32 B written per element.
#include <algorithm>

#include "common.h"
#include "mx_formats.h"
#include "mx_quant_block.h"

namespace cch {

// mx_quant.hip: 1 when the fast streaming kernel does not take the shape, else its launch status
int mx_quant_rows_fast_half(const void *x, void *payload, void *scales, int64_t m, int64_t k, int fmt, hipStream_t stream);

constexpr int F16Q_THREADS = 512;

// Grid-stride over (row, 8-element group): `tpr` groups per row, a multiple of four so that the
// four lanes of a block sit in one quad.  VEC: k % 8 == 0 and 16-byte aligned rows.
template <int FMT, int RND, bool VEC, bool HWCVT>
__global__ __launch_bounds__(F16Q_THREADS) void mx_quant_rows_f16_kernel(const uint16_t *__restrict__ x, uint8_t *__restrict__ payload,
                                                                        uint8_t *__restrict__ scales, int64_t m, int k, int tpr,
                                                                        int pld, int sld)
{
    using T = FmtTraits<FMT>;
    constexpr bool FP4 = is_fp4_v<FMT>;
    const int nblk = (k + 31) / 32;
    const int64_t total = m * (int64_t)tpr;
    for (int64_t gid = (int64_t)blockIdx.x * F16Q_THREADS + threadIdx.x; gid < total; gid += (int64_t)gridDim.x * F16Q_THREADS) {
        const int64_t row = gid / tpr;
        const int t = (int)(gid - row * tpr);      // 8-element group inside the row
        const int k0 = t * 8;
        const uint16_t *xr = x + row * k;
        uint32_t h[8];
        if (VEC) {
            if (k0 < k) {
                // streamed once: non-temporal, like the stores below
                const u32x4 v = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(xr + k0));
                h[0] = v[0] & 0xFFFFu; h[1] = v[0] >> 16; h[2] = v[1] & 0xFFFFu; h[3] = v[1] >> 16;
                h[4] = v[2] & 0xFFFFu; h[5] = v[2] >> 16; h[6] = v[3] & 0xFFFFu; h[7] = v[3] >> 16;
            } else {
#pragma unroll
                for (int i = 0; i < 8; i++) h[i] = 0;
            }
        } else {
#pragma unroll
            for (int i = 0; i < 8; i++) h[i] = (k0 + i < k) ? xr[k0 + i] : 0u;   // a ragged last block is zero padded
        }
        // block maximum of the |half| patterns over the quad's 32 elements
        uint32_t amax_bits = 0;
#pragma unroll
        for (int i = 0; i < 8; i++) amax_bits = max(amax_bits, h[i] & 0x7FFFu);
        amax_bits = max(amax_bits, (uint32_t)__shfl_xor((int)amax_bits, 1, 4));
        amax_bits = max(amax_bits, (uint32_t)__shfl_xor((int)amax_bits, 2, 4));
        const bool is_nan = amax_bits >= 0x7C00u;   // Inf or NaN in the block
        int e;
        const uint32_t sbyte = shared_exp_byte_f32<FMT>(half_bits_to_f32(amax_bits), is_nan, e);
        const float rscale = pow2i(-e);             // finite half input keeps e within [-24 - EMAX, 15 - EMAX]
        uint32_t code[8];
        if constexpr (HWCVT) {
            const uint32_t w[4] = {h[0] | h[1] << 16, h[2] | h[3] << 16, h[4] | h[5] << 16, h[6] | h[7] << 16};
            uint32_t o[2];
            quant8_f16_hw<FMT>(w, e, o);
            constexpr int CB = FP4 ? 4 : 8;                   // bits per code
#pragma unroll
            for (int i = 0; i < 8; i++) code[i] = is_nan ? T::NANCODE : ((o[(i * CB) >> 5] >> ((i * CB) & 31)) & ((1u << CB) - 1u));
        } else {
#pragma unroll
            for (int i = 0; i < 8; i++) {
                // exact: a power-of-two multiple of a half value that stays a normal fp32 number
                const float y = half_bits_to_f32(h[i]) * rscale;
                code[i] = is_nan ? T::NANCODE : encode_small<FMT, RND>(y);
            }
        }
        if (FP4) {
            const uint32_t w = code[0] | code[1] << 4 | code[2] << 8 | code[3] << 12 | code[4] << 16 | code[5] << 20 |
                               code[6] << 24 | code[7] << 28;
            uint8_t *pr = payload + row * pld + (k0 >> 1);
            if (VEC) {
                if (k0 < k) __builtin_nontemporal_store(w, reinterpret_cast<uint32_t *>(pr));
            } else {
#pragma unroll
                for (int i = 0; i < 4; i++)
                    if (k0 + 2 * i < k) pr[i] = (uint8_t)(w >> (8 * i));
            }
        } else {
            const uint32_t lo = code[0] | code[1] << 8 | code[2] << 16 | code[3] << 24;
            const uint32_t hi = code[4] | code[5] << 8 | code[6] << 16 | code[7] << 24;
            uint8_t *pr = payload + row * pld + k0;
            if (VEC) {
                if (k0 < k) __builtin_nontemporal_store((u32x2){lo, hi}, reinterpret_cast<u32x2 *>(pr));
            } else {
#pragma unroll
                for (int i = 0; i < 8; i++)
                    if (k0 + i < k) pr[i] = (uint8_t)code[i];
            }
        }
        // one lane of the quad writes the block's scale; the lane of the last block also writes
        // the padding entry (1.0 = 127) when the block count is odd
        if ((t & 3) == 0) {
            const int b = t >> 2;
            uint8_t *sr = scales + row * sld;
            if (b < nblk) sr[b] = (uint8_t)sbyte;
            if (b == nblk - 1 && nblk < sld) sr[nblk] = 127;
        }
    }
}

template <int FMT, int RND>
static int launch_f16(const void *x, void *payload, void *scales, int64_t m, int64_t k, hipStream_t stream)
{
    const int nblk = (int)((k + 31) / 32);
    const int tpr = nblk * 4;
    const int sld = 2 * ((nblk + 1) / 2);
    const int pld = is_fp4_v<FMT> ? (int)((k + 1) / 2) : (int)k;
    const int64_t total = m * (int64_t)tpr;
    int dev = 0, cus = 0;
    CCH_HIP(hipGetDevice(&dev));
    CCH_HIP(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev));
    const int64_t want = (total + F16Q_THREADS - 1) / F16Q_THREADS;
    const unsigned grid = (unsigned)std::max<int64_t>(1, std::min<int64_t>(want, (int64_t)cus * 8));
    // 16-byte loads, 8-byte (FP8) or 4-byte (FP4) stores: whole groups and aligned rows
    const bool vec = k % 8 == 0 && aligned(x, 16) && aligned(payload, 8);
    const uint16_t *xi = static_cast<const uint16_t *>(x);
    uint8_t *p = static_cast<uint8_t *>(payload), *s = static_cast<uint8_t *>(scales);
    // the fused conversions exist for round-to-nearest-even into E4M3, E5M2 and E2M1
    constexpr bool HW = RND == CCH_ROUND_RNE && FMT != CCH_FMT_E1M2;
    if (vec)
        hipLaunchKernelGGL((mx_quant_rows_f16_kernel<FMT, RND, true, HW>), dim3(grid), dim3(F16Q_THREADS), 0, stream, xi, p, s, m,
                           (int)k, tpr, pld, sld);
    else
        hipLaunchKernelGGL((mx_quant_rows_f16_kernel<FMT, RND, false, HW>), dim3(grid), dim3(F16Q_THREADS), 0, stream, xi, p, s, m,
                           (int)k, tpr, pld, sld);
    return launch_status("mx_quant_rows_f16_kernel");
}

}  // namespace cch

extern "C" int cch_mx_quant_rows_f16(const void *x, void *payload, void *scales, int64_t m, int64_t k, int fmt, int rounding,
                                     void *stream)
{
    using namespace cch;
    CCH_REQUIRE(m >= 0 && k >= 0, "cch_mx_quant_rows_f16: negative shape m=%lld k=%lld", (long long)m, (long long)k);
    CCH_REQUIRE(k < (int64_t)1 << 30, "cch_mx_quant_rows_f16: k=%lld too large", (long long)k);
    CCH_REQUIRE(rounding == CCH_ROUND_RNE || rounding == CCH_ROUND_LUT, "cch_mx_quant_rows_f16: rounding %d", rounding);
    CCH_REQUIRE(fmt == CCH_FMT_E4M3 || fmt == CCH_FMT_E5M2 || fmt == CCH_FMT_E2M1 || fmt == CCH_FMT_E1M2,
                "cch_mx_quant_rows_f16: unknown format %d", fmt);
    if (m == 0 || k == 0) return CCH_OK;
    CCH_REQUIRE(x && payload && scales, "cch_mx_quant_rows_f16: null pointer");
    hipStream_t s = static_cast<hipStream_t>(stream);
    const bool lut = rounding == CCH_ROUND_LUT;
    if (!lut) {
        // whole 1024-element pieces per row and aligned buffers: the streaming form shared with the bf16 quantiser
        const int rc = mx_quant_rows_fast_half(x, payload, scales, m, k, fmt, s);
        if (rc != 1) return rc;
    }
    switch (fmt) {
        case CCH_FMT_E4M3:
            return lut ? launch_f16<CCH_FMT_E4M3, CCH_ROUND_LUT>(x, payload, scales, m, k, s)
                       : launch_f16<CCH_FMT_E4M3, CCH_ROUND_RNE>(x, payload, scales, m, k, s);
        case CCH_FMT_E5M2:
            return lut ? launch_f16<CCH_FMT_E5M2, CCH_ROUND_LUT>(x, payload, scales, m, k, s)
                       : launch_f16<CCH_FMT_E5M2, CCH_ROUND_RNE>(x, payload, scales, m, k, s);
        case CCH_FMT_E2M1:
            return lut ? launch_f16<CCH_FMT_E2M1, CCH_ROUND_LUT>(x, payload, scales, m, k, s)
                       : launch_f16<CCH_FMT_E2M1, CCH_ROUND_RNE>(x, payload, scales, m, k, s);
        default:
            return lut ? launch_f16<CCH_FMT_E1M2, CCH_ROUND_LUT>(x, payload, scales, m, k, s)
                       : launch_f16<CCH_FMT_E1M2, CCH_ROUND_RNE>(x, payload, scales, m, k, s);
    }
}
