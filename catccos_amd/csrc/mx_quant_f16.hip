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

namespace cch {

constexpr int F16Q_THREADS = 512;

__device__ __forceinline__ float half_bits_to_f32(uint32_t h)
{
    return (float)__builtin_bit_cast(_Float16, (uint16_t)h);
}

// E8M0 byte and applied exponent from the block maximum as fp32 (the rule of shared_exp_byte,
// on the fp32 exponent field: a subnormal half maximum is a normal fp32 number).
template <int FMT>
__device__ __forceinline__ uint32_t shared_exp_byte_f32(float amax, bool is_nan, int &e_out)
{
    using T = FmtTraits<FMT>;
    int e = (int)((__float_as_uint(amax) >> 23) & 0xFFu) - 127 - T::EMAX;
    e = max(-128, min(127, e));
    if (amax < 1e-12f) e = 0;
    e_out = max(e, -127);
    return is_nan ? 0xFFu : (uint32_t)max(e + 127, 0);
}

typedef short s16x2 __attribute__((ext_vector_type(2)));
typedef unsigned short u16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

// Round-to-nearest-even payloads of 8 packed halves (w[i] = elements 2i, 2i+1) with gfx950's fused
// conversions, which divide by the power-of-two scale and round straight from packed half.  The
// FP4 form saturates; the FP8 forms return NaN above the format maximum, so magnitudes are first
// clamped, as 16-bit integers, to the half pattern of MAXV * 2^e = 1.75 * 2^(e + EMAX) (for a
// subnormal block maximum that limit is subnormal too: the pattern 0x700 shifted down).
template <int FMT>
__device__ __forceinline__ void quant8_f16_hw(const uint32_t (&w)[4], int e, uint32_t (&out)[2])
{
    using T = FmtTraits<FMT>;
    const float scale = __uint_as_float((uint32_t)(e + 127) << 23);
    if constexpr (FMT == CCH_FMT_E2M1) {
        uint32_t r = 0;
        r = __builtin_amdgcn_cvt_scalef32_pk_fp4_f16(r, __builtin_bit_cast(f16x2, w[0]), scale, 0);
        r = __builtin_amdgcn_cvt_scalef32_pk_fp4_f16(r, __builtin_bit_cast(f16x2, w[1]), scale, 1);
        r = __builtin_amdgcn_cvt_scalef32_pk_fp4_f16(r, __builtin_bit_cast(f16x2, w[2]), scale, 2);
        r = __builtin_amdgcn_cvt_scalef32_pk_fp4_f16(r, __builtin_bit_cast(f16x2, w[3]), scale, 3);
        out[0] = r;
        out[1] = 0;
    } else {
        const int fe = e + T::EMAX + 15;   // half exponent field of the limit
        const uint32_t t16 = fe > 30 ? 0x7BFFu : fe >= 1 ? (((uint32_t)fe << 10) | 0x300u) : (0x700u >> min(1 - fe, 11));
        const u16x2 lim = {(unsigned short)t16, (unsigned short)t16};
        f16x2 c[4];
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const u16x2 mag = __builtin_elementwise_min(__builtin_bit_cast(u16x2, w[i] & 0x7FFF7FFFu), lim);
            c[i] = __builtin_bit_cast(f16x2, __builtin_bit_cast(uint32_t, mag) | (w[i] & 0x80008000u));
        }
        s16x2 r0 = {0, 0}, r1 = {0, 0};
        if constexpr (FMT == CCH_FMT_E4M3) {
            r0 = __builtin_amdgcn_cvt_scalef32_pk_fp8_f16(r0, c[0], scale, false);
            r0 = __builtin_amdgcn_cvt_scalef32_pk_fp8_f16(r0, c[1], scale, true);
            r1 = __builtin_amdgcn_cvt_scalef32_pk_fp8_f16(r1, c[2], scale, false);
            r1 = __builtin_amdgcn_cvt_scalef32_pk_fp8_f16(r1, c[3], scale, true);
        } else {
            r0 = __builtin_amdgcn_cvt_scalef32_pk_bf8_f16(r0, c[0], scale, false);
            r0 = __builtin_amdgcn_cvt_scalef32_pk_bf8_f16(r0, c[1], scale, true);
            r1 = __builtin_amdgcn_cvt_scalef32_pk_bf8_f16(r1, c[2], scale, false);
            r1 = __builtin_amdgcn_cvt_scalef32_pk_bf8_f16(r1, c[3], scale, true);
        }
        out[0] = __builtin_bit_cast(uint32_t, r0);
        out[1] = __builtin_bit_cast(uint32_t, r1);
    }
}

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
