// Device-side number formats of the MX path: bf16, E4M3 / E5M2 / E2M1 / E1M2 payload codes,
// E8M0 block scales.  Arithmetic is integer-exact so that results are bit-identical
// to the CPU golden of the reference (examples/utils/gen_mx_quant_allgather_data.py).
#pragma once
#include <hip/hip_runtime.h>

#include <cstdint>

#include "catccos_hip.h"

namespace cch {

template <int FMT> struct FmtTraits;
template <> struct FmtTraits<CCH_FMT_E4M3> {
    static constexpr int MB = 3, BIAS = 7, EMAX = 8;
    static constexpr float MAXV = 448.0f;
    static constexpr uint32_t SIGN = 0x80u, NANCODE = 0x7Fu;
};
template <> struct FmtTraits<CCH_FMT_E5M2> {
    static constexpr int MB = 2, BIAS = 15, EMAX = 15;
    static constexpr float MAXV = 57344.0f;
    static constexpr uint32_t SIGN = 0x80u, NANCODE = 0x7Fu;
};
template <> struct FmtTraits<CCH_FMT_E2M1> {
    static constexpr int MB = 1, BIAS = 1, EMAX = 2;
    static constexpr float MAXV = 6.0f;
    static constexpr uint32_t SIGN = 0x8u, NANCODE = 0x7u;
};

// E1M2 (examples/utils/gen_mx_quant_allgather_data.py:65-72): subnormals m/4, normals 1 + m/4.
template <> struct FmtTraits<CCH_FMT_E1M2> {
    static constexpr int MB = 2, BIAS = 1, EMAX = 0;
    static constexpr float MAXV = 1.75f;
    static constexpr uint32_t SIGN = 0x8u, NANCODE = 0x7u;
};
// The two 4-bit formats share the packing: two codes per byte, element 2j in the low nibble.
template <int FMT> constexpr bool is_fp4_v = FMT == CCH_FMT_E2M1 || FMT == CCH_FMT_E1M2;

__device__ __forceinline__ float bf16_bits_to_f32(uint32_t h) { return __uint_as_float(h << 16); }

// fp32 -> bf16 bits, round to nearest even (NaN kept quiet).
__device__ __forceinline__ uint32_t f32_to_bf16_bits(float f)
{
    uint32_t u = __float_as_uint(f);
    uint32_t r = (u + 0x7FFFu + ((u >> 16) & 1u)) >> 16;
    return (f != f) ? ((u >> 16) | 0x40u) : r;
}

// 2^e as fp32 for e in [-126,127].
__device__ __forceinline__ float pow2i(int e) { return __uint_as_float((uint32_t)(e + 127) << 23); }

// Rounds an already scaled, finite value to the nearest code of FMT, saturating at the
// format maximum.  RND = CCH_ROUND_RNE: ties to the even code, sign kept on zero.
// RND = CCH_ROUND_LUT: ties to the smaller magnitude, every zero result is +0.
template <int FMT, int RND>
__device__ __forceinline__ uint32_t encode_small(float y)
{
    using T = FmtTraits<FMT>;
    constexpr int SHIFT = 23 - T::MB;
    const uint32_t sign = __float_as_uint(y) >> 31;
    const float a = fminf(fabsf(y), T::MAXV);
    const uint32_t ab = __float_as_uint(a);
    uint32_t code;
    if (a >= __uint_as_float((uint32_t)(1 - T::BIAS + 127) << 23)) {
        uint32_t r = ab + ((1u << (SHIFT - 1)) - 1u);
        if (RND == CCH_ROUND_RNE) r += (ab >> SHIFT) & 1u;
        code = (r >> SHIFT) - ((uint32_t)(127 - T::BIAS) << T::MB);
    } else {
        const float t = a * __uint_as_float((uint32_t)(T::BIAS - 1 + T::MB + 127) << 23);  // exact
        code = (RND == CCH_ROUND_RNE) ? (uint32_t)rintf(t) : (uint32_t)ceilf(t - 0.5f);
    }
    if (RND == CCH_ROUND_LUT && code == 0) return 0;
    return code | (sign ? T::SIGN : 0u);
}

// Shared exponent of a block from the bf16 bit pattern of its absolute maximum
// (gen_mx_quant_allgather_data.py:168-189).  Returns the E8M0 byte; `e_out` is the exponent
// actually applied to the payload.  Blocks holding Inf/NaN give 0xFF.
template <int FMT>
__device__ __forceinline__ uint32_t shared_exp_byte(uint32_t amax_bits, int &e_out, bool &is_nan)
{
    using T = FmtTraits<FMT>;
    is_nan = amax_bits >= 0x7F80u;
    const float amax = bf16_bits_to_f32(amax_bits);
    int e = (int)(amax_bits >> 7) - 127 - T::EMAX;
    e = max(-128, min(127, e));
    if (amax < 1e-12f) e = 0;
    e_out = max(e, -127);
    return is_nan ? 0xFFu : (uint32_t)max(e + 127, 0);
}

}  // namespace cch
