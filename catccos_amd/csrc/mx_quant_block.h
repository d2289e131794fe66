// Quantisation of one MX block held by a quad of lanes: every lane owns 8 consecutive bf16
// elements (four packed dwords), four neighbouring lanes own the 32-element block.  Shared by the
// streaming quantisers and by the GEMM epilogue that writes its activation in MX form.
//
// Follows CommBlockMxQuant::ComputeMxQuant (include/catccos/comm/block/comm_block_mx_quant.hpp:414-663)
// in intent and the generator examples/utils/gen_mx_quant_allgather_data.py:255-313, :385-449
// bit for bit.
#pragma once
#include "mx_formats.h"

namespace cch {

typedef short s16x2 __attribute__((ext_vector_type(2)));
typedef unsigned short u16x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));

// Software path: scale in fp32, round with the integer encoder (any rounding rule).
template <int FMT, int RND>
__device__ __forceinline__ void quant8_soft(const uint32_t (&w)[4], int e, bool is_nan, uint32_t (&out)[2])
{
    using T = FmtTraits<FMT>;
    // 2^-e in two exact factors: 2^-127 (a format whose largest exponent is 0 meets a block
    // maximum of 2^127) is no normal float
    const float inv = pow2i(-min(e, 126)), inv2 = e > 126 ? 0.5f : 1.0f;
    float y[8];
#pragma unroll
    for (int i = 0; i < 4; i++) {
        y[2 * i] = __uint_as_float(w[i] << 16) * inv * inv2;
        y[2 * i + 1] = __uint_as_float(w[i] & 0xFFFF0000u) * inv * inv2;
    }
    if constexpr (is_fp4_v<FMT>) {
        uint32_t r = 0;
#pragma unroll
        for (int i = 0; i < 8; i++) r |= (is_nan ? T::NANCODE : encode_small<FMT, RND>(y[i])) << (4 * i);
        out[0] = r;
        out[1] = 0;
    } else {
        uint32_t r0 = 0, r1 = 0;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            r0 |= (is_nan ? T::NANCODE : encode_small<FMT, RND>(y[i])) << (8 * i);
            r1 |= (is_nan ? T::NANCODE : encode_small<FMT, RND>(y[4 + i])) << (8 * i);
        }
        out[0] = r0;
        out[1] = r1;
    }
}

// Hardware path (round to nearest even, sign kept on zero): the packed bf16 -> FP8 / FP4
// conversions of gfx950 divide by a power-of-two scale and round in one instruction, two values
// at a time, straight from the packed bf16 input.  The FP4 form saturates; the FP8 forms return
// NaN above the format maximum, so magnitudes are first clamped, as 16-bit integers, to the bf16
// pattern of MAXV * 2^e.  Checked against the software path for every finite bf16 input and
// every applied exponent from -127 to 119.
template <int FMT>
__device__ __forceinline__ void quant8_hw(const uint32_t (&w)[4], int e, bool is_nan, uint32_t (&out)[2])
{
    using T = FmtTraits<FMT>;
    const float scale = __uint_as_float((uint32_t)(e + 127) << 23);  // exponent field 0 stands for 2^-127
    if constexpr (FMT == CCH_FMT_E2M1) {
        uint32_t r = 0;
        r = __builtin_amdgcn_cvt_scalef32_pk_fp4_bf16(r, __builtin_bit_cast(bf16x2, w[0]), scale, 0);
        r = __builtin_amdgcn_cvt_scalef32_pk_fp4_bf16(r, __builtin_bit_cast(bf16x2, w[1]), scale, 1);
        r = __builtin_amdgcn_cvt_scalef32_pk_fp4_bf16(r, __builtin_bit_cast(bf16x2, w[2]), scale, 2);
        r = __builtin_amdgcn_cvt_scalef32_pk_fp4_bf16(r, __builtin_bit_cast(bf16x2, w[3]), scale, 3);
        out[0] = is_nan ? 0x77777777u : r;
        out[1] = 0;
    } else {
        // MAXV = 1.75 * 2^EMAX in both FP8 formats: mantissa bits 1100000 under exponent e + EMAX
        const int te = e + T::EMAX + 127;
        const uint32_t t16 = te > 254 ? 0x7F7Fu : (((uint32_t)te << 7) | 0x60u);
        const u16x2 lim = {(unsigned short)t16, (unsigned short)t16};
        bf16x2 c[4];
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const u16x2 mag = __builtin_elementwise_min(__builtin_bit_cast(u16x2, w[i] & 0x7FFF7FFFu), lim);
            c[i] = __builtin_bit_cast(bf16x2, __builtin_bit_cast(uint32_t, mag) | (w[i] & 0x80008000u));
        }
        s16x2 r0 = {0, 0}, r1 = {0, 0};
        if constexpr (FMT == CCH_FMT_E4M3) {
            r0 = __builtin_amdgcn_cvt_scalef32_pk_fp8_bf16(r0, c[0], scale, false);
            r0 = __builtin_amdgcn_cvt_scalef32_pk_fp8_bf16(r0, c[1], scale, true);
            r1 = __builtin_amdgcn_cvt_scalef32_pk_fp8_bf16(r1, c[2], scale, false);
            r1 = __builtin_amdgcn_cvt_scalef32_pk_fp8_bf16(r1, c[3], scale, true);
        } else {
            r0 = __builtin_amdgcn_cvt_scalef32_pk_bf8_bf16(r0, c[0], scale, false);
            r0 = __builtin_amdgcn_cvt_scalef32_pk_bf8_bf16(r0, c[1], scale, true);
            r1 = __builtin_amdgcn_cvt_scalef32_pk_bf8_bf16(r1, c[2], scale, false);
            r1 = __builtin_amdgcn_cvt_scalef32_pk_bf8_bf16(r1, c[3], scale, true);
        }
        out[0] = is_nan ? 0x7F7F7F7Fu : __builtin_bit_cast(uint32_t, r0);
        out[1] = is_nan ? 0x7F7F7F7Fu : __builtin_bit_cast(uint32_t, r1);
    }
}

template <int FMT, int RND, bool HWCVT>
__device__ __forceinline__ void quant8(const uint32_t (&w)[4], int e, bool is_nan, uint32_t (&out)[2])
{
    if constexpr (HWCVT) quant8_hw<FMT>(w, e, is_nan, out);
    else quant8_soft<FMT, RND>(w, e, is_nan, out);
}

// Largest |bf16| bit pattern among the 8 values packed in w, then across the 4 lanes of the quad.
__device__ __forceinline__ uint32_t block_amax_bits(const uint32_t (&w)[4])
{
    const u16x2 a0 = __builtin_bit_cast(u16x2, w[0] & 0x7FFF7FFFu), a1 = __builtin_bit_cast(u16x2, w[1] & 0x7FFF7FFFu);
    const u16x2 a2 = __builtin_bit_cast(u16x2, w[2] & 0x7FFF7FFFu), a3 = __builtin_bit_cast(u16x2, w[3] & 0x7FFF7FFFu);
    const u16x2 mm = __builtin_elementwise_max(__builtin_elementwise_max(a0, a1), __builtin_elementwise_max(a2, a3));
    uint32_t m = max((uint32_t)mm[0], (uint32_t)mm[1]);
    m = max(m, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)m, 0xB1, 0xF, 0xF, true));  // quad_perm [1,0,3,2]
    m = max(m, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)m, 0x4E, 0xF, 0xF, true));  // quad_perm [2,3,0,1]
    return m;
}

// ---- IEEE half input (the `half` instantiation of the reference's quantiser, MxQuantTraits<half>,
// include/catccos/epilogue/block/block_epilogue_dynamic_mx_quant.hpp:57-71)

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

}  // namespace cch
