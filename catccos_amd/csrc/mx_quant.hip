// MX block quantiser: bf16 -> FP8 (E4M3/E5M2) or FP4 (E2M1) payload + one E8M0 scale per
// 32 elements.  Streaming, HBM-bound kernel: every lane owns 8 consecutive elements (one
// 16-byte load), four neighbouring lanes own one MX block and reduce its maximum with two
// DPP quad permutes; payload leaves as one 8-byte (FP8) or 4-byte (FP4) store per lane.
//
// Follows CommBlockMxQuant::ComputeMxQuant (include/catccos/comm/block/comm_block_mx_quant.hpp:414-663)
// in intent and the generator examples/utils/gen_mx_quant_allgather_data.py:255-313, :385-449
// bit for bit.
#include "common.h"
#include "mx_formats.h"

namespace cch {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

constexpr int QUANT_THREADS = 256;
constexpr int QUANT_UNROLL = 4;  // wave-steps (64 lanes x 8 elements) per wave

template <int FMT, int RND, bool HWCVT>
__device__ __forceinline__ void quant8(const uint32_t (&w)[4], int e, bool is_nan, uint32_t (&out)[2])
{
    using T = FmtTraits<FMT>;
    const float inv = pow2i(-e);
    float y[8];
#pragma unroll
    for (int i = 0; i < 4; i++) {
        y[2 * i] = __uint_as_float(w[i] << 16) * inv;
        y[2 * i + 1] = __uint_as_float(w[i] & 0xFFFF0000u) * inv;
    }
    if constexpr (FMT == CCH_FMT_E2M1) {
        uint32_t r = 0;
#pragma unroll
        for (int i = 0; i < 8; i++) r |= (is_nan ? T::NANCODE : encode_small<FMT, RND>(y[i])) << (4 * i);
        out[0] = r;
        out[1] = 0;
    } else if constexpr (HWCVT) {
        // Hardware cast: round to nearest even; the clamp keeps it away from its overflow rule.
        int r0 = 0, r1 = 0;
#pragma unroll
        for (int i = 0; i < 8; i++) y[i] = __builtin_amdgcn_fmed3f(y[i], -T::MAXV, T::MAXV);
        r0 = __builtin_amdgcn_cvt_pk_fp8_f32(y[0], y[1], r0, false);
        r0 = __builtin_amdgcn_cvt_pk_fp8_f32(y[2], y[3], r0, true);
        r1 = __builtin_amdgcn_cvt_pk_fp8_f32(y[4], y[5], r1, false);
        r1 = __builtin_amdgcn_cvt_pk_fp8_f32(y[6], y[7], r1, true);
        out[0] = is_nan ? 0x7F7F7F7Fu : (uint32_t)r0;
        out[1] = is_nan ? 0x7F7F7F7Fu : (uint32_t)r1;
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

// Largest |bf16| bit pattern among the 8 values packed in w, then across the 4 lanes of the quad.
__device__ __forceinline__ uint32_t block_amax_bits(const uint32_t (&w)[4])
{
    uint32_t m = 0;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const uint32_t a = w[i] & 0x7FFF7FFFu;
        m = max(m, max(a & 0xFFFFu, a >> 16));
    }
    m = max(m, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)m, 0xB1, 0xF, 0xF, true));  // quad_perm [1,0,3,2]
    m = max(m, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)m, 0x4E, 0xF, 0xF, true));  // quad_perm [2,3,0,1]
    return m;
}

// x [rows,K] bf16.  One wave-step = 64 lanes x 8 elements of one row; a row has `wpr` wave-steps.
// VEC: K % 8 == 0 and all pointers suitably aligned, so whole-vector accesses are legal.
template <int FMT, int RND, bool HWCVT, bool VEC>
__global__ __launch_bounds__(QUANT_THREADS) void mx_quant_rows_kernel(
    const uint16_t *__restrict__ x, uint8_t *__restrict__ payload, uint8_t *__restrict__ scales, int rows, int K,
    int nblk, int sld, int pld, int wpr, int total_ws)
{
    constexpr bool FP4 = FMT == CCH_FMT_E2M1;
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane((int)(blockIdx.x * (QUANT_THREADS / 64) + (threadIdx.x >> 6)));
    uint32_t w[QUANT_UNROLL][4];
    int row[QUANT_UNROLL], k0[QUANT_UNROLL];

#pragma unroll
    for (int u = 0; u < QUANT_UNROLL; u++) {
        const int ws = wave * QUANT_UNROLL + u;
        const int r = ws / wpr;
        row[u] = ws < total_ws ? r : -1;
        k0[u] = ((ws - r * wpr) * 64 + lane) * 8;
        w[u][0] = w[u][1] = w[u][2] = w[u][3] = 0;
        if (row[u] >= 0 && k0[u] < K) {
            const uint16_t *src = x + (size_t)row[u] * K + k0[u];
            if (VEC) {
                const u32x4 v = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(src));
                w[u][0] = v[0]; w[u][1] = v[1]; w[u][2] = v[2]; w[u][3] = v[3];
            } else {
#pragma unroll
                for (int i = 0; i < 8; i++)
                    if (k0[u] + i < K) w[u][i >> 1] |= (uint32_t)src[i] << ((i & 1) * 16);
            }
        }
    }

#pragma unroll
    for (int u = 0; u < QUANT_UNROLL; u++) {
        if (row[u] < 0) continue;  // wave-uniform
        const uint32_t amax_bits = block_amax_bits(w[u]);
        int e;
        bool is_nan;
        const uint32_t sbyte = shared_exp_byte<FMT>(amax_bits, e, is_nan);
        uint32_t q[2];
        quant8<FMT, RND, HWCVT>(w[u], e, is_nan, q);
        const int blk = k0[u] >> 5;
        if (k0[u] < K) {
            uint8_t *dst = payload + (size_t)row[u] * pld + (FP4 ? (k0[u] >> 1) : k0[u]);
            if (VEC) {
                if (FP4) {
                    __builtin_nontemporal_store(q[0], reinterpret_cast<uint32_t *>(dst));
                } else {
                    u32x2 o = {q[0], q[1]};
                    __builtin_nontemporal_store(o, reinterpret_cast<u32x2 *>(dst));
                }
            } else if (FP4) {
                for (int i = 0; i < 4; i++)
                    if (k0[u] + 2 * i < K) dst[i] = (uint8_t)(q[0] >> (8 * i)) & (k0[u] + 2 * i + 1 < K ? 0xFF : 0x0F);
            } else {
                for (int i = 0; i < 8; i++)
                    if (k0[u] + i < K) dst[i] = (uint8_t)(q[i >> 2] >> (8 * (i & 3)));
            }
        }
        if (blk < nblk) {
            uint8_t *srow = scales + (size_t)row[u] * sld;
            if ((lane & 3) == 0) srow[blk] = (uint8_t)sbyte;
            if ((lane & 3) == 1 && blk == nblk - 1 && sld != nblk) srow[nblk] = 127;  // even padding, 1.0
        }
    }
}

template <int FMT, int RND, bool HWCVT>
static int launch_rows(const void *x, void *payload, void *scales, int64_t m, int64_t k, hipStream_t stream)
{
    const bool fp4 = FMT == CCH_FMT_E2M1;
    const int64_t nblk = (k + 31) / 32, sld = 2 * ((nblk + 1) / 2), pld = fp4 ? (k + 1) / 2 : k;
    const int64_t wpr = (nblk * 4 + 63) / 64;
    const bool vec = (k % 8 == 0) && aligned(x, 16) && aligned(payload, 8);
    const int64_t rows_per_launch = std::max<int64_t>(1, (int64_t)(1 << 30) / wpr);
    for (int64_t r0 = 0; r0 < m; r0 += rows_per_launch) {
        const int64_t rows = std::min(rows_per_launch, m - r0);
        const int64_t total_ws = rows * wpr;
        const int64_t waves = (total_ws + QUANT_UNROLL - 1) / QUANT_UNROLL;
        const unsigned grid = (unsigned)((waves + QUANT_THREADS / 64 - 1) / (QUANT_THREADS / 64));
        const uint16_t *xs = static_cast<const uint16_t *>(x) + r0 * k;
        uint8_t *ps = static_cast<uint8_t *>(payload) + r0 * pld;
        uint8_t *ss = static_cast<uint8_t *>(scales) + r0 * sld;
        if (vec)
            hipLaunchKernelGGL((mx_quant_rows_kernel<FMT, RND, HWCVT, true>), dim3(grid), dim3(QUANT_THREADS), 0, stream,
                               xs, ps, ss, (int)rows, (int)k, (int)nblk, (int)sld, (int)pld, (int)wpr, (int)total_ws);
        else
            hipLaunchKernelGGL((mx_quant_rows_kernel<FMT, RND, HWCVT, false>), dim3(grid), dim3(QUANT_THREADS), 0,
                               stream, xs, ps, ss, (int)rows, (int)k, (int)nblk, (int)sld, (int)pld, (int)wpr,
                               (int)total_ws);
        int rc = launch_status("mx_quant_rows_kernel");
        if (rc) return rc;
    }
    return CCH_OK;
}


// Quantiser for a right-hand operand b [K,N] with MX blocks running down K.  One thread owns
// two adjacent columns of one 32-row block: 32 coalesced 4-byte loads, results written in
// either boundary layout.  Input preparation, not a hot path.
template <int FMT, int RND>
__global__ __launch_bounds__(256) void mx_quant_b_kernel(const uint32_t *__restrict__ b, uint8_t *__restrict__ payload,
                                                         uint8_t *__restrict__ scales, int K, int N, int trans_b)
{
    using T = FmtTraits<FMT>;
    constexpr bool FP4 = FMT == CCH_FMT_E2M1;
    const int np = blockIdx.x * 256 + threadIdx.x;  // column pair
    const int kb = blockIdx.y;
    if (np * 2 >= N) return;
    const int sld = K / 32;
    uint32_t w[32];
    uint32_t m0 = 0, m1 = 0;
#pragma unroll
    for (int i = 0; i < 32; i++) {
        w[i] = b[((size_t)(kb * 32 + i) * N) / 2 + np];
        m0 = max(m0, w[i] & 0x7FFFu);
        m1 = max(m1, (w[i] >> 16) & 0x7FFFu);
    }
    int e0, e1;
    bool n0, n1;
    const uint32_t s0 = shared_exp_byte<FMT>(m0, e0, n0), s1 = shared_exp_byte<FMT>(m1, e1, n1);
    const float i0 = pow2i(-e0), i1 = pow2i(-e1);
    uint32_t q0[32], q1[32];
#pragma unroll
    for (int i = 0; i < 32; i++) {
        q0[i] = n0 ? T::NANCODE : encode_small<FMT, RND>(__uint_as_float(w[i] << 16) * i0);
        q1[i] = n1 ? T::NANCODE : encode_small<FMT, RND>(__uint_as_float(w[i] & 0xFFFF0000u) * i1);
    }
    const int n = np * 2;
    if (!trans_b) {
#pragma unroll
        for (int i = 0; i < 32; i++) {
            const size_t k = (size_t)kb * 32 + i;
            if (FP4) payload[k * (N / 2) + np] = (uint8_t)(q0[i] | (q1[i] << 4));
            else *reinterpret_cast<uint16_t *>(payload + k * N + n) = (uint16_t)(q0[i] | (q1[i] << 8));
        }
        uint8_t *sp = scales + ((size_t)(kb >> 1) * N + n) * 2 + (kb & 1);
        sp[0] = (uint8_t)s0;
        sp[2] = (uint8_t)s1;
    } else {
        if (FP4) {
            uint8_t *d0 = payload + (size_t)n * (K / 2) + kb * 16, *d1 = d0 + K / 2;
#pragma unroll
            for (int i = 0; i < 16; i++) {
                d0[i] = (uint8_t)(q0[2 * i] | (q0[2 * i + 1] << 4));
                d1[i] = (uint8_t)(q1[2 * i] | (q1[2 * i + 1] << 4));
            }
        } else {
            uint8_t *d0 = payload + (size_t)n * K + kb * 32, *d1 = d0 + K;
#pragma unroll
            for (int i = 0; i < 32; i++) {
                d0[i] = (uint8_t)q0[i];
                d1[i] = (uint8_t)q1[i];
            }
        }
        scales[(size_t)n * sld + kb] = (uint8_t)s0;
        scales[(size_t)(n + 1) * sld + kb] = (uint8_t)s1;
    }
}

template <int FMT, int RND>
static int launch_b(const void *b, void *payload, void *scales, int64_t k, int64_t n, int trans_b, hipStream_t stream)
{
    dim3 grid((unsigned)((n / 2 + 255) / 256), (unsigned)(k / 32));
    hipLaunchKernelGGL((mx_quant_b_kernel<FMT, RND>), grid, dim3(256), 0, stream, static_cast<const uint32_t *>(b),
                       static_cast<uint8_t *>(payload), static_cast<uint8_t *>(scales), (int)k, (int)n, trans_b);
    return launch_status("mx_quant_b_kernel");
}

}  // namespace cch

extern "C" int cch_mx_quant_rows(const void *x, void *payload, void *scales, int64_t m, int64_t k, int fmt,
                                 int rounding, void *stream)
{
    using namespace cch;
    CCH_REQUIRE(m >= 0 && k >= 0, "cch_mx_quant_rows: negative shape m=%lld k=%lld", (long long)m, (long long)k);
    CCH_REQUIRE(k < (int64_t)1 << 30, "cch_mx_quant_rows: k=%lld too large", (long long)k);
    CCH_REQUIRE(rounding == CCH_ROUND_RNE || rounding == CCH_ROUND_LUT, "cch_mx_quant_rows: rounding %d", rounding);
    if (m == 0 || k == 0) return CCH_OK;
    CCH_REQUIRE(x && payload && scales, "cch_mx_quant_rows: null pointer");
    hipStream_t s = static_cast<hipStream_t>(stream);
    const bool lut = rounding == CCH_ROUND_LUT;
    switch (fmt) {
        case CCH_FMT_E4M3:
            return lut ? launch_rows<CCH_FMT_E4M3, CCH_ROUND_LUT, false>(x, payload, scales, m, k, s)
                       : launch_rows<CCH_FMT_E4M3, CCH_ROUND_RNE, true>(x, payload, scales, m, k, s);
        case CCH_FMT_E5M2:
            return lut ? launch_rows<CCH_FMT_E5M2, CCH_ROUND_LUT, false>(x, payload, scales, m, k, s)
                       : launch_rows<CCH_FMT_E5M2, CCH_ROUND_RNE, false>(x, payload, scales, m, k, s);
        case CCH_FMT_E2M1:
            return lut ? launch_rows<CCH_FMT_E2M1, CCH_ROUND_LUT, false>(x, payload, scales, m, k, s)
                       : launch_rows<CCH_FMT_E2M1, CCH_ROUND_RNE, false>(x, payload, scales, m, k, s);
        default:
            return fail(CCH_EINVAL, "cch_mx_quant_rows: unknown format %d", fmt);
    }
}

// Test hook: the same E4M3 round-to-nearest-even quantiser through the integer encoder instead
// of the hardware cast, so the two can be compared bit for bit on the device.
extern "C" int cch_mx_quant_rows_e4m3_int(const void *x, void *payload, void *scales, int64_t m, int64_t k,
                                           void *stream)
{
    using namespace cch;
    if (m <= 0 || k <= 0) return CCH_OK;
    CCH_REQUIRE(x && payload && scales, "cch_mx_quant_rows_e4m3_int: null pointer");
    return launch_rows<CCH_FMT_E4M3, CCH_ROUND_RNE, false>(x, payload, scales, m, k, static_cast<hipStream_t>(stream));
}

extern "C" int cch_mx_quant_b(const void *b, void *payload, void *scales, int64_t k, int64_t n, int fmt, int rounding,
                              int trans_b, void *stream)
{
    using namespace cch;
    CCH_REQUIRE(k >= 0 && n >= 0, "cch_mx_quant_b: negative shape");
    CCH_REQUIRE(k % 64 == 0 && n % 2 == 0, "cch_mx_quant_b: needs k %% 64 == 0 and n %% 2 == 0 (k=%lld n=%lld)",
                (long long)k, (long long)n);
    CCH_REQUIRE(k / 32 <= 65535 && k * n < ((int64_t)1 << 40), "cch_mx_quant_b: shape too large");
    CCH_REQUIRE(rounding == CCH_ROUND_RNE || rounding == CCH_ROUND_LUT, "cch_mx_quant_b: rounding %d", rounding);
    CCH_REQUIRE(trans_b == 0 || trans_b == 1, "cch_mx_quant_b: trans_b %d", trans_b);
    if (k == 0 || n == 0) return CCH_OK;
    CCH_REQUIRE(b && payload && scales, "cch_mx_quant_b: null pointer");
    CCH_REQUIRE(aligned(b, 4) && aligned(payload, 2), "cch_mx_quant_b: misaligned pointer");
    hipStream_t s = static_cast<hipStream_t>(stream);
    const bool lut = rounding == CCH_ROUND_LUT;
    switch (fmt) {
        case CCH_FMT_E4M3:
            return lut ? launch_b<CCH_FMT_E4M3, CCH_ROUND_LUT>(b, payload, scales, k, n, trans_b, s)
                       : launch_b<CCH_FMT_E4M3, CCH_ROUND_RNE>(b, payload, scales, k, n, trans_b, s);
        case CCH_FMT_E5M2:
            return lut ? launch_b<CCH_FMT_E5M2, CCH_ROUND_LUT>(b, payload, scales, k, n, trans_b, s)
                       : launch_b<CCH_FMT_E5M2, CCH_ROUND_RNE>(b, payload, scales, k, n, trans_b, s);
        case CCH_FMT_E2M1:
            return lut ? launch_b<CCH_FMT_E2M1, CCH_ROUND_LUT>(b, payload, scales, k, n, trans_b, s)
                       : launch_b<CCH_FMT_E2M1, CCH_ROUND_RNE>(b, payload, scales, k, n, trans_b, s);
        default:
            return fail(CCH_EINVAL, "cch_mx_quant_b: unknown format %d", fmt);
    }
}
