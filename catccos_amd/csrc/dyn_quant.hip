// Per-token dynamic int8 quantiser with row gather: the step that turns bf16 tokens into the
// int8 rows and per-token scales the MoE grouped GEMM consumes.  Streaming, HBM-bound: one wave
// owns one output row (two or four waves share a row longer than 4096 columns), keeps it in
// registers (16-byte non-temporal loads, up to 16384 columns), reduces |x| across the wave(s), and
// writes 8 int8 per lane per chunk.  Longer rows are read twice.
//
// Follows MoeV2GatherDynamicQuant::Compute
// (examples/aux_ops/moe_init_routing_quant_v2/moe_v2_gather_dynamic_quant.h:117-150) and its
// gather loop (:229-236); CCH_DQ_GOLDEN follows the generator's golden
// (examples/utils/gen_data_dispatch_gmm_dequant_swiglu.py:275-280).  With a smoothing vector
// (:127-130; one for all rows :170-174, or one per expert :241) the registers hold the fp32
// products instead of the bf16 pairs.
#include "common.h"
#include "mx_formats.h"

namespace cch {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef unsigned short u16x2 __attribute__((ext_vector_type(2)));

constexpr int DQ_THREADS = 256;   // 4 rows per workgroup
constexpr int DQ_MAX_CHUNKS = 32; // 32 x 512 columns held in registers, by up to four waves

__device__ __forceinline__ uint32_t wave_max_u32(uint32_t v)
{
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) v = max(v, (uint32_t)__shfl_xor((int)v, off, 64));
    return v;
}

// Correctly rounded a / b for a divisor shared by a whole row.  With y = RN(1/b), q0 = RN(a*y)
// and the exact remainder r = a - b*q0 (one FMA), RN(q0 + r*y) is the correctly rounded quotient
// (Markstein) provided b's significand is not all ones and nothing leaves the normal range; the
// caller falls back to the division instruction sequence otherwise (`fast` false).
struct RowDivisor {
    float b, y;
    bool fast;
};
__device__ __forceinline__ RowDivisor make_divisor(float b)
{
    RowDivisor d;
    d.b = b;
    d.y = 1.0f / b;
    const uint32_t bits = __float_as_uint(b);
    const int e = (int)((bits >> 23) & 0xFF);
    d.fast = e > 40 && e < 215 && (bits & 0x7FFFFFu) != 0x7FFFFFu;
    return d;
}
__device__ __forceinline__ float row_div(float a, const RowDivisor &d)
{
    if (!d.fast) return a / d.b;   // wave-uniform
    const float q0 = a * d.y;
    const float r = __builtin_fmaf(-d.b, q0, a);
    return __builtin_fmaf(r, d.y, q0);
}

// One value: MODE 0 = fp32 divide by the scale, truncate to half, round halves away from zero;
// MODE 1 = rint(x * 127 / amax).  `d` divides by the scale (MODE 0) or by amax (MODE 1).
template <int MODE>
__device__ __forceinline__ int quant_one(float v, const RowDivisor &d)
{
    float y;
    if (MODE == 0) {
        float t = row_div(v, d);
        // |t| <= 127.000008: a half in that range keeps 10 fraction bits of the fp32 pattern; values
        // below the half normal range end up as 0 either way
        t = __uint_as_float(__float_as_uint(t) & 0xFFFFE000u);
        y = truncf(t + copysignf(0.5f, t));
    } else {
        y = rintf(row_div(v * 127.0f, d));
    }
    return (int)y;   // |y| <= 127: |x| <= amax, and the quotient of amax itself rounds to 127
}

// WPR waves share a row (CHUNKS is then the share of one wave): long rows keep few enough
// registers per wave for full occupancy, and the grid has WPR times as many, shorter, pieces of
// work.  The partial maxima meet in LDS.  SMOOTH: every element is first multiplied by the row's
// fp32 smoothing vector (vector `smooth_rows[row]`, or vector 0 without that list).
template <int MODE, int CHUNKS, int WPR = 1, bool SMOOTH = false>
__global__ __launch_bounds__(DQ_THREADS) void dyn_quant_rows_kernel(const uint16_t *__restrict__ x, const int32_t *__restrict__ src,
                                                                   const float *__restrict__ smooth,
                                                                   const int32_t *__restrict__ smooth_rows, int num_smooth,
                                                                   int8_t *__restrict__ q, float *__restrict__ scale, int rows_in,
                                                                   int T, int K, int topk)
{
    constexpr int ROWS_PER_WG = DQ_THREADS / 64 / WPR;
    constexpr int NW = SMOOTH ? 8 : 4;   // registers per chunk: fp32 products or bf16 pairs
    __shared__ uint32_t part[DQ_THREADS / 64];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const int share = wave % WPR;   // which part of the row this wave owns
    const int row = __builtin_amdgcn_readfirstlane((int)(blockIdx.x * ROWS_PER_WG + wave / WPR));
    if (WPR == 1 && row >= T) return;
    const bool present = row < T;   // WPR > 1: every wave reaches the barrier
    int r = present ? row : -1;
    if (src && present) {
        const int s = src[row];
        r = s < 0 ? -1 : s / topk;
    }
    int sv = 0;
    if (SMOOTH && smooth_rows && present) sv = smooth_rows[row];
    int8_t *qo = q + (size_t)(present ? row : 0) * K;
    const bool live = r >= 0 && r < rows_in && (!SMOOTH || (sv >= 0 && sv < num_smooth));   // wave-uniform
    const uint16_t *xr = x + (size_t)(live ? r : 0) * K;
    const float *sm = SMOOTH ? smooth + (size_t)(live ? sv : 0) * K : nullptr;
    const bool vec = (K % 8 == 0) && ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(q)) % 16 == 0) &&
                     (!SMOOTH || reinterpret_cast<uintptr_t>(smooth) % 16 == 0);

    if (CHUNKS > 0 && vec) {
        // register path
        uint32_t w[CHUNKS > 0 ? CHUNKS : 1][NW];
        uint32_t m = 0;
#pragma unroll
        for (int c = 0; c < CHUNKS; c++) {
            const int k0 = ((share * CHUNKS + c) * 64 + lane) * 8;
            u32x4 v = {0, 0, 0, 0};
            if (live && k0 < K) v = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(xr + k0));
            if constexpr (SMOOTH) {
                f32x4 s0 = {0, 0, 0, 0}, s1 = {0, 0, 0, 0};
                if (live && k0 < K) {
                    s0 = *reinterpret_cast<const f32x4 *>(sm + k0);
                    s1 = *reinterpret_cast<const f32x4 *>(sm + k0 + 4);
                }
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    const float lo = __uint_as_float(v[i] << 16), hi = __uint_as_float(v[i] & 0xFFFF0000u);
                    const float sl = i < 2 ? s0[2 * i] : s1[2 * i - 4], sh = i < 2 ? s0[2 * i + 1] : s1[2 * i - 3];
                    w[c][2 * i] = __float_as_uint(lo * sl);
                    w[c][2 * i + 1] = __float_as_uint(hi * sh);
                    m = max(m, max(w[c][2 * i] & 0x7FFFFFFFu, w[c][2 * i + 1] & 0x7FFFFFFFu));
                }
            } else {
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    w[c][i] = v[i];
                    const u16x2 a = __builtin_bit_cast(u16x2, v[i] & 0x7FFF7FFFu);
                    m = max(m, max((uint32_t)a[0], (uint32_t)a[1]));
                }
            }
        }
        m = wave_max_u32(m);   // the largest |value| pattern is the largest magnitude
        if constexpr (WPR > 1) {
            if (lane == 0) part[wave] = m;
            __syncthreads();
#pragma unroll
            for (int h = 0; h < WPR; h++) m = max(m, part[wave - share + h]);
            if (!present) return;
        }
        const float amax = __uint_as_float(SMOOTH ? m : m << 16);
        const bool zero = !(amax > 0.0f);
        const float sc = zero ? 0.0f : amax / 127.0f;
        if (lane == 0 && share == 0) scale[row] = sc;
        const RowDivisor dv = make_divisor(zero ? 1.0f : (MODE == 0 ? sc : amax));
#pragma unroll
        for (int c = 0; c < CHUNKS; c++) {
            const int k0 = ((share * CHUNKS + c) * 64 + lane) * 8;
            if (k0 >= K) continue;
            uint32_t o[2] = {0, 0};
            if (!zero) {
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    const float v0 = __uint_as_float(SMOOTH ? w[c][(2 * i) % NW] : w[c][i % NW] << 16);
                    const float v1 = __uint_as_float(SMOOTH ? w[c][(2 * i + 1) % NW] : w[c][i % NW] & 0xFFFF0000u);
                    const int q0 = quant_one<MODE>(v0, dv);
                    const int q1 = quant_one<MODE>(v1, dv);
                    o[i >> 1] |= ((uint32_t)(q0 & 0xFF) | ((uint32_t)(q1 & 0xFF) << 8)) << (16 * (i & 1));
                }
            }
            __builtin_nontemporal_store((u32x2){o[0], o[1]}, reinterpret_cast<u32x2 *>(qo + k0));
        }
    } else {
        // two passes over the row, any K and alignment
        auto value = [&](int k) {
            const float v = __uint_as_float((uint32_t)xr[k] << 16);
            return SMOOTH ? v * sm[k] : v;
        };
        uint32_t m = 0;
        if (live)
            for (int k = lane; k < K; k += 64) m = max(m, __float_as_uint(value(k)) & 0x7FFFFFFFu);
        m = wave_max_u32(m);
        const float amax = __uint_as_float(m);
        const bool zero = !(amax > 0.0f);
        const float sc = zero ? 0.0f : amax / 127.0f;
        if (lane == 0) scale[row] = sc;
        const RowDivisor dv = make_divisor(zero ? 1.0f : (MODE == 0 ? sc : amax));
        for (int k = lane; k < K; k += 64) qo[k] = zero ? (int8_t)0 : (int8_t)quant_one<MODE>(value(k), dv);
    }
}

template <int MODE, bool SMOOTH>
static int launch_dq(const void *x, const int32_t *src, const float *smooth, const int32_t *smooth_rows, int num_smooth, void *q,
                     float *scale, int64_t rows_in, int64_t t, int64_t k, int topk, hipStream_t stream)
{
    // rows that cannot be moved 16 bytes at a time take the two-pass path
    const bool vec = (k % 8 == 0) && aligned(x, 16) && aligned(q, 16) && (!SMOOTH || aligned(smooth, 16));
    const int chunks = vec ? (int)((k + 511) / 512) : DQ_MAX_CHUNKS + 1;
#define CCH_DQ_LAUNCH(C, W)                                                                                                \
    do {                                                                                                                   \
        constexpr int rows_per_wg = DQ_THREADS / 64 / W;                                                                   \
        const unsigned grid = (unsigned)((t + rows_per_wg - 1) / rows_per_wg);                                             \
        hipLaunchKernelGGL((dyn_quant_rows_kernel<MODE, C, W, SMOOTH>), dim3(grid), dim3(DQ_THREADS), 0, stream,           \
                           static_cast<const uint16_t *>(x), src, smooth, smooth_rows, num_smooth, static_cast<int8_t *>(q), \
                           scale, (int)rows_in, (int)t, (int)k, topk);                                                     \
    } while (0)
    // four chunks per wave where the row allows: few registers (full occupancy) and many short
    // pieces of work measured fastest (5.8 TB/s at K = 7168 against 5.4 with two waves per row
    // and 5.0 with one)
    if (chunks <= 4) CCH_DQ_LAUNCH(4, 1);
    else if (chunks <= 8) CCH_DQ_LAUNCH(4, 2);
    else if (chunks <= 16) CCH_DQ_LAUNCH(4, 4);
    else if (chunks <= 32) CCH_DQ_LAUNCH(8, 4);
    else CCH_DQ_LAUNCH(0, 1);
#undef CCH_DQ_LAUNCH
    return launch_status("dyn_quant_rows_kernel");
}

static int dyn_quant_entry(const char *who, const void *x, const int32_t *src_rows, const float *smooth, const int32_t *smooth_rows,
                           int64_t num_smooth, void *q, float *scale, int64_t rows_in, int64_t t, int64_t k, int topk, int mode,
                           void *stream)
{
    CCH_REQUIRE(rows_in >= 0 && t >= 0 && k >= 0, "%s: negative shape", who);
    CCH_REQUIRE(rows_in < ((int64_t)1 << 31) && t < ((int64_t)1 << 31) && k < ((int64_t)1 << 31), "%s: shape too large", who);
    CCH_REQUIRE(topk >= 1, "%s: topk %d", who, topk);
    CCH_REQUIRE(mode == CCH_DQ_DEVICE || mode == CCH_DQ_GOLDEN, "%s: mode %d", who, mode);
    CCH_REQUIRE(smooth == nullptr || (num_smooth >= 1 && num_smooth < ((int64_t)1 << 31)), "%s: num_smooth %lld", who,
                (long long)num_smooth);
    CCH_REQUIRE(smooth != nullptr || smooth_rows == nullptr, "%s: smooth_rows without smooth", who);
    if (t == 0) return CCH_OK;
    CCH_REQUIRE(q != nullptr || k == 0, "%s: null output", who);
    CCH_REQUIRE(scale != nullptr, "%s: null scale", who);
    CCH_REQUIRE(x != nullptr || rows_in == 0 || k == 0, "%s: null input", who);
    CCH_REQUIRE(src_rows != nullptr || t <= rows_in, "%s: %lld output rows from %lld input rows without a row map", who,
                (long long)t, (long long)rows_in);
    hipStream_t s = static_cast<hipStream_t>(stream);
    const int ns = (int)num_smooth;
    if (smooth)
        return mode == CCH_DQ_DEVICE ? launch_dq<0, true>(x, src_rows, smooth, smooth_rows, ns, q, scale, rows_in, t, k, topk, s)
                                     : launch_dq<1, true>(x, src_rows, smooth, smooth_rows, ns, q, scale, rows_in, t, k, topk, s);
    return mode == CCH_DQ_DEVICE ? launch_dq<0, false>(x, src_rows, nullptr, nullptr, 0, q, scale, rows_in, t, k, topk, s)
                                 : launch_dq<1, false>(x, src_rows, nullptr, nullptr, 0, q, scale, rows_in, t, k, topk, s);
}

}  // namespace cch

extern "C" int cch_dyn_quant_i8_rows(const void *x, const int32_t *src_rows, void *q, float *scale, int64_t rows_in, int64_t t,
                                     int64_t k, int topk, int mode, void *stream)
{
    return cch::dyn_quant_entry("cch_dyn_quant_i8_rows", x, src_rows, nullptr, nullptr, 0, q, scale, rows_in, t, k, topk, mode, stream);
}

extern "C" int cch_dyn_quant_i8_rows_smooth(const void *x, const int32_t *src_rows, const float *smooth, const int32_t *smooth_rows,
                                            int64_t num_smooth, void *q, float *scale, int64_t rows_in, int64_t t, int64_t k,
                                            int topk, int mode, void *stream)
{
    CCH_REQUIRE(smooth != nullptr, "cch_dyn_quant_i8_rows_smooth: null smooth");
    return cch::dyn_quant_entry("cch_dyn_quant_i8_rows_smooth", x, src_rows, smooth, smooth_rows, num_smooth, q, scale, rows_in, t, k,
                                topk, mode, stream);
}
