// Shape-agnostic GEMM path: one thread per output element, fp32 (or int32) accumulation in
// ascending k.  Used for shapes and layouts the tiled MFMA kernels do not take, and as an
// on-device cross-check of them.  Covers every format, both B layouts, groups and epilogues.
#include "common.h"
#include "gemm_common.h"
#include "mx_formats.h"

namespace cch {

__device__ __forceinline__ float decode_small(uint32_t c, int fmt)
{
    int eb, mb, bias;
    uint32_t sign;
    if (fmt == CCH_FMT_E4M3) { eb = 4; mb = 3; bias = 7; sign = c & 0x80u; c &= 0x7Fu; if (c == 0x7Fu) return __uint_as_float(0x7FC00000u); }
    else if (fmt == CCH_FMT_E5M2) { eb = 5; mb = 2; bias = 15; sign = c & 0x80u; c &= 0x7Fu; if (c >= 0x7Cu) return __uint_as_float(c == 0x7Cu ? (sign ? 0xFF800000u : 0x7F800000u) : 0x7FC00000u); }
    else { eb = 2; mb = 1; bias = 1; sign = c & 0x8u; c &= 0x7u; }
    const uint32_t e = (c >> mb) & ((1u << eb) - 1u), m = c & ((1u << mb) - 1u);
    const float v = e ? ldexpf((float)((1u << mb) + m), (int)e - bias - mb) : ldexpf((float)m, 1 - bias - mb);
    return sign ? -v : v;
}

__device__ __forceinline__ float e8m0_value(uint32_t b)
{
    if (b == 0xFFu) return __uint_as_float(0x7FC00000u);
    return b == 0 ? __uint_as_float(0x00400000u) : __uint_as_float(b << 23);  // 2^-127 is subnormal
}

template <int KIND>
__device__ __forceinline__ float dot_column(const GemmProblem &p, int row, int e, int col)
{
    const uint8_t *b = p.b + (size_t)e * p.b_stride;
    if (KIND == KIND_I8) {
        const int8_t *ar = reinterpret_cast<const int8_t *>(p.a) + (size_t)row * p.K;
        const int8_t *bi = reinterpret_cast<const int8_t *>(b);
        int acc = 0;
        for (int k = 0; k < p.K; k++) {
            const int bv = p.trans_b ? bi[(size_t)col * p.K + k] : bi[(size_t)k * p.N + col];
            acc += (int)ar[k] * bv;
        }
        return (float)acc;
    }
    const bool fp4 = KIND == KIND_F4;
    const uint8_t *sb = p.sb + (size_t)e * p.sb_stride;
    const size_t lda = fp4 ? (p.K + 1) / 2 : p.K;
    const size_t ldb = p.trans_b ? lda : (fp4 ? (size_t)(p.N + 1) / 2 : (size_t)p.N);
    float acc = 0.0f;
    for (int k = 0; k < p.K; k++) {
        uint32_t qa = p.a[(size_t)row * (p.a_pitch ? (size_t)p.a_pitch : lda) + (fp4 ? k >> 1 : k)];
        if (fp4) qa = (qa >> ((k & 1) * 4)) & 0xFu;
        uint32_t qb;
        if (p.trans_b) {
            qb = b[(size_t)col * ldb + (fp4 ? k >> 1 : k)];
            if (fp4) qb = (qb >> ((k & 1) * 4)) & 0xFu;
        } else {
            qb = b[(size_t)k * ldb + (fp4 ? col >> 1 : col)];
            if (fp4) qb = (qb >> ((col & 1) * 4)) & 0xFu;
        }
        const int kb = k >> 5;
        const uint32_t sa_b = p.sa[(size_t)row * (p.sa_pitch ? (size_t)p.sa_pitch : (size_t)p.sld) + kb];
        const uint32_t sb_b = p.trans_b ? sb[(size_t)col * p.sld + kb] : sb[((size_t)(kb >> 1) * p.N + col) * 2 + (kb & 1)];
        const float av = decode_small(qa, p.fmt) * e8m0_value(sa_b);
        const float bv = decode_small(qb, p.fmt) * e8m0_value(sb_b);
        acc += av * bv;
    }
    return acc;
}

template <int KIND, int EPI>
__global__ __launch_bounds__(256) void gemm_naive_kernel(GemmProblem p)
{
    __shared__ GroupTable tab;
    if (threadIdx.x == 0) build_group_table(tab, p.group_sizes, p.num_groups, p.T, 1);
    __syncthreads();
    const int col = blockIdx.y * 256 + threadIdx.x;
    const int row = blockIdx.x;   // rows on the grid's x axis: it takes 2^31 - 1 of them
    if (col >= p.n_out) return;
    const int e = find_group(tab, p.num_groups, row);  // bm = 1: tile rows are rows
    size_t out_row = (size_t)row;
    if (p.out_row_map) {
        // mapped output: rows of no group and rows mapped to a negative index are not written
        if (e >= p.num_groups || p.out_row_map[row] < 0 || p.out_row_map[row] >= p.out_rows) return;
        out_row = (size_t)p.out_row_map[row];
    }
    float v = 0.0f;
    if (e < p.num_groups) {
        if (EPI == EPI_SWIGLU) {
            // gate and up as the bf16 tile of the up projection, then the activation in fp32
            const float g = bf16_bits_to_f32(f32_to_bf16_bits(dot_column<KIND>(p, row, e, col)));
            const float u = bf16_bits_to_f32(f32_to_bf16_bits(dot_column<KIND>(p, row, e, col + p.n_out)));
            v = g / (1.0f + expf(-g)) * u;
        } else if (EPI == EPI_DEQUANT_SWIGLU) {
            float g = dot_column<KIND>(p, row, e, col) * p.per_ch[(size_t)e * p.N + col];
            float u = dot_column<KIND>(p, row, e, col + p.n_out) * p.per_ch[(size_t)e * p.N + col + p.n_out];
            if (p.i8_fp16_step) {
                // the reference's device hands the per-channel product on as IEEE half (gemm_common.h); the fp32 product
                // is rounded first, as the golden's two casts do (no fused product-and-convert instruction)
                asm volatile("" : "+v"(g), "+v"(u));
                g = (float)(_Float16)g;
                u = (float)(_Float16)u;
            }
            g *= p.per_tok[row];
            u *= p.per_tok[row];
            v = g * (1.0f / (1.0f + expf(-g))) * u;
        } else if (EPI == EPI_DEQUANT) {
            const float a = dot_column<KIND>(p, row, e, col);
            if (p.i8_fp16_step) {
                float prod = a * p.per_ch[(size_t)e * p.N + col];
                asm volatile("" : "+v"(prod));
                v = (float)(_Float16)prod * p.per_tok[row];
            } else {
                v = a * p.per_tok[row] * p.per_ch[(size_t)e * p.N + col];
            }
        } else {
            v = dot_column<KIND>(p, row, e, col);
        }
    }
    p.out[out_row * p.n_out + col] = p.out_fp16 ? __builtin_bit_cast(uint16_t, (_Float16)v) : (uint16_t)f32_to_bf16_bits(v);
}

// The grouped GEMMs with SwiGLU (int8 with dequantisation, or MX) whose activation leaves MX-quantised:
// what the row quantiser makes of the bf16 output of the kernel above, without the bf16 tensor in
// between.  32 neighbouring lanes hold one block of a row (the last block of a row may be shorter).
template <int KIND, int FMT>
__global__ __launch_bounds__(256) void gemm_naive_swiglu_mx_kernel(GemmProblem p)
{
    using T = FmtTraits<FMT>;
    __shared__ GroupTable tab;
    if (threadIdx.x == 0) build_group_table(tab, p.group_sizes, p.num_groups, p.T, 1);
    __syncthreads();
    const int col = blockIdx.y * 256 + threadIdx.x;
    const int row = blockIdx.x;
    const bool live = col < p.n_out;
    const int e = find_group(tab, p.num_groups, row);
    float v = 0.0f;
    if (live && e < p.num_groups) {
        if (KIND == KIND_I8) {
            float g = dot_column<KIND>(p, row, e, col) * p.per_ch[(size_t)e * p.N + col];
            float u = dot_column<KIND>(p, row, e, col + p.n_out) * p.per_ch[(size_t)e * p.N + col + p.n_out];
            if (p.i8_fp16_step) {
                asm volatile("" : "+v"(g), "+v"(u));
                g = (float)(_Float16)g;
                u = (float)(_Float16)u;
            }
            g *= p.per_tok[row];
            u *= p.per_tok[row];
            v = g * (1.0f / (1.0f + expf(-g))) * u;
        } else {
            const float g = bf16_bits_to_f32(f32_to_bf16_bits(dot_column<KIND>(p, row, e, col)));
            const float u = bf16_bits_to_f32(f32_to_bf16_bits(dot_column<KIND>(p, row, e, col + p.n_out)));
            v = g / (1.0f + expf(-g)) * u;
        }
    }
    const uint32_t h = live ? f32_to_bf16_bits(v) : 0u;
    uint32_t amax = h & 0x7FFFu;
#pragma unroll
    for (int d = 1; d < 32; d <<= 1) amax = max(amax, (uint32_t)__shfl_xor((int)amax, d, 32));
    int ex;
    bool is_nan;
    const uint32_t sbyte = shared_exp_byte<FMT>(amax, ex, is_nan);
    // 2^-ex in two exact factors (2^-127 is no normal float)
    const float y = bf16_bits_to_f32(h) * pow2i(-min(ex, 126)) * (ex > 126 ? 0.5f : 1.0f);
    const uint32_t code = is_nan ? T::NANCODE : encode_small<FMT, CCH_ROUND_RNE>(y);
    uint8_t *payload = reinterpret_cast<uint8_t *>(p.out);
    if constexpr (is_fp4_v<FMT>) {
        const uint32_t hi = (uint32_t)__shfl_down((int)code, 1, 32);
        if (live && (col & 1) == 0) payload[((size_t)row * p.n_out + col) >> 1] = (uint8_t)(code | ((col + 1 < p.n_out ? hi : 0u) << 4));
    } else {
        if (live) payload[(size_t)row * p.n_out + col] = (uint8_t)code;
    }
    if (live && (col & 31) == 0) {
        p.out_scales[(size_t)row * p.mx_out_sld + (col >> 5)] = (uint8_t)sbyte;
        const int nblk = (p.n_out + 31) >> 5;
        if ((nblk & 1) && (col >> 5) == nblk - 1) p.out_scales[(size_t)row * p.mx_out_sld + nblk] = 127;
    }
}

template <int KIND, int EPI>
static int launch_naive_t(const GemmProblem &p, hipStream_t stream)
{
    if (p.T == 0 || p.n_out == 0) return CCH_OK;
    if ((p.n_out + 255) / 256 > 65535) return fail(CCH_ENOSUP, "generic GEMM path takes at most 65535 * 256 output columns per call (got %d)", p.n_out);
    dim3 grid((unsigned)p.T, (unsigned)((p.n_out + 255) / 256));
    hipLaunchKernelGGL((gemm_naive_kernel<KIND, EPI>), grid, dim3(256), 0, stream, p);
    return launch_status("gemm_naive_kernel");
}

int launch_gemm_naive(const GemmProblem &p, int kind, int epi, hipStream_t stream)
{
    if (p.mx_out) {
        if (epi != EPI_DEQUANT_SWIGLU && epi != EPI_SWIGLU) return fail(CCH_ENOSUP, "MX-quantised output exists for the SwiGLU epilogues only");
        if (p.T == 0 || p.n_out == 0) return CCH_OK;
        if ((p.n_out + 255) / 256 > 65535) return fail(CCH_ENOSUP, "generic GEMM path takes at most 65535 * 256 output columns per call (got %d)", p.n_out);
        dim3 grid((unsigned)p.T, (unsigned)((p.n_out + 255) / 256));
#define CCH_NAIVE_MX_OUT(K)                                                                                                                        \
    do {                                                                                                                                           \
        if (p.mx_out_fmt == CCH_FMT_E4M3) hipLaunchKernelGGL((gemm_naive_swiglu_mx_kernel<K, CCH_FMT_E4M3>), grid, dim3(256), 0, stream, p);      \
        else if (p.mx_out_fmt == CCH_FMT_E5M2) hipLaunchKernelGGL((gemm_naive_swiglu_mx_kernel<K, CCH_FMT_E5M2>), grid, dim3(256), 0, stream, p); \
        else hipLaunchKernelGGL((gemm_naive_swiglu_mx_kernel<K, CCH_FMT_E2M1>), grid, dim3(256), 0, stream, p);                                   \
    } while (0)
        if (kind == KIND_I8) CCH_NAIVE_MX_OUT(KIND_I8);
        else if (kind == KIND_F8) CCH_NAIVE_MX_OUT(KIND_F8);
        else CCH_NAIVE_MX_OUT(KIND_F4);
#undef CCH_NAIVE_MX_OUT
        return launch_status("gemm_naive_swiglu_mx_kernel");
    }
    if (kind == KIND_I8 && epi == EPI_DEQUANT) return launch_naive_t<KIND_I8, EPI_DEQUANT>(p, stream);
    if (kind == KIND_I8 && epi == EPI_DEQUANT_SWIGLU) return launch_naive_t<KIND_I8, EPI_DEQUANT_SWIGLU>(p, stream);
    if (kind == KIND_F8 && epi == EPI_PLAIN) return launch_naive_t<KIND_F8, EPI_PLAIN>(p, stream);
    if (kind == KIND_F4 && epi == EPI_PLAIN) return launch_naive_t<KIND_F4, EPI_PLAIN>(p, stream);
    if (kind == KIND_F8 && epi == EPI_SWIGLU) return launch_naive_t<KIND_F8, EPI_SWIGLU>(p, stream);
    if (kind == KIND_F4 && epi == EPI_SWIGLU) return launch_naive_t<KIND_F4, EPI_SWIGLU>(p, stream);
    return fail(CCH_ENOSUP, "no generic GEMM kernel for kind %d with epilogue %d", kind, epi);
}

}  // namespace cch
