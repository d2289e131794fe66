/*
 * CPU oracle for the per-rank compute half of five CATCCOS fused operators.
 *
 * THIS IS TEST INFRASTRUCTURE, NOT PRODUCT CODE.  Only tests, the smoke check
 * and the benchmark's cpu_baseline leg may load it.  It restates, in plain C,
 * the arithmetic of the reference's Python golden generators (paths relative to
 * the reference tree):
 *
 *   formats / MX block quantiser  examples/utils/gen_mx_quant_allgather_data.py
 *                                 :41-73 (emax, max), :79-128 (FP8 tables),
 *                                 :168-189 (E8M0 exponent), :198-247 (table
 *                                 rounding), :255-313 (FP8 rows), :352-449
 *                                 (FP4 table, nibble packing, FP4 rows),
 *                                 :497-503 (bf16 rounding)
 *   int8 GEMM + dequant           examples/utils/gen_quant_data_mmdqrs.py:76-79
 *   grouped int8 + SwiGLU         examples/utils/gen_data_dispatch_gmm_dequant_swiglu.py
 *                                 :269-273 (swiglu), :298-320 (grouped GEMM,
 *                                 per-channel, fp16 step, per-token, swiglu)
 *   MX GEMM / grouped MX GEMM     examples/ascend950_mxfp8_matmul_reduce_scatter/scripts/
 *                                 gen_data_mxfp8_mmrs.py:299-356 and
 *                                 examples/utils/gen_data_fp4_mx_alltoallv_gmm.py
 *                                 :522-545 (nibbles), :586-620 (B scale layout),
 *                                 :724-734 (grouped matmul)
 *   token prefix sums             include/catccos/comm/block/comm_block_scheduler_alltoallv_gmm.hpp
 *                                 :92-159
 *   grouped tile order            include/catccos/dgemm/block/block_scheduler_alltoallv_allgather.hpp
 *                                 :122-168 and include/catccos/catccos.hpp:141-163
 *
 * Parity status of each function is recorded next to it ("pinned by ...").
 * Functions never pinned by an independent check would say "parity unpinned";
 * none do at present except where marked.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#define ORC_FMT_E4M3 0
#define ORC_FMT_E5M2 1
#define ORC_FMT_E2M1 2
#define ORC_FMT_E1M2 3
#define ORC_IS_FP4(fmt) ((fmt) == ORC_FMT_E2M1 || (fmt) == ORC_FMT_E1M2)
/* rounding rule of the payload cast */
#define ORC_ROUND_RNE 0 /* nearest, ties to even code, sign of zero kept      */
#define ORC_ROUND_LUT 1 /* nearest, ties to the smaller magnitude, zero is +0 */

/* ------------------------------------------------------------------ bf16 */

/* pinned by: torch.bfloat16 casts over random and special values */
float orc_bf16_to_f32(uint16_t h)
{
    uint32_t u = (uint32_t)h << 16;
    float f;
    memcpy(&f, &u, 4);
    return f;
}

/* gen_mx_quant_allgather_data.py:497-503; NaN kept quiet as utils.py:68-87 */
uint16_t orc_f32_to_bf16(float f)
{
    uint32_t u;
    memcpy(&u, &f, 4);
    if ((u & 0x7F800000u) == 0x7F800000u && (u & 0x007FFFFFu)) return (uint16_t)((u >> 16) | 0x0040u);
    u += 0x7FFFu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}

/* ------------------------------------------------------- format decoders */

/* Value of a small-float code with `eb` exponent bits, `mb` mantissa bits. */
static float small_decode(uint32_t mag, int eb, int mb, int bias)
{
    uint32_t e = (mag >> mb) & ((1u << eb) - 1u);
    uint32_t m = mag & ((1u << mb) - 1u);
    if (e == 0) return ldexpf((float)m, 1 - bias - mb);
    return ldexpf((float)((1u << mb) + m), (int)e - bias - mb);
}

/* E4M3 "fn": 0x7F / 0xFF are NaN, no infinities.
 * pinned by: torch.float8_e4m3fn over all 256 codes */
float orc_e4m3_decode(uint8_t c)
{
    uint32_t mag = c & 0x7Fu;
    float v = (mag == 0x7Fu) ? NAN : small_decode(mag, 4, 3, 7);
    return (c & 0x80u) ? -v : v;
}

/* E5M2: IEEE-like, exponent 31 is Inf/NaN.
 * pinned by: torch.float8_e5m2 over all 256 codes */
float orc_e5m2_decode(uint8_t c)
{
    uint32_t mag = c & 0x7Fu;
    float v;
    if (mag == 0x7Cu) v = INFINITY;
    else if (mag > 0x7Cu) v = NAN;
    else v = small_decode(mag, 5, 2, 15);
    return (c & 0x80u) ? -v : v;
}

/* E2M1 nibble: magnitudes {0,.5,1,1.5,2,3,4,6}.
 * pinned by: the closed list in gen_data_fp4_mx_alltoallv_gmm.py:99-129 */
float orc_e2m1_decode(uint8_t nib)
{
    float v = small_decode(nib & 7u, 2, 1, 1);
    return (nib & 8u) ? -v : v;
}

/* E1M2 nibble: magnitudes {0,.25,.5,.75,1,1.25,1.5,1.75}
 * (gen_mx_quant_allgather_data.py:65-72 with the table builder :352-375: one exponent bit,
 * two mantissa bits, bias 1).
 * pinned by: the closed list above, spelled out in the test */
float orc_e1m2_decode(uint8_t nib)
{
    float v = small_decode(nib & 7u, 1, 2, 1);
    return (nib & 8u) ? -v : v;
}

/* E8M0: 2^(b-127); 0xFF is NaN.  pinned by: torch.float8_e8m0fnu, 256 codes */
float orc_e8m0_decode(uint8_t b)
{
    if (b == 0xFFu) return NAN;
    return ldexpf(1.0f, (int)b - 127);
}

/* ------------------------------------------------------- format encoders */

typedef struct {
    int ncodes;        /* number of finite non-negative codes             */
    float val[128];    /* val[i] = magnitude of code i, ascending          */
    float maxv;
    int emax;
    uint32_t signbit;
    uint8_t nan_code;
} fmt_table;

static fmt_table g_tab[4];
static int g_tab_ready = 0;

static void build_tables(void)
{
    if (g_tab_ready) return;
    fmt_table *t = &g_tab[ORC_FMT_E4M3];
    t->ncodes = 127; /* 0x00..0x7E */
    for (int i = 0; i < 127; i++) t->val[i] = small_decode((uint32_t)i, 4, 3, 7);
    t->maxv = 448.0f; t->emax = 8; t->signbit = 0x80u; t->nan_code = 0x7Fu;
    t = &g_tab[ORC_FMT_E5M2];
    t->ncodes = 124; /* 0x00..0x7B */
    for (int i = 0; i < 124; i++) t->val[i] = small_decode((uint32_t)i, 5, 2, 15);
    t->maxv = 57344.0f; t->emax = 15; t->signbit = 0x80u; t->nan_code = 0x7Fu;
    t = &g_tab[ORC_FMT_E2M1];
    t->ncodes = 8;
    for (int i = 0; i < 8; i++) t->val[i] = small_decode((uint32_t)i, 2, 1, 1);
    t->maxv = 6.0f; t->emax = 2; t->signbit = 0x8u; t->nan_code = 0x7u; /* E2M1 has no NaN */
    t = &g_tab[ORC_FMT_E1M2];
    t->ncodes = 8;
    for (int i = 0; i < 8; i++) t->val[i] = small_decode((uint32_t)i, 1, 2, 1);
    t->maxv = 1.75f; t->emax = 0; t->signbit = 0x8u; t->nan_code = 0x7u; /* no NaN either */
#pragma omp flush
    g_tab_ready = 1;
}

/*
 * Round an already-scaled value to the nearest code of the format.
 *   clamp to +-max first (gen_mx_quant_allgather_data.py:284-285, :389),
 *   nearest table entry (:214-233); on a tie RNE takes the even code,
 *   the table rule takes the smaller magnitude (`<=`, :231);
 *   the table rule writes +0 for every zero result (:236-243), RNE keeps the sign.
 * NaN input gives the format's NaN code (E2M1: the maximum).
 * pinned by: torch float8 casts (RNE) on dense sweeps incl. all midpoints;
 *            brute-force argmin over the full table (table rule); idempotence
 *            encode(decode(c)) == c for every code.
 */
uint8_t orc_encode(float y, int fmt, int rounding)
{
    build_tables();
    const fmt_table *t = &g_tab[fmt];
    uint32_t u;
    memcpy(&u, &y, 4);
    uint32_t neg = u >> 31;
    if (y != y) return (uint8_t)((neg ? t->signbit : 0u) | t->nan_code);
    float mag = fabsf(y);
    if (mag > t->maxv) mag = t->maxv;
    /* first index with val >= mag */
    int lo = 0, hi = t->ncodes - 1;
    while (lo < hi) {
        int mid = (lo + hi) >> 1;
        if (t->val[mid] < mag) lo = mid + 1; else hi = mid;
    }
    int up = lo, dn = up > 0 ? up - 1 : 0;
    float du = t->val[up] - mag, dd = mag - t->val[dn];
    int code;
    if (dd < du) code = dn;
    else if (du < dd) code = up;
    else if (rounding == ORC_ROUND_LUT) code = dn;
    else code = (dn & 1) ? up : dn;
    if (code == 0 && rounding == ORC_ROUND_LUT) return 0;
    return (uint8_t)(code | (neg ? t->signbit : 0u));
}

float orc_decode(uint8_t c, int fmt)
{
    if (fmt == ORC_FMT_E4M3) return orc_e4m3_decode(c);
    if (fmt == ORC_FMT_E5M2) return orc_e5m2_decode(c);
    if (fmt == ORC_FMT_E1M2) return orc_e1m2_decode(c);
    return orc_e2m1_decode(c);
}

/* --------------------------------------------------------- E8M0 exponent */

/* IEEE half bits -> fp32 (exact; subnormals normalised, Inf/NaN kept). */
float orc_f16_to_f32(uint16_t h)
{
    uint32_t sign = (uint32_t)(h >> 15) << 31, ex = (h >> 10) & 0x1Fu, man = h & 0x3FFu, u;
    float f;
    if (ex == 0) {
        f = ldexpf((float)man, -24);
        memcpy(&u, &f, 4);
        u |= sign;
    } else if (ex == 31) {
        u = sign | 0x7F800000u | (man << 13);
    } else {
        u = sign | ((ex + 112u) << 23) | (man << 13);
    }
    memcpy(&f, &u, 4);
    return f;
}

/*
 * Shared exponent of one block from its absolute maximum
 * (gen_mx_quant_allgather_data.py:168-189):
 *   amax < 1e-12 -> 0 ; else clamp(floor(log2 amax) - emax, -128, 127),
 * with floor(log2) read from the biased exponent field.  The byte is e+127;
 * e = -128 cannot be written as E8M0 and is stored as byte 0 (2^-127).
 * Inf/NaN maxima give byte 0xFF (comm_block_mx_quant.hpp:505).
 * pinned by: 2^e <= amax/2^emax < 2^(e+1) over all positive bf16 maxima.
 */
int orc_shared_exp(float amax, int emax, int *is_nan)
{
    uint32_t u;
    *is_nan = 0;
    if (amax != amax || isinf(amax)) { *is_nan = 1; return 0; }
    if (amax < 1e-12f) return 0;
    memcpy(&u, &amax, 4);
    int e = (int)((u >> 23) & 0xFFu) - 127 - emax;
    if (e < -128) e = -128;
    if (e > 127) e = 127;
    return e;
}

static int fmt_emax(int fmt) { build_tables(); return g_tab[fmt].emax; }

/*
 * MX quantisation of a bf16 matrix [M,K] along its last axis, block 32
 * (gen_mx_quant_allgather_data.py:255-313 for FP8, :385-449 for FP4).
 *   payload  FP8: [M,K] bytes.  FP4: [M,ceil(K/2)] bytes, element 2j in the
 *            low nibble, 2j+1 in the high nibble (:400-411).
 *   scales   [M, 2*ceil(nblk/2)] E8M0 bytes; padding entries are 1.0 = 127
 *            (:307-311).
 * A ragged last block is zero padded (:267-273).
 * pinned by: closed forms of its parts (above), scale-shift invariance,
 *            idempotence on dequantised data (the check the reference's own
 *            run.sh performs), torch-cast cross-check on random data.
 */
static int mx_quant_rows_impl(const uint16_t *x, int in_half, int64_t M, int64_t K, int fmt, int rounding,
                              uint8_t *payload, uint8_t *scales)
{
    build_tables();
    const int64_t nblk = (K + 31) / 32;
    const int64_t sld = ((nblk + 1) / 2) * 2;
    const int64_t pld = ORC_IS_FP4(fmt) ? (K + 1) / 2 : K;
    const int emax = fmt_emax(fmt);
#pragma omp parallel for schedule(static)
    for (int64_t m = 0; m < M; m++) {
        const uint16_t *xr = x + m * K;
        uint8_t *pr = payload + m * pld;
        uint8_t *sr = scales + m * sld;
        if (ORC_IS_FP4(fmt)) memset(pr, 0, (size_t)pld);
        for (int64_t b = 0; b < sld; b++) {
            if (b >= nblk) { sr[b] = 127; continue; }
            int64_t k0 = b * 32, k1 = k0 + 32 < K ? k0 + 32 : K;
            float amax = 0.0f;
            int bad = 0;
            for (int64_t k = k0; k < k1; k++) {
                float v = fabsf(in_half ? orc_f16_to_f32(xr[k]) : orc_bf16_to_f32(xr[k]));
                if (v != v) bad = 1;
                if (v > amax) amax = v;
            }
            int is_nan;
            int e = orc_shared_exp(bad ? NAN : amax, emax, &is_nan);
            if (is_nan) {
                sr[b] = 0xFF;
            } else {
                sr[b] = (uint8_t)(e + 127 < 0 ? 0 : e + 127);
            }
            if (e < -127) e = -127;
            for (int64_t k = k0; k < k1; k++) {
                float v = in_half ? orc_f16_to_f32(xr[k]) : orc_bf16_to_f32(xr[k]);
                /* division by 2^e is exact in fp32 unless the quotient is subnormal */
                float y = is_nan ? NAN : ldexpf(v, -e);
                uint8_t q = orc_encode(y, fmt, rounding);
                if (ORC_IS_FP4(fmt)) pr[k >> 1] |= (uint8_t)(q << ((k & 1) * 4));
                else pr[k] = q;
            }
        }
    }
    return 0;
}

int orc_mx_quant_rows(const uint16_t *x, int64_t M, int64_t K, int fmt, int rounding,
                      uint8_t *payload, uint8_t *scales)
{
    return mx_quant_rows_impl(x, 0, M, K, fmt, rounding, payload, scales);
}

/*
 * The same quantiser on IEEE half input: the reference's `half` instantiation
 * widens to fp32 and takes the shared exponent from the fp32 exponent field
 * (MxQuantTraits<half>, include/catccos/epilogue/block/block_epilogue_dynamic_mx_quant.hpp:57-71:
 * CalcType float, EXP_MASK 0x7F800000, SHR_NUM 23), then scales and casts as the
 * bf16 path does.  The reference holds no golden for half input; the rule is the
 * same OCP recipe applied to the widened values.
 * pinned by: the independent numpy / torch recipe on half data incl. half
 *            subnormals as block maxima, and equality with orc_mx_quant_rows on
 *            values that both input types represent exactly.
 */
int orc_mx_quant_rows_f16(const uint16_t *x, int64_t M, int64_t K, int fmt, int rounding,
                          uint8_t *payload, uint8_t *scales)
{
    return mx_quant_rows_impl(x, 1, M, K, fmt, rounding, payload, scales);
}

/*
 * Quantise each token row once and write the same packed row
 * [payload | E8M0 scales, padded to an even count] to every routed
 * destination row (CommBlockMxQuant::QuantScatterPacked,
 * include/catccos/comm/block/comm_block_mx_quant.hpp:319-369: packedRowBytes =
 * quantBytes + AlignUp(CeilDiv(N, 32), 2); dstRow = expandedRowIdx[token *
 * topK + route], a negative dstRow is skipped).  Rows of packed_out that no
 * route names are left as they were.
 * pinned by: it is orc_mx_quant_rows (pinned above) followed by row copies;
 *            the test rebuilds the result from orc_mx_quant_rows with numpy
 *            indexing and checks untouched rows stay untouched.
 */
int orc_mx_quant_scatter_packed(const uint16_t *x, const int32_t *expanded_row_idx, int64_t tokens, int64_t K,
                                int top_k, int fmt, int rounding, uint8_t *packed_out)
{
    const int64_t nblk = (K + 31) / 32;
    const int64_t sld = ((nblk + 1) / 2) * 2;
    const int64_t pld = ORC_IS_FP4(fmt) ? (K + 1) / 2 : K;
    const int64_t row_bytes = pld + sld;
    uint8_t *row = (uint8_t *)malloc((size_t)row_bytes);
    if (!row) return -1;
    for (int64_t t = 0; t < tokens; t++) {
        orc_mx_quant_rows(x + t * K, 1, K, fmt, rounding, row, row + pld);
        for (int r = 0; r < top_k; r++) {
            const int32_t dst = expanded_row_idx[t * top_k + r];
            if (dst < 0) continue;
            memcpy(packed_out + (int64_t)dst * row_bytes, row, (size_t)row_bytes);
        }
    }
    free(row);
    return 0;
}

/*
 * MX quantisation of a bf16 matrix B [K,N] (row-major) along axis 0, as the
 * reference prepares the right-hand GEMM operand
 * (gen_data_mxfp8_mmrs.py:202-217 = quantise the transpose by rows;
 * gen_data_fp4_mx_alltoallv_gmm.py:586-620).
 *   trans_b = 0: payload [K,N] (FP4: [K,N/2], adjacent columns share a byte),
 *                scales physical [ceil(K/64), N, 2]
 *   trans_b = 1: payload [N,K] (FP4: [N,K/2]), scales [N, 2*ceil(K/64)]
 * pinned by: equality with orc_mx_quant_rows on the explicit transpose.
 */
int orc_mx_quant_b(const uint16_t *b, int64_t K, int64_t N, int fmt, int rounding, int trans_b,
                   uint8_t *payload, uint8_t *scales)
{
    const int64_t nblk = (K + 31) / 32;
    const int64_t sld = ((nblk + 1) / 2) * 2;
    const int fp4 = ORC_IS_FP4(fmt);
    const int64_t pldT = fp4 ? (K + 1) / 2 : K;
    uint16_t *bt = (uint16_t *)malloc((size_t)(N * K) * 2);
    uint8_t *pt = (uint8_t *)malloc((size_t)(N * pldT));
    uint8_t *st = (uint8_t *)malloc((size_t)(N * sld));
    if (!bt || !pt || !st) { free(bt); free(pt); free(st); return -1; }
#pragma omp parallel for schedule(static)
    for (int64_t n = 0; n < N; n++)
        for (int64_t k = 0; k < K; k++) bt[n * K + k] = b[k * N + n];
    orc_mx_quant_rows(bt, N, K, fmt, rounding, pt, st);
    if (trans_b) {
        memcpy(payload, pt, (size_t)(N * pldT));
        memcpy(scales, st, (size_t)(N * sld));
    } else {
        const int64_t pld = fp4 ? (N + 1) / 2 : N;
        if (fp4) memset(payload, 0, (size_t)(K * pld));
#pragma omp parallel for schedule(static)
        for (int64_t k = 0; k < K; k++)
            for (int64_t n = 0; n < N; n++) {
                if (fp4) {
                    uint8_t q = (pt[n * pldT + (k >> 1)] >> ((k & 1) * 4)) & 0xF;
                    payload[k * pld + (n >> 1)] |= (uint8_t)(q << ((n & 1) * 4));
                } else {
                    payload[k * N + n] = pt[n * K + k];
                }
            }
        for (int64_t kb = 0; kb < sld; kb++)
            for (int64_t n = 0; n < N; n++)
                scales[((kb >> 1) * N + n) * 2 + (kb & 1)] = st[n * sld + kb];
    }
    free(bt); free(pt); free(st);
    return 0;
}

/* Dequantise an MX row-quantised matrix back to fp32 [M,K]
 * (gen_mx_quant_allgather_data.py:293; exact: small float times power of two).
 * pinned by: round trip with orc_mx_quant_rows. */
void orc_mx_dequant_rows(const uint8_t *payload, const uint8_t *scales, int64_t M, int64_t K, int fmt,
                         float *out)
{
    const int64_t nblk = (K + 31) / 32;
    const int64_t sld = ((nblk + 1) / 2) * 2;
    const int64_t pld = ORC_IS_FP4(fmt) ? (K + 1) / 2 : K;
#pragma omp parallel for schedule(static)
    for (int64_t m = 0; m < M; m++)
        for (int64_t k = 0; k < K; k++) {
            uint8_t q = ORC_IS_FP4(fmt) ? (payload[m * pld + (k >> 1)] >> ((k & 1) * 4)) & 0xF
                                              : payload[m * pld + k];
            out[m * K + k] = orc_decode(q, fmt) * orc_e8m0_decode(scales[m * sld + k / 32]);
        }
}

/* ------------------------------------------------------- int8 GEMM paths */

static float sigmoidf_(float x) { return 1.0f / (1.0f + expf(-x)); }

/*
 * out[m,n] = float(sum_k a[m,k]*b[k,n] as int32) * per_tok[m] * per_ch[n]
 * (gen_quant_data_mmdqrs.py:76-79), stored as fp32 and, if out_bf16 != NULL,
 * rounded to bf16.  `rows` (may be NULL = all) lists the output rows to
 * compute; out row i holds rows[i].  B is [K,N] (trans_b=0) or [N,K].
 * pinned by: int64 numpy matmul on small shapes (int32 sums are exact).
 */
void orc_gemm_i8_dequant(const int8_t *a, const int8_t *b, const float *per_tok, const float *per_ch,
                         int64_t M, int64_t N, int64_t K, int trans_b, const int64_t *rows, int64_t nrows,
                         float *out_f32, uint16_t *out_bf16)
{
    if (!rows) nrows = M;
#pragma omp parallel
    {
        int32_t *acc = (int32_t *)malloc((size_t)N * 4);
#pragma omp for schedule(dynamic, 1)
        for (int64_t i = 0; i < nrows; i++) {
            int64_t m = rows ? rows[i] : i;
            const int8_t *ar = a + m * K;
            memset(acc, 0, (size_t)N * 4);
            if (!trans_b) {
                for (int64_t k = 0; k < K; k++) {
                    int32_t av = ar[k];
                    const int8_t *br = b + k * N;
                    for (int64_t n = 0; n < N; n++) acc[n] += av * (int32_t)br[n];
                }
            } else {
                for (int64_t n = 0; n < N; n++) {
                    const int8_t *bc = b + n * K;
                    int32_t s = 0;
                    for (int64_t k = 0; k < K; k++) s += (int32_t)ar[k] * (int32_t)bc[k];
                    acc[n] = s;
                }
            }
            for (int64_t n = 0; n < N; n++) {
                float v = (float)acc[n] * per_tok[m] * per_ch[n];
                if (out_f32) out_f32[i * N + n] = v;
                if (out_bf16) out_bf16[i * N + n] = orc_f32_to_bf16(v);
            }
        }
        free(acc);
    }
}

/* Round an fp32 value to the nearest IEEE half (ties to even) and widen it
 * back.  pinned by: torch.float16 casts. */
float orc_round_through_f16(float v)
{
    if (v != v) return v;
    float a = fabsf(v);
    if (a >= 65520.0f) return v < 0 ? -INFINITY : INFINITY;
    int e;
    (void)frexpf(a, &e);               /* a = f * 2^e, f in [0.5,1) */
    int q = (e - 1 < -14 ? -14 : e - 1) - 10; /* spacing of halves near a is 2^q */
    float r = ldexpf(rintf(ldexpf(a, -q)), q); /* rintf: ties to even in the default mode */
    return v < 0 ? -r : r;
}
static float f32_to_f16_to_f32(float v) { return orc_round_through_f16(v); }

/* Truncate an fp32 value toward zero to IEEE half precision and widen it back
 * (the reference's Cast(..., RoundMode::CAST_TRUNC) to half).  Finite inputs
 * below the half range only.  pinned by: brute force over all 65536 half bit
 * patterns (largest |half| not above |v|). */
float orc_trunc_through_f16(float v)
{
    if (v != v) return v;
    float a = fabsf(v);
    if (a >= 65504.0f) a = 65504.0f;
    int e;
    (void)frexpf(a, &e);                      /* a = f * 2^e, f in [0.5,1) */
    int q = (e - 1 < -14 ? -14 : e - 1) - 10; /* spacing of halves near a is 2^q */
    float r = ldexpf(floorf(ldexpf(a, -q)), q);
    return v < 0 ? -r : r;
}

/*
 * Per-token dynamic int8 quantisation with an optional row gather, the step
 * that feeds the MoE int8 grouped GEMM
 * (examples/aux_ops/moe_init_routing_quant_v2/moe_v2_gather_dynamic_quant.h).
 *   x        bf16 [rows_in, K]
 *   src      int32 [T] or NULL: output row i quantises input row src[i] / topk
 *            (:229-236, srcIdx / k); a negative entry or one past the input
 *            gives a zero row with scale 0 (the reference skips such rows,
 *            :198-201).  NULL: row i.
 *   mode 0   the device kernel's arithmetic (:132-150): scale = amax / 127
 *            (fp32), y = x / scale (fp32), y truncated to half, then rounded
 *            to the nearest integer with halves away from zero
 *   mode 1   the generator's golden (gen_data_dispatch_gmm_dequant_swiglu.py
 *            :275-280): q = rint(x * 127 / amax) in fp32 (ties to even),
 *            scale = amax / 127
 *   smooth   fp32 [num_smooth, K] or NULL: every element is multiplied (in
 *            fp32, one rounding) by the smoothing vector of its row before
 *            anything else (:127-130).  smooth_rows int32 [T] picks the vector
 *            of output row i (the row's expert, :241); NULL: vector 0 for every
 *            row (:170-174).  An index outside [0, num_smooth) gives a zero row.
 *   An all-zero row gives q = 0 and scale 0 in both modes (the reference
 *   divides 0 by 0 there).
 * pinned by: mode 1 against torch (abs/max/round on the same data); mode 0
 *            against a numpy restatement built on the brute-force half
 *            truncation; |q| <= 127 with 127 reached in every non-zero row;
 *            |x - q*scale| <= scale (mode 0) and <= scale/2 (mode 1);
 *            smoothing: the same two restatements on the fp32 products, and
 *            power-of-two vectors against the unsmoothed routine on the
 *            pre-scaled input (the products are then exact bf16 values).
 */
void orc_dyn_quant_i8_rows(const uint16_t *x, const int32_t *src, int64_t rows_in, int64_t T, int64_t K, int topk,
                           int mode, const float *smooth, const int32_t *smooth_rows, int64_t num_smooth, int8_t *q,
                           float *scale)
{
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < T; i++) {
        int64_t r = src ? (src[i] < 0 ? -1 : (int64_t)src[i] / topk) : i;
        int8_t *qo = q + i * K;
        const int64_t sv = smooth ? (smooth_rows ? (int64_t)smooth_rows[i] : 0) : 0;
        if (r < 0 || r >= rows_in || (smooth && (sv < 0 || sv >= num_smooth))) {
            memset(qo, 0, (size_t)K);
            scale[i] = 0.0f;
            continue;
        }
        const uint16_t *xr = x + r * K;
        const float *sm = smooth ? smooth + sv * K : NULL;
        float amax = 0.0f;
        for (int64_t k = 0; k < K; k++) {
            float v = orc_bf16_to_f32(xr[k]);
            if (sm) v = v * sm[k];
            const float a = fabsf(v);
            if (a > amax) amax = a;
        }
        if (!(amax > 0.0f)) {
            memset(qo, 0, (size_t)K);
            scale[i] = 0.0f;
            continue;
        }
        const float sc = amax / 127.0f;
        scale[i] = sc;
        for (int64_t k = 0; k < K; k++) {
            float v = orc_bf16_to_f32(xr[k]);
            if (sm) v = v * sm[k];
            float y;
            if (mode == 0) {
                const float t = orc_trunc_through_f16(v / sc);
                y = truncf(t + (t < 0 ? -0.5f : 0.5f));   /* exact: t has at most 11 significant bits */
            } else {
                y = rintf(v * 127.0f / amax);
            }
            if (y > 127.0f) y = 127.0f;
            if (y < -128.0f) y = -128.0f;
            qo[k] = (int8_t)y;
        }
    }
}

/*
 * Grouped int8 GEMM + per-channel dequant + per-token dequant + SwiGLU
 * (gen_data_dispatch_gmm_dequant_swiglu.py:298-320, swiglu :269-273).
 *   x [T,K] int8, rows of expert e are contiguous, group_sizes[e] rows each;
 *   w [E,K,N] int8; per_ch [E,N]; per_tok [T];
 *   c = float(acc) * per_ch[e,n]           (optionally rounded through fp16,
 *                                           as the reference's :309-310)
 *   c = c * per_tok[r]
 *   out[r,j] = c[j] * sigmoid(c[j]) * c[j + N/2],  j < N/2  (first half = gate)
 * Rows past sum(group_sizes) are zero (:319-320).
 * pinned by: torch.nn.functional.silu on the fp32 intermediate + the pinned
 *            int8 GEMM; per-group equality with the dense routine.
 */
void orc_gmm_i8_dequant_swiglu(const int8_t *x, const int8_t *w, const int32_t *group_sizes, int64_t E,
                               int64_t T, int64_t K, int64_t N, const float *per_tok, const float *per_ch,
                               int fp16_step, const int64_t *rows, int64_t nrows, float *out_f32,
                               uint16_t *out_bf16)
{
    const int64_t H = N / 2;
    int64_t *row_expert = (int64_t *)malloc((size_t)(T > 0 ? T : 1) * 8);
    int64_t r = 0;
    for (int64_t e = 0; e < E; e++)
        for (int32_t i = 0; i < group_sizes[e] && r < T; i++) row_expert[r++] = e;
    for (; r < T; r++) row_expert[r] = -1;
    if (!rows) nrows = T;
#pragma omp parallel
    {
        int32_t *acc = (int32_t *)malloc((size_t)N * 4);
        float *c = (float *)malloc((size_t)N * 4);
#pragma omp for schedule(dynamic, 1)
        for (int64_t i = 0; i < nrows; i++) {
            int64_t m = rows ? rows[i] : i;
            int64_t e = row_expert[m];
            if (e < 0) {
                for (int64_t j = 0; j < H; j++) {
                    if (out_f32) out_f32[i * H + j] = 0.0f;
                    if (out_bf16) out_bf16[i * H + j] = 0;
                }
                continue;
            }
            const int8_t *ar = x + m * K;
            const int8_t *we = w + e * K * N;
            memset(acc, 0, (size_t)N * 4);
            for (int64_t k = 0; k < K; k++) {
                int32_t av = ar[k];
                const int8_t *br = we + k * N;
                for (int64_t n = 0; n < N; n++) acc[n] += av * (int32_t)br[n];
            }
            for (int64_t n = 0; n < N; n++) {
                float v = (float)acc[n] * per_ch[e * N + n];
                if (fp16_step) v = f32_to_f16_to_f32(v);
                c[n] = v * per_tok[m];
            }
            for (int64_t j = 0; j < H; j++) {
                float g = c[j];
                float v = g * sigmoidf_(g) * c[j + H];
                if (out_f32) out_f32[i * H + j] = v;
                if (out_bf16) out_bf16[i * H + j] = orc_f32_to_bf16(v);
            }
        }
        free(acc);
        free(c);
    }
    free(row_expert);
}

/* --------------------------------------------------------- MX GEMM paths */

static inline uint8_t payload_at(const uint8_t *p, int64_t ld_elems, int64_t r, int64_t c, int fp4)
{
    if (fp4) {
        int64_t ldb = (ld_elems + 1) / 2;
        return (p[r * ldb + (c >> 1)] >> ((c & 1) * 4)) & 0xF;
    }
    return p[r * ld_elems + c];
}

/*
 * Grouped (E >= 1) MX GEMM golden: C = deq(A) @ deq(B_e), fp32 accumulate
 * (gen_data_mxfp8_mmrs.py:345-355; gen_data_fp4_mx_alltoallv_gmm.py:724-734),
 *   deq(x)[m,k] = decode(q[m,k]) * 2^(s[m,k/32]-127).
 *   a  payload [T,K] (FP4 [T,K/2]); sa [T, 2*ceil(K/64)]
 *   b  per expert: trans_b=0 payload [K,N] (FP4 [K,N/2]), sb [ceil(K/64),N,2]
 *                  trans_b=1 payload [N,K] (FP4 [N,K/2]), sb [N,2*ceil(K/64)]
 *   group_sizes NULL means one dense problem (E must be 1).
 * Rows past sum(group_sizes) are zero (:788-790).
 * Accumulation runs over k in ascending order in fp32; `out_f64` (optional)
 * receives the same sums accumulated in double for tolerance studies.
 * pinned by: fp64 numpy matmul of independently dequantised operands on small
 *            shapes; scales == 127 reduces to a plain FP8 GEMM; one-hot rows.
 */
void orc_mx_gmm(const uint8_t *a, const uint8_t *sa, const uint8_t *b, const uint8_t *sb,
                const int32_t *group_sizes, int64_t E, int64_t T, int64_t N, int64_t K, int fmt, int trans_b,
                const int64_t *rows, int64_t nrows, float *out_f32, uint16_t *out_bf16, double *out_f64)
{
    const int fp4 = fmt == ORC_FMT_E2M1;
    const int64_t nblk = (K + 31) / 32;
    const int64_t sld = ((nblk + 1) / 2) * 2;
    const int64_t b_bytes = fp4 ? (trans_b ? N * ((K + 1) / 2) : K * ((N + 1) / 2)) : K * N;
    const int64_t sb_bytes = sld * N;
    int64_t *row_expert = (int64_t *)malloc((size_t)(T > 0 ? T : 1) * 8);
    if (group_sizes) {
        int64_t r = 0;
        for (int64_t e = 0; e < E; e++)
            for (int32_t i = 0; i < group_sizes[e] && r < T; i++) row_expert[r++] = e;
        for (; r < T; r++) row_expert[r] = -1;
    } else {
        for (int64_t r = 0; r < T; r++) row_expert[r] = 0;
    }
    if (!rows) nrows = T;
#pragma omp parallel
    {
        float *arow = (float *)malloc((size_t)K * 4);
        float *acc = (float *)malloc((size_t)N * 4);
        double *acc64 = out_f64 ? (double *)malloc((size_t)N * 8) : NULL;
#pragma omp for schedule(dynamic, 1)
        for (int64_t i = 0; i < nrows; i++) {
            int64_t m = rows ? rows[i] : i;
            int64_t e = row_expert[m];
            for (int64_t n = 0; n < N; n++) { acc[n] = 0.0f; if (acc64) acc64[n] = 0.0; }
            if (e >= 0) {
                const uint8_t *be = b + e * b_bytes;
                const uint8_t *sbe = sb + e * sb_bytes;
                for (int64_t k = 0; k < K; k++)
                    arow[k] = orc_decode(payload_at(a, K, m, k, fp4), fmt) * orc_e8m0_decode(sa[m * sld + k / 32]);
                if (!trans_b) {
                    for (int64_t k = 0; k < K; k++) {
                        float av = arow[k];
                        int64_t kb = k / 32;
                        const uint8_t *srow = sbe + (kb >> 1) * N * 2 + (kb & 1);
                        for (int64_t n = 0; n < N; n++) {
                            float bv = orc_decode(payload_at(be, N, k, n, fp4), fmt) * orc_e8m0_decode(srow[n * 2]);
                            acc[n] += av * bv;
                            if (acc64) acc64[n] += (double)av * (double)bv;
                        }
                    }
                } else {
                    for (int64_t n = 0; n < N; n++) {
                        float s = 0.0f;
                        double s64 = 0.0;
                        for (int64_t k = 0; k < K; k++) {
                            float bv = orc_decode(payload_at(be, K, n, k, fp4), fmt) *
                                       orc_e8m0_decode(sbe[n * sld + k / 32]);
                            s += arow[k] * bv;
                            s64 += (double)arow[k] * (double)bv;
                        }
                        acc[n] = s;
                        if (acc64) acc64[n] = s64;
                    }
                }
            }
            for (int64_t n = 0; n < N; n++) {
                if (out_f32) out_f32[i * N + n] = acc[n];
                if (out_bf16) out_bf16[i * N + n] = orc_f32_to_bf16(acc[n]);
                if (out_f64) out_f64[i * N + n] = acc64[n];
            }
        }
        free(arow); free(acc); free(acc64);
    }
    free(row_expert);
}

/*
 * SwiGLU of a bf16 [T, N] tile, gate = columns [0, N/2), up = [N/2, N), as the reference's
 * register-level routine computes it from the up projection's bf16 planes
 * (include/catccos/epilogue/block/block_epilogue_regbase_swiglu.hpp:38-80): widen both to fp32,
 *   d = exp(gate * -1) + 1;  r = gate / d;  r = r * up;  out = bf16(r), round to nearest even.
 * pinned by: torch.nn.functional.silu(gate.float()) * up.float() rounded to bf16 (equal up to one
 *            bf16 step where the two fp32 formulas round differently, equal exactly on most inputs),
 *            the closed forms at gate = 0, large positive and large negative gate.
 */
void orc_swiglu_bf16(const uint16_t *c, int64_t T, int64_t N, uint16_t *out)
{
    const int64_t H = N / 2;
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < T; r++)
        for (int64_t j = 0; j < H; j++) {
            float g = orc_bf16_to_f32(c[r * N + j]), u = orc_bf16_to_f32(c[r * N + j + H]);
            float d = expf(g * -1.0f) + 1.0f;
            float v = g / d;
            v = v * u;
            out[r * H + j] = orc_f32_to_bf16(v);
        }
}

/* ------------------------------------------------ blocked CPU baselines */

/*
 * The routines above compute one output row at a time and decode every
 * weight again for every row: fine as a golden, a straw man as a CPU
 * baseline.  The *_blocked routines below produce THE SAME VALUES (same
 * operands, same k-ascending accumulation with one fused multiply-add per
 * term in fp32, exact int32 sums for int8) with the work organised the way a
 * CPU GEMM is: per expert the selected rows of A are decoded once, each
 * thread owns a block of BLK_N output columns, decodes a BLK_K x BLK_N panel
 * of the expert's weights once and runs a 4 x 16 register tile over it.
 * pinned by: equality with orc_mx_gmm / orc_gemm_i8_dequant /
 *            orc_gmm_i8_dequant_swiglu on ragged shapes, both layouts, all
 *            payload formats (tests/test_oracle_blocked.py).
 */
#define BLK_N 128
#define BLK_K 256
typedef float vf8 __attribute__((vector_size(32), aligned(4)));
typedef int32_t vi8 __attribute__((vector_size(32), aligned(4)));

/* selected output indices ordered by expert: order[start[e] .. start[e+1]) */
static void rows_by_expert(const int64_t *row_expert, const int64_t *rows, int64_t nrows, int64_t E,
                           int64_t *start, int64_t *order)
{
    for (int64_t e = 0; e <= E; e++) start[e] = 0;
    for (int64_t i = 0; i < nrows; i++) {
        int64_t e = row_expert[rows ? rows[i] : i];
        if (e >= 0) start[e + 1]++;
    }
    for (int64_t e = 0; e < E; e++) start[e + 1] += start[e];
    int64_t *fill = (int64_t *)malloc((size_t)(E + 1) * 8);
    memcpy(fill, start, (size_t)(E + 1) * 8);
    for (int64_t i = 0; i < nrows; i++) {
        int64_t e = row_expert[rows ? rows[i] : i];
        if (e >= 0) order[fill[e]++] = i;
    }
    free(fill);
}

/* c[cnt][BLK_N] += a[cnt][lda] (columns k0..k0+kc) x panel[kc][BLK_N], fp32, k ascending */
static void tile_f32(const float *a, int64_t lda, int64_t cnt, const float *panel, int64_t kc, float *c)
{
    int64_t r = 0;
    for (; r + 4 <= cnt; r += 4)
        for (int64_t n0 = 0; n0 < BLK_N; n0 += 16) {
            vf8 acc[4][2];
            for (int i = 0; i < 4; i++)
                for (int h = 0; h < 2; h++) acc[i][h] = *(const vf8 *)(c + (r + i) * BLK_N + n0 + 8 * h);
            for (int64_t k = 0; k < kc; k++) {
                const vf8 b0 = *(const vf8 *)(panel + k * BLK_N + n0), b1 = *(const vf8 *)(panel + k * BLK_N + n0 + 8);
                for (int i = 0; i < 4; i++) {
                    const float av = a[(r + i) * lda + k];
                    const vf8 a8 = {av, av, av, av, av, av, av, av};
                    acc[i][0] += a8 * b0;
                    acc[i][1] += a8 * b1;
                }
            }
            for (int i = 0; i < 4; i++)
                for (int h = 0; h < 2; h++) *(vf8 *)(c + (r + i) * BLK_N + n0 + 8 * h) = acc[i][h];
        }
    for (; r < cnt; r++)
        for (int64_t n0 = 0; n0 < BLK_N; n0 += 8) {
            vf8 acc = *(const vf8 *)(c + r * BLK_N + n0);
            for (int64_t k = 0; k < kc; k++) {
                const float av = a[r * lda + k];
                const vf8 a8 = {av, av, av, av, av, av, av, av};
                acc += a8 * *(const vf8 *)(panel + k * BLK_N + n0);
            }
            *(vf8 *)(c + r * BLK_N + n0) = acc;
        }
}

static void tile_i32(const int32_t *a, int64_t lda, int64_t cnt, const int32_t *panel, int64_t kc, int32_t *c)
{
    int64_t r = 0;
    for (; r + 4 <= cnt; r += 4)
        for (int64_t n0 = 0; n0 < BLK_N; n0 += 16) {
            vi8 acc[4][2];
            for (int i = 0; i < 4; i++)
                for (int h = 0; h < 2; h++) acc[i][h] = *(const vi8 *)(c + (r + i) * BLK_N + n0 + 8 * h);
            for (int64_t k = 0; k < kc; k++) {
                const vi8 b0 = *(const vi8 *)(panel + k * BLK_N + n0), b1 = *(const vi8 *)(panel + k * BLK_N + n0 + 8);
                for (int i = 0; i < 4; i++) {
                    const int32_t av = a[(r + i) * lda + k];
                    const vi8 a8 = {av, av, av, av, av, av, av, av};
                    acc[i][0] += a8 * b0;
                    acc[i][1] += a8 * b1;
                }
            }
            for (int i = 0; i < 4; i++)
                for (int h = 0; h < 2; h++) *(vi8 *)(c + (r + i) * BLK_N + n0 + 8 * h) = acc[i][h];
        }
    for (; r < cnt; r++)
        for (int64_t n = 0; n < BLK_N; n++) {
            int32_t s = c[r * BLK_N + n];
            for (int64_t k = 0; k < kc; k++) s += a[r * lda + k] * panel[k * BLK_N + n];
            c[r * BLK_N + n] = s;
        }
}

/* Same arguments and results as orc_mx_gmm (without the fp64 copy). */
void orc_mx_gmm_blocked(const uint8_t *a, const uint8_t *sa, const uint8_t *b, const uint8_t *sb,
                        const int32_t *group_sizes, int64_t E, int64_t T, int64_t N, int64_t K, int fmt, int trans_b,
                        const int64_t *rows, int64_t nrows, float *out_f32, uint16_t *out_bf16)
{
    const int fp4 = fmt == ORC_FMT_E2M1;
    const int64_t nblk = (K + 31) / 32;
    const int64_t sld = ((nblk + 1) / 2) * 2;
    const int64_t b_bytes = fp4 ? (trans_b ? N * ((K + 1) / 2) : K * ((N + 1) / 2)) : K * N;
    const int64_t sb_bytes = sld * N;
    int64_t *row_expert = (int64_t *)malloc((size_t)(T > 0 ? T : 1) * 8);
    if (group_sizes) {
        int64_t r = 0;
        for (int64_t e = 0; e < E; e++)
            for (int32_t i = 0; i < group_sizes[e] && r < T; i++) row_expert[r++] = e;
        for (; r < T; r++) row_expert[r] = -1;
    } else {
        for (int64_t r = 0; r < T; r++) row_expert[r] = 0;
    }
    if (!rows) nrows = T;
    int64_t *start = (int64_t *)malloc((size_t)(E + 1) * 8);
    int64_t *order = (int64_t *)malloc((size_t)(nrows > 0 ? nrows : 1) * 8);
    rows_by_expert(row_expert, rows, nrows, E, start, order);
    /* rows that belong to no group are zero */
    for (int64_t i = 0; i < nrows; i++)
        if (row_expert[rows ? rows[i] : i] < 0)
            for (int64_t n = 0; n < N; n++) {
                if (out_f32) out_f32[i * N + n] = 0.0f;
                if (out_bf16) out_bf16[i * N + n] = 0;
            }
    const int64_t ncb = (N + BLK_N - 1) / BLK_N;
    for (int64_t e = 0; e < E; e++) {
        const int64_t cnt = start[e + 1] - start[e];
        if (cnt == 0) continue;
        const int64_t *ord = order + start[e];
        const uint8_t *be = b + e * b_bytes;
        const uint8_t *sbe = sb + e * sb_bytes;
        float *adeq = (float *)malloc((size_t)cnt * K * 4);
#pragma omp parallel for schedule(static)
        for (int64_t i = 0; i < cnt; i++) {
            const int64_t m = rows ? rows[ord[i]] : ord[i];
            for (int64_t k = 0; k < K; k++)
                adeq[i * K + k] = orc_decode(payload_at(a, K, m, k, fp4), fmt) * orc_e8m0_decode(sa[m * sld + k / 32]);
        }
#pragma omp parallel
        {
            float *panel = (float *)malloc((size_t)BLK_K * BLK_N * 4);
            float *c = (float *)malloc((size_t)cnt * BLK_N * 4);
#pragma omp for schedule(dynamic, 1)
            for (int64_t cb = 0; cb < ncb; cb++) {
                const int64_t n0 = cb * BLK_N, nc = N - n0 < BLK_N ? N - n0 : BLK_N;
                memset(c, 0, (size_t)cnt * BLK_N * 4);
                for (int64_t k0 = 0; k0 < K; k0 += BLK_K) {
                    const int64_t kc = K - k0 < BLK_K ? K - k0 : BLK_K;
                    for (int64_t kk = 0; kk < kc; kk++) {
                        const int64_t k = k0 + kk, kb = k / 32;
                        float *prow = panel + kk * BLK_N;
                        for (int64_t j = 0; j < nc; j++) {
                            const int64_t n = n0 + j;
                            prow[j] = trans_b ? orc_decode(payload_at(be, K, n, k, fp4), fmt) * orc_e8m0_decode(sbe[n * sld + kb])
                                              : orc_decode(payload_at(be, N, k, n, fp4), fmt) *
                                                    orc_e8m0_decode(sbe[(kb >> 1) * N * 2 + n * 2 + (kb & 1)]);
                        }
                        for (int64_t j = nc; j < BLK_N; j++) prow[j] = 0.0f;
                    }
                    tile_f32(adeq + k0, K, cnt, panel, kc, c);
                }
                for (int64_t i = 0; i < cnt; i++)
                    for (int64_t j = 0; j < nc; j++) {
                        if (out_f32) out_f32[ord[i] * N + n0 + j] = c[i * BLK_N + j];
                        if (out_bf16) out_bf16[ord[i] * N + n0 + j] = orc_f32_to_bf16(c[i * BLK_N + j]);
                    }
            }
            free(panel);
            free(c);
        }
        free(adeq);
    }
    free(order); free(start); free(row_expert);
}

/* int8 x int8 -> int32 for the selected rows of one expert (or of the dense problem): acc[cnt][N] */
static void i8_expert_blocked(const int8_t *x, const int8_t *w, int64_t N, int64_t K, int trans_b, const int64_t *rows,
                              const int64_t *ord, int64_t cnt, int32_t *acc)
{
    int32_t *a32 = (int32_t *)malloc((size_t)cnt * K * 4);
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < cnt; i++) {
        const int64_t m = rows ? rows[ord[i]] : ord[i];
        for (int64_t k = 0; k < K; k++) a32[i * K + k] = x[m * K + k];
    }
    const int64_t ncb = (N + BLK_N - 1) / BLK_N;
#pragma omp parallel
    {
        int32_t *panel = (int32_t *)malloc((size_t)BLK_K * BLK_N * 4);
        int32_t *c = (int32_t *)malloc((size_t)cnt * BLK_N * 4);
#pragma omp for schedule(dynamic, 1)
        for (int64_t cb = 0; cb < ncb; cb++) {
            const int64_t n0 = cb * BLK_N, nc = N - n0 < BLK_N ? N - n0 : BLK_N;
            memset(c, 0, (size_t)cnt * BLK_N * 4);
            for (int64_t k0 = 0; k0 < K; k0 += BLK_K) {
                const int64_t kc = K - k0 < BLK_K ? K - k0 : BLK_K;
                for (int64_t kk = 0; kk < kc; kk++) {
                    int32_t *prow = panel + kk * BLK_N;
                    for (int64_t j = 0; j < nc; j++) prow[j] = trans_b ? w[(n0 + j) * K + k0 + kk] : w[(k0 + kk) * N + n0 + j];
                    for (int64_t j = nc; j < BLK_N; j++) prow[j] = 0;
                }
                tile_i32(a32 + k0, K, cnt, panel, kc, c);
            }
            for (int64_t i = 0; i < cnt; i++)
                for (int64_t j = 0; j < nc; j++) acc[i * N + n0 + j] = c[i * BLK_N + j];
        }
        free(panel);
        free(c);
    }
    free(a32);
}

/* Same arguments and results as orc_gemm_i8_dequant. */
void orc_gemm_i8_dequant_blocked(const int8_t *a, const int8_t *b, const float *per_tok, const float *per_ch,
                                 int64_t M, int64_t N, int64_t K, int trans_b, const int64_t *rows, int64_t nrows,
                                 float *out_f32, uint16_t *out_bf16)
{
    if (!rows) nrows = M;
    int64_t *ord = (int64_t *)malloc((size_t)(nrows > 0 ? nrows : 1) * 8);
    for (int64_t i = 0; i < nrows; i++) ord[i] = i;
    int32_t *acc = (int32_t *)malloc((size_t)(nrows > 0 ? nrows : 1) * N * 4);
    i8_expert_blocked(a, b, N, K, trans_b, rows, ord, nrows, acc);
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < nrows; i++) {
        const int64_t m = rows ? rows[i] : i;
        for (int64_t n = 0; n < N; n++) {
            float v = (float)acc[i * N + n] * per_tok[m] * per_ch[n];
            if (out_f32) out_f32[i * N + n] = v;
            if (out_bf16) out_bf16[i * N + n] = orc_f32_to_bf16(v);
        }
    }
    free(acc); free(ord);
}

/* Same arguments and results as orc_gmm_i8_dequant_swiglu. */
void orc_gmm_i8_dequant_swiglu_blocked(const int8_t *x, const int8_t *w, const int32_t *group_sizes, int64_t E,
                                       int64_t T, int64_t K, int64_t N, const float *per_tok, const float *per_ch,
                                       int fp16_step, const int64_t *rows, int64_t nrows, float *out_f32,
                                       uint16_t *out_bf16)
{
    const int64_t H = N / 2;
    int64_t *row_expert = (int64_t *)malloc((size_t)(T > 0 ? T : 1) * 8);
    int64_t r = 0;
    for (int64_t e = 0; e < E; e++)
        for (int32_t i = 0; i < group_sizes[e] && r < T; i++) row_expert[r++] = e;
    for (; r < T; r++) row_expert[r] = -1;
    if (!rows) nrows = T;
    int64_t *start = (int64_t *)malloc((size_t)(E + 1) * 8);
    int64_t *order = (int64_t *)malloc((size_t)(nrows > 0 ? nrows : 1) * 8);
    rows_by_expert(row_expert, rows, nrows, E, start, order);
    for (int64_t i = 0; i < nrows; i++)
        if (row_expert[rows ? rows[i] : i] < 0)
            for (int64_t j = 0; j < H; j++) {
                if (out_f32) out_f32[i * H + j] = 0.0f;
                if (out_bf16) out_bf16[i * H + j] = 0;
            }
    for (int64_t e = 0; e < E; e++) {
        const int64_t cnt = start[e + 1] - start[e];
        if (cnt == 0) continue;
        const int64_t *ord = order + start[e];
        int32_t *acc = (int32_t *)malloc((size_t)cnt * N * 4);
        i8_expert_blocked(x, w + e * K * N, N, K, 0, rows, ord, cnt, acc);
#pragma omp parallel for schedule(static)
        for (int64_t i = 0; i < cnt; i++) {
            const int64_t m = rows ? rows[ord[i]] : ord[i];
            for (int64_t j = 0; j < H; j++) {
                float g = (float)acc[i * N + j] * per_ch[e * N + j];
                float u = (float)acc[i * N + j + H] * per_ch[e * N + j + H];
                if (fp16_step) { g = f32_to_f16_to_f32(g); u = f32_to_f16_to_f32(u); }
                g *= per_tok[m];
                u *= per_tok[m];
                float v = g * sigmoidf_(g) * u;
                if (out_f32) out_f32[ord[i] * H + j] = v;
                if (out_bf16) out_bf16[ord[i] * H + j] = orc_f32_to_bf16(v);
            }
        }
        free(acc);
    }
    free(order); free(start); free(row_expert);
}

/* ---------------------------------------------- token-count prefix sums */

/* comm_block_scheduler_alltoallv_gmm.hpp:113-121: rows that source core
 * `core_idx` has already sent to ranks below `rank`.
 * pinned by: the reference's unit-test vector (test_comm_block_scheduler_alltoallv_gmm.cpp:96-102) */
int32_t orc_sched_src_prev_sum(const int32_t *token_per_expert, int32_t rank, int32_t ep,
                               int32_t expert_per_rank, uint32_t core_idx)
{
    int32_t s = 0;
    if ((int64_t)core_idx < ep)
        for (int32_t i = 0; i < rank * expert_per_rank; i++)
            s += token_per_expert[(int64_t)core_idx * ep * expert_per_rank + i];
    return s;
}

/* :92-105.  pinned by: the same unit-test vector */
uint32_t orc_sched_comm_loops(int32_t ep, uint32_t core_idx, uint32_t core_num)
{
    if (core_num == 0) return 1;
    uint32_t res = (uint32_t)ep / core_num;
    if (core_idx < ((uint32_t)ep % core_num)) res++;
    return res;
}

/* :123-128.  pinned by: the same unit-test vector */
uint32_t orc_sched_block_offset_row(uint32_t core_idx, uint32_t core_num, uint32_t comm_idx)
{
    return core_idx + comm_idx * core_num;
}

/* :130-159: cumsum_mm[r][e] = sum_{r'<=r} token_per_expert[r'][rank*E_loc + e];
 * the last row holds each local expert's total row count.
 * pinned by: numpy cumsum (closed form) */
void orc_sched_cumsum_mm(const int32_t *token_per_expert, int32_t rank, int32_t ep, int32_t expert_per_rank,
                         int32_t *cumsum_mm)
{
    for (int32_t e = 0; e < expert_per_rank; e++) {
        int32_t s = 0;
        for (int32_t r = 0; r < ep; r++) {
            s += token_per_expert[(int64_t)r * ep * expert_per_rank + rank * expert_per_rank + e];
            cumsum_mm[r * expert_per_rank + e] = s;
        }
    }
}

/*
 * Grouped-GEMM tile order on one device (source-rank dimension collapsed):
 * groups are visited in expert order; group g has ceil(m_g/BM) x ceil(N/BN)
 * tiles numbered row-major with every odd tile-row reversed
 * (MatrixSwizzle<1,0>, catccos.hpp:141-163); tiles are dealt to `nblocks`
 * workers round-robin with the remainder carried into the next group
 * (block_scheduler_alltoallv_allgather.hpp:132-153), i.e. the global tile
 * index modulo nblocks picks the worker.  Output rows of group g start at the
 * exclusive prefix sum of the sizes (:66-73).
 * Writes up to `cap` records {worker, group, row0, col0, rows, cols} and
 * returns the total number of tiles.
 * pinned by: partition invariants (every output element covered once, empty
 *            groups give no tile) and hand-worked small cases.
 */
int64_t orc_grouped_tile_order(const int32_t *group_sizes, int64_t E, int64_t N, int32_t bm, int32_t bn,
                               int32_t nblocks, int64_t cap, int64_t *rec)
{
    int64_t total = 0, row_base = 0;
    int64_t gn = (N + bn - 1) / bn;
    for (int64_t g = 0; g < E; g++) {
        int64_t mg = group_sizes[g];
        int64_t gm = (mg + bm - 1) / bm;
        for (int64_t t = 0; t < gm * gn; t++) {
            int64_t tr = t / gn, tc = t % gn;
            if (tr & 1) tc = gn - 1 - tc;
            if (total < cap) {
                int64_t *q = rec + total * 6;
                q[0] = total % nblocks;
                q[1] = g;
                q[2] = row_base + tr * bm;
                q[3] = tc * bn;
                q[4] = (mg - tr * bm) < bm ? (mg - tr * bm) : bm;
                q[5] = (N - tc * bn) < bn ? (N - tc * bn) : bn;
            }
            total++;
        }
        row_base += mg;
    }
    return total;
}

/* ----------------------------------------------------- comparison metrics */

/*
 * Error metrics of verify_result.py:154-196 and the 1e-2 gate of the task:
 *   m[0] = max |d-g| / max(|g|, 1)        (the reference's floor, :172)
 *   m[1] = max |d-g| / max(|g|, rms(g))   (floor that is not vacuous for small g)
 *   m[2] = mean((d-g)/max(1,|g|))         (the reference's "eb", :52-61)
 *   m[3] = rms(g)
 *   m[4] = fraction of elements with |d-g| > rtol*max(1,|g|)
 * pinned by: numpy restatement on random data.
 */
void orc_compare(const float *d, const float *g, int64_t n, float rtol, double *m)
{
    double ss = 0.0;
    for (int64_t i = 0; i < n; i++) ss += (double)g[i] * (double)g[i];
    double rms = n ? sqrt(ss / (double)n) : 0.0;
    double m0 = 0.0, m1 = 0.0, eb = 0.0;
    int64_t bad = 0;
    for (int64_t i = 0; i < n; i++) {
        double dv = d[i], gv = g[i];
        if (dv != dv || isinf(dv)) dv = 0.0;
        if (gv != gv || isinf(gv)) gv = 0.0;
        double diff = fabs(dv - gv), ag = fabs(gv);
        double f1 = ag > 1.0 ? ag : 1.0, f2 = ag > rms ? ag : rms;
        if (diff / f1 > m0) m0 = diff / f1;
        if (f2 > 0.0 && diff / f2 > m1) m1 = diff / f2;
        eb += (dv - gv) / f1;
        if (diff > (double)rtol * f1) bad++;
    }
    m[0] = m0; m[1] = m1; m[2] = n ? eb / (double)n : 0.0; m[3] = rms; m[4] = n ? (double)bad / (double)n : 0.0;
}

/*
 * The "double golden" acceptance metric of verify_result.py:198-246 (cal_double_precision_eb_percent), the one
 * examples/ascend950_mxfp8_matmul_reduce_scatter/scripts/run.sh:56-61 applies: the device result d and a
 * low-precision golden glow are both measured against the high-precision golden g,
 *   rel(x) = |x - g| / (|g| + 1e-7)     (:224-225; NaN and Inf count as 0, :206-211, everything in fp32 as torch does)
 * and the result passes (double_precision_performance_analysis, :105-117) when
 *   m[0] = max rel(d)  / max(max rel(glow),  err_threshold) < 10
 *   m[1] = mean rel(d) / max(mean rel(glow), err_threshold) < 2
 *   m[2] = rmse(d)     / max(rmse(glow),     err_threshold) < 2
 *   m[3] = |mean((d - g) / max(1, |g|))| / eb_threshold * 100 <= 100
 * with err_threshold = 2^-8 and eb_threshold = 2^-7 for a bfloat16 result (:66-68).  m[4..9] are the six
 * quantities themselves (max, mean, rmse of d, then of glow).  The low-precision golden of that example is the fp32
 * matmul of the dequantised operands cast to bfloat16 (gen_data_mxfp8_mmrs.py:349-355), i.e. g rounded to bf16.
 * pinned by: a numpy restatement in fp32 on random data, and closed forms (d == g gives zeros; d == glow gives
 *            ratios of exactly 1 where glow's error is above the floor).
 */
void orc_compare_double(const float *d, const float *g, const float *glow, int64_t n, float err_threshold, float eb_threshold,
                        double *m)
{
    const float eps = 1e-7f;
    float max_d = 0.0f, max_l = 0.0f;
    double sum_d = 0.0, sum_l = 0.0, sq_d = 0.0, sq_l = 0.0, eb = 0.0;
    for (int64_t i = 0; i < n; i++) {
        float dv = d[i], gv = g[i], lv = glow[i];
        if (dv != dv || isinf(dv)) dv = 0.0f;
        if (gv != gv || isinf(gv)) gv = 0.0f;
        if (lv != lv || isinf(lv)) lv = 0.0f;
        const float dd = dv - gv, dl = lv - gv, den = fabsf(gv) + eps;
        const float rd = fabsf(dd) / den, rl = fabsf(dl) / den;
        if (rd > max_d) max_d = rd;
        if (rl > max_l) max_l = rl;
        sum_d += rd; sum_l += rl;
        sq_d += (double)(dd * dd); sq_l += (double)(dl * dl);
        eb += (double)(dd / fmaxf(1.0f, fabsf(gv)));
    }
    const double nn = n ? (double)n : 1.0;
    const double mean_d = sum_d / nn, mean_l = sum_l / nn, rmse_d = sqrt(sq_d / nn), rmse_l = sqrt(sq_l / nn);
    const double thr = err_threshold;
    m[0] = (double)max_d / fmax((double)max_l, thr);
    m[1] = mean_d / fmax(mean_l, thr);
    m[2] = rmse_d / fmax(rmse_l, thr);
    m[3] = eb_threshold != 0.0f ? fabs(eb / nn) / (double)eb_threshold * 100.0 : 0.0;
    m[4] = max_d; m[5] = mean_d; m[6] = rmse_d; m[7] = max_l; m[8] = mean_l; m[9] = rmse_l;
}

int orc_num_threads(void)
{
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

/*
 * MoE token un-permute: out[t] = sum over the top_k routes of token t of
 * permuted[sorted_indices[t*top_k + j]] * probs[t*top_k + j], as the reference
 * kernel computes it (examples/aux_ops/moe_token_unpermute/moe_token_unpermute.h:
 * 235-279): fp32 throughout, the product of each route rounded on its own
 * (Muls, :315 / :330) before it is added (Add, :333), route 0 assigns (or the
 * sum starts at zero when its index is not below `rows`, :247-258), routes
 * with an index outside [0, rows) are skipped, and the result is cast with
 * CAST_RINT (:353) = round to nearest even.  probs may be NULL (no weighting).
 * The reference's Python fallback (gen_data_moe.py:60-70) accumulates in the
 * token dtype instead and takes the inverse permutation as its index; it is not
 * what this function follows.
 * pinned by: a torch restatement with one separately rounded fp32 op per step,
 *            gather special case (top_k = 1, probs = 1), linearity in probs by
 *            powers of two.
 */
__attribute__((optimize("fp-contract=off")))
int orc_moe_token_unpermute(const uint16_t *permuted, const int32_t *sorted_indices, const float *probs,
                            int64_t rows, int64_t tokens, int64_t hidden, int top_k, uint16_t *out)
{
#pragma omp parallel for schedule(static)
    for (int64_t t = 0; t < tokens; t++) {
        for (int64_t h = 0; h < hidden; h++) {
            float acc = 0.0f;
            for (int j = 0; j < top_k; j++) {
                const int64_t idx = sorted_indices[t * top_k + j];
                if (idx < 0 || idx >= rows) continue;
                volatile float v = orc_bf16_to_f32(permuted[idx * hidden + h]);
                if (probs) v = v * probs[t * top_k + j];
                if (j == 0) acc = v;
                else acc = acc + v;
            }
            out[t * hidden + h] = orc_f32_to_bf16(acc);
        }
    }
    return 0;
}
