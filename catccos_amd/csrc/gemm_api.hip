// C ABI of the GEMM family: argument checks, problem description, kernel choice.
#include <atomic>
#include <cstring>

#include "common.h"
#include "gemm_common.h"

namespace cch {
int launch_gemm_naive(const GemmProblem &p, int kind, int epi, hipStream_t stream);
int launch_gemm_tile(const GemmProblem &p, int kind, int epi, hipStream_t stream);
const char *gemm_tile_unsupported(const GemmProblem &p, int kind, int epi);
bool quant_set_option(const char *name, int value);   // mx_quant.hip
extern std::atomic<int> g_route_three_launches;        // routing.hip

static std::atomic<int> g_force_generic{0};
static std::atomic<int> g_require_tiled{0};
static std::atomic<int> g_tile_order{-1};   // -1: chosen per problem
static std::atomic<int> g_nt_out{-1};      // -1: chosen per problem
static std::atomic<int> g_i8_fp16_step{0};

static int run(const GemmProblem &prob, int kind, int epi, hipStream_t stream)
{
    // the message of this thread describes this call only: a fall-back note of an earlier call must not outlive it
    clear_error();
    if (prob.T == 0 || prob.n_out == 0) return CCH_OK;
    GemmProblem p = prob;
    const int order = g_tile_order.load();
    p.tile_order = order >= 0 ? order : 2;
    p.i8_fp16_step = g_i8_fp16_step.load() != 0;
    const int nto = g_nt_out.load();
    p.nt_out = nto >= 0 ? nto : (kind == KIND_F4);
    const bool forced = g_force_generic.load() != 0;
    const char *why = forced ? "force_generic_gemm is set" : gemm_tile_unsupported(p, kind, epi);
    if (why == nullptr) return launch_gemm_tile(p, kind, epi, stream);
    if (g_require_tiled.load())
        return fail(CCH_ENOSUP, "the tiled MFMA kernels do not take this problem (T=%d N=%d K=%d trans_b=%d: %s) and "
                                "require_tiled_gemm is set", p.T, p.N, p.K, p.trans_b, why);
    // The generic kernels are orders of magnitude slower: leave a note for cch_last_error() on every
    // such call (the call still succeeds) and say it once per process on stderr.
    fail(CCH_OK, "note: T=%d N=%d K=%d trans_b=%d ran on the one-thread-per-element kernels: %s", p.T, p.N, p.K, p.trans_b, why);
    if (!forced) {
        static std::atomic<int> told{0};
        if (told.exchange(1) == 0)
            fprintf(stderr, "[WARN] catccos_hip: GEMM T=%d N=%d K=%d trans_b=%d falls back to the generic kernels (%s); "
                            "further fall-backs are reported through cch_last_error() only\n", p.T, p.N, p.K, p.trans_b, why);
    }
    return launch_gemm_naive(p, kind, epi, stream);
}

static int check_shape(const char *who, int64_t t, int64_t n, int64_t k)
{
    CCH_REQUIRE(t >= 0 && n >= 0 && k >= 0, "%s: negative shape", who);
    CCH_REQUIRE(t < ((int64_t)1 << 31) && n < ((int64_t)1 << 31) && k < ((int64_t)1 << 31), "%s: shape too large", who);
    return CCH_OK;
}
}  // namespace cch

using namespace cch;

extern "C" {

int cch_set_option(const char *name, int value)
{
    CCH_REQUIRE(name != nullptr, "cch_set_option: null name");
    if (strcmp(name, "force_generic_gemm") == 0) {
        g_force_generic.store(value);
        return CCH_OK;
    }
    if (strcmp(name, "require_tiled_gemm") == 0) {
        g_require_tiled.store(value);
        return CCH_OK;
    }
    if (strcmp(name, "gemm_nt_output") == 0) {
        g_nt_out.store(value);
        return CCH_OK;
    }
    if (strcmp(name, "i8_epilogue_fp16_step") == 0) {
        g_i8_fp16_step.store(value);
        return CCH_OK;
    }
    if (strcmp(name, "gemm_tile_order") == 0) {
        g_tile_order.store(value);
        return CCH_OK;
    }
    if (strcmp(name, "routing_three_launches") == 0) {
        g_route_three_launches.store(value);
        return CCH_OK;
    }
    if (quant_set_option(name, value)) return CCH_OK;
    return fail(CCH_EINVAL, "cch_set_option: unknown option %s", name);
}

int cch_gemm_i8_dequant(const void *a, const void *b, const float *per_tok, const float *per_ch, void *out, int64_t m,
                        int64_t n, int64_t k, int trans_b, void *stream)
{
    return cch_gemm_i8_dequant_out(a, b, per_tok, per_ch, out, m, n, k, trans_b, CCH_OUT_BF16, stream);
}

int cch_gemm_i8_dequant_out(const void *a, const void *b, const float *per_tok, const float *per_ch, void *out, int64_t m,
                            int64_t n, int64_t k, int trans_b, int out_dtype, void *stream)
{
    int rc = check_shape("cch_gemm_i8_dequant", m, n, k);
    if (rc) return rc;
    CCH_REQUIRE(out_dtype == CCH_OUT_BF16 || out_dtype == CCH_OUT_FP16, "cch_gemm_i8_dequant: out_dtype %d", out_dtype);
    CCH_REQUIRE(trans_b == 0 || trans_b == 1, "cch_gemm_i8_dequant: trans_b %d", trans_b);
    if (m == 0 || n == 0) return CCH_OK;
    CCH_REQUIRE(out && per_tok && per_ch && (k == 0 || (a && b)), "cch_gemm_i8_dequant: null pointer");
    GemmProblem p{};
    p.a = static_cast<const uint8_t *>(a);
    p.b = static_cast<const uint8_t *>(b);
    p.per_tok = per_tok;
    p.per_ch = per_ch;
    p.out = static_cast<uint16_t *>(out);
    p.num_groups = 1;
    p.T = (int)m; p.N = (int)n; p.K = (int)k; p.n_out = (int)n;
    p.trans_b = trans_b;
    p.out_fp16 = out_dtype == CCH_OUT_FP16;
    return run(p, KIND_I8, EPI_DEQUANT, static_cast<hipStream_t>(stream));
}

int cch_gmm_i8_dequant_swiglu(const void *x, const void *w, const int32_t *group_sizes, const float *per_tok,
                              const float *per_ch, void *out, int64_t num_experts, int64_t t, int64_t n, int64_t k,
                              int trans_b, void *stream)
{
    return cch_gmm_i8_dequant_swiglu_out(x, w, group_sizes, per_tok, per_ch, out, num_experts, t, n, k, trans_b, CCH_OUT_BF16, stream);
}

int cch_gmm_i8_dequant_swiglu_out(const void *x, const void *w, const int32_t *group_sizes, const float *per_tok,
                                  const float *per_ch, void *out, int64_t num_experts, int64_t t, int64_t n, int64_t k,
                                  int trans_b, int out_dtype, void *stream)
{
    int rc = check_shape("cch_gmm_i8_dequant_swiglu", t, n, k);
    if (rc) return rc;
    CCH_REQUIRE(out_dtype == CCH_OUT_BF16 || out_dtype == CCH_OUT_FP16, "cch_gmm_i8_dequant_swiglu: out_dtype %d", out_dtype);
    CCH_REQUIRE(trans_b == 0 || trans_b == 1, "cch_gmm_i8_dequant_swiglu: trans_b %d", trans_b);
    CCH_REQUIRE(n % 2 == 0, "cch_gmm_i8_dequant_swiglu: n=%lld must be even (gate | up halves)", (long long)n);
    CCH_REQUIRE(num_experts >= 1 && num_experts <= MAX_GROUPS, "cch_gmm_i8_dequant_swiglu: num_experts=%lld outside 1..%d", (long long)num_experts, MAX_GROUPS);
    if (t == 0 || n == 0) return CCH_OK;
    CCH_REQUIRE(out && per_tok && per_ch && group_sizes && (k == 0 || (x && w)), "cch_gmm_i8_dequant_swiglu: null pointer");
    GemmProblem p{};
    p.a = static_cast<const uint8_t *>(x);
    p.b = static_cast<const uint8_t *>(w);
    p.per_tok = per_tok;
    p.per_ch = per_ch;
    p.out = static_cast<uint16_t *>(out);
    p.group_sizes = group_sizes;
    p.num_groups = (int)num_experts;
    p.T = (int)t; p.N = (int)n; p.K = (int)k; p.n_out = (int)(n / 2);
    p.trans_b = trans_b;
    p.b_stride = n * k;
    p.out_fp16 = out_dtype == CCH_OUT_FP16;
    return run(p, KIND_I8, EPI_DEQUANT_SWIGLU, static_cast<hipStream_t>(stream));
}

int cch_gmm_i8_dequant_swiglu_mx(const void *x, const void *w, const int32_t *group_sizes, const float *per_tok,
                                 const float *per_ch, void *payload, void *scales, int64_t num_experts, int64_t t, int64_t n,
                                 int64_t k, int trans_b, int fmt, void *stream)
{
    int rc = check_shape("cch_gmm_i8_dequant_swiglu_mx", t, n, k);
    if (rc) return rc;
    CCH_REQUIRE(fmt == CCH_FMT_E4M3 || fmt == CCH_FMT_E5M2 || fmt == CCH_FMT_E2M1, "cch_gmm_i8_dequant_swiglu_mx: fmt %d (E4M3, E5M2 or E2M1)", fmt);
    CCH_REQUIRE(trans_b == 0 || trans_b == 1, "cch_gmm_i8_dequant_swiglu_mx: trans_b %d", trans_b);
    CCH_REQUIRE(n % 2 == 0, "cch_gmm_i8_dequant_swiglu_mx: n=%lld must be even (gate | up halves)", (long long)n);
    CCH_REQUIRE(fmt != CCH_FMT_E2M1 || n % 4 == 0, "cch_gmm_i8_dequant_swiglu_mx: n=%lld: FP4 rows hold two codes per byte", (long long)n);
    CCH_REQUIRE(num_experts >= 1 && num_experts <= MAX_GROUPS, "cch_gmm_i8_dequant_swiglu_mx: num_experts=%lld outside 1..%d", (long long)num_experts, MAX_GROUPS);
    if (t == 0 || n == 0) return CCH_OK;
    CCH_REQUIRE(payload && scales && per_tok && per_ch && group_sizes && (k == 0 || (x && w)), "cch_gmm_i8_dequant_swiglu_mx: null pointer");
    GemmProblem p{};
    p.a = static_cast<const uint8_t *>(x);
    p.b = static_cast<const uint8_t *>(w);
    p.per_tok = per_tok;
    p.per_ch = per_ch;
    p.out = static_cast<uint16_t *>(payload);
    p.out_scales = static_cast<uint8_t *>(scales);
    p.mx_out = 1;
    p.mx_out_fmt = fmt;
    p.group_sizes = group_sizes;
    p.num_groups = (int)num_experts;
    p.T = (int)t; p.N = (int)n; p.K = (int)k; p.n_out = (int)(n / 2);
    p.mx_out_sld = (int)(2 * ((p.n_out + 63) / 64));
    p.trans_b = trans_b;
    p.b_stride = n * k;
    return run(p, KIND_I8, EPI_DEQUANT_SWIGLU, static_cast<hipStream_t>(stream));
}

int cch_gmm_i8_dequant(const void *x, const void *w, const int32_t *group_sizes, const float *per_tok, const float *per_ch,
                       void *out, int64_t num_experts, int64_t t, int64_t n, int64_t k, int trans_b, void *stream)
{
    return cch_gmm_i8_dequant_out(x, w, group_sizes, per_tok, per_ch, out, num_experts, t, n, k, trans_b, CCH_OUT_BF16, stream);
}

int cch_gmm_i8_dequant_out(const void *x, const void *w, const int32_t *group_sizes, const float *per_tok, const float *per_ch,
                           void *out, int64_t num_experts, int64_t t, int64_t n, int64_t k, int trans_b, int out_dtype,
                           void *stream)
{
    int rc = check_shape("cch_gmm_i8_dequant", t, n, k);
    if (rc) return rc;
    CCH_REQUIRE(out_dtype == CCH_OUT_BF16 || out_dtype == CCH_OUT_FP16, "cch_gmm_i8_dequant: out_dtype %d", out_dtype);
    CCH_REQUIRE(trans_b == 0 || trans_b == 1, "cch_gmm_i8_dequant: trans_b %d", trans_b);
    CCH_REQUIRE(num_experts >= 1 && num_experts <= MAX_GROUPS, "cch_gmm_i8_dequant: num_experts=%lld outside 1..%d", (long long)num_experts, MAX_GROUPS);
    if (t == 0 || n == 0) return CCH_OK;
    CCH_REQUIRE(out && per_tok && per_ch && group_sizes && (k == 0 || (x && w)), "cch_gmm_i8_dequant: null pointer");
    GemmProblem p{};
    p.a = static_cast<const uint8_t *>(x);
    p.b = static_cast<const uint8_t *>(w);
    p.per_tok = per_tok;
    p.per_ch = per_ch;
    p.out = static_cast<uint16_t *>(out);
    p.group_sizes = group_sizes;
    p.num_groups = (int)num_experts;
    p.T = (int)t; p.N = (int)n; p.K = (int)k; p.n_out = (int)n;
    p.trans_b = trans_b;
    p.b_stride = n * k;
    p.out_fp16 = out_dtype == CCH_OUT_FP16;
    return run(p, KIND_I8, EPI_DEQUANT, static_cast<hipStream_t>(stream));
}

static int mx_problem(const char *who, GemmProblem &p, const void *a, const void *sa, const void *b, const void *sb,
                      const int32_t *group_sizes, void *out, int64_t num_experts, int64_t t, int64_t n, int64_t k,
                      int fmt, int trans_b, int *kind)
{
    int rc = check_shape(who, t, n, k);
    if (rc) return rc;
    CCH_REQUIRE(trans_b == 0 || trans_b == 1, "%s: trans_b %d", who, trans_b);
    CCH_REQUIRE(fmt == CCH_FMT_E4M3 || fmt == CCH_FMT_E5M2 || fmt == CCH_FMT_E2M1, "%s: unknown format %d", who, fmt);
    CCH_REQUIRE(num_experts >= 1 && num_experts <= MAX_GROUPS, "%s: num_experts=%lld outside 1..%d", who, (long long)num_experts, MAX_GROUPS);
    CCH_REQUIRE(t == 0 || n == 0 || (a && sa && b && sb && out) || k == 0, "%s: null pointer", who);
    const bool fp4 = fmt == CCH_FMT_E2M1;
    CCH_REQUIRE(!fp4 || (k % 2 == 0 && n % 2 == 0), "%s: FP4 needs even k and n", who);
    p.a = static_cast<const uint8_t *>(a);
    p.sa = static_cast<const uint8_t *>(sa);
    p.b = static_cast<const uint8_t *>(b);
    p.sb = static_cast<const uint8_t *>(sb);
    p.out = static_cast<uint16_t *>(out);
    p.group_sizes = group_sizes;
    p.num_groups = (int)num_experts;
    p.T = (int)t; p.N = (int)n; p.K = (int)k; p.n_out = (int)n;
    p.fmt = fmt;
    p.trans_b = trans_b;
    p.sld = (int)(2 * ((k + 63) / 64));
    p.b_stride = fp4 ? n * k / 2 : n * k;
    p.sb_stride = (int64_t)p.sld * n;
    *kind = fp4 ? KIND_F4 : KIND_F8;
    return CCH_OK;
}

int cch_mx_gemm(const void *a, const void *sa, const void *b, const void *sb, void *out, int64_t m, int64_t n, int64_t k,
                int fmt, int trans_b, void *stream)
{
    return cch_mx_gemm_out(a, sa, b, sb, out, m, n, k, fmt, trans_b, CCH_OUT_BF16, stream);
}

int cch_mx_gemm_out(const void *a, const void *sa, const void *b, const void *sb, void *out, int64_t m, int64_t n, int64_t k,
                    int fmt, int trans_b, int out_dtype, void *stream)
{
    GemmProblem p{};
    int kind = 0;
    CCH_REQUIRE(out_dtype == CCH_OUT_BF16 || out_dtype == CCH_OUT_FP16, "cch_mx_gemm: out_dtype %d", out_dtype);
    int rc = mx_problem("cch_mx_gemm", p, a, sa, b, sb, nullptr, out, 1, m, n, k, fmt, trans_b, &kind);
    if (rc) return rc;
    p.out_fp16 = out_dtype == CCH_OUT_FP16;
    return run(p, kind, EPI_PLAIN, static_cast<hipStream_t>(stream));
}

int cch_mx_gmm(const void *a, const void *sa, const void *b, const void *sb, const int32_t *group_sizes, void *out,
               int64_t num_experts, int64_t t, int64_t n, int64_t k, int fmt, int trans_b, void *stream)
{
    GemmProblem p{};
    int kind = 0;
    CCH_REQUIRE(group_sizes != nullptr || t == 0, "cch_mx_gmm: null group_sizes");
    int rc = mx_problem("cch_mx_gmm", p, a, sa, b, sb, group_sizes, out, num_experts, t, n, k, fmt, trans_b, &kind);
    if (rc) return rc;
    return run(p, kind, EPI_PLAIN, static_cast<hipStream_t>(stream));
}

int cch_mx_gmm_swiglu(const void *a, const void *sa, const void *b, const void *sb, const int32_t *group_sizes, void *out,
                      int64_t num_experts, int64_t t, int64_t n, int64_t k, int fmt, int trans_b, int out_dtype, void *stream)
{
    GemmProblem p{};
    int kind = 0;
    CCH_REQUIRE(out_dtype == CCH_OUT_BF16 || out_dtype == CCH_OUT_FP16, "cch_mx_gmm_swiglu: out_dtype %d", out_dtype);
    CCH_REQUIRE(group_sizes != nullptr || t == 0, "cch_mx_gmm_swiglu: null group_sizes");
    CCH_REQUIRE(n % 2 == 0, "cch_mx_gmm_swiglu: n=%lld must be even (gate | up halves)", (long long)n);
    int rc = mx_problem("cch_mx_gmm_swiglu", p, a, sa, b, sb, group_sizes, out, num_experts, t, n, k, fmt, trans_b, &kind);
    if (rc) return rc;
    p.n_out = (int)(n / 2);
    p.out_fp16 = out_dtype == CCH_OUT_FP16;
    return run(p, kind, EPI_SWIGLU, static_cast<hipStream_t>(stream));
}

int cch_mx_gmm_swiglu_mx(const void *a, const void *sa, const void *b, const void *sb, const int32_t *group_sizes, void *payload,
                         void *scales, int64_t num_experts, int64_t t, int64_t n, int64_t k, int fmt, int trans_b, int out_fmt,
                         void *stream)
{
    GemmProblem p{};
    int kind = 0;
    CCH_REQUIRE(out_fmt == CCH_FMT_E4M3 || out_fmt == CCH_FMT_E5M2 || out_fmt == CCH_FMT_E2M1, "cch_mx_gmm_swiglu_mx: out_fmt %d (E4M3, E5M2 or E2M1)",
                out_fmt);
    CCH_REQUIRE(group_sizes != nullptr || t == 0, "cch_mx_gmm_swiglu_mx: null group_sizes");
    CCH_REQUIRE(n % 2 == 0, "cch_mx_gmm_swiglu_mx: n=%lld must be even (gate | up halves)", (long long)n);
    CCH_REQUIRE(out_fmt != CCH_FMT_E2M1 || n % 4 == 0, "cch_mx_gmm_swiglu_mx: n=%lld: FP4 rows hold two codes per byte", (long long)n);
    CCH_REQUIRE(t == 0 || n == 0 || scales != nullptr, "cch_mx_gmm_swiglu_mx: null pointer");
    int rc = mx_problem("cch_mx_gmm_swiglu_mx", p, a, sa, b, sb, group_sizes, payload, num_experts, t, n, k, fmt, trans_b, &kind);
    if (rc) return rc;
    p.n_out = (int)(n / 2);
    p.out_scales = static_cast<uint8_t *>(scales);
    p.mx_out = 1;
    p.mx_out_fmt = out_fmt;
    p.mx_out_sld = (int)(2 * ((p.n_out + 63) / 64));
    return run(p, kind, EPI_SWIGLU, static_cast<hipStream_t>(stream));
}

int cch_mx_gmm_swiglu_mx_packed(const void *packed_a, const void *b, const void *sb, const int32_t *group_sizes, void *payload,
                                void *scales, int64_t num_experts, int64_t t, int64_t n, int64_t k, int fmt, int trans_b, int out_fmt,
                                void *stream)
{
    GemmProblem p{};
    int kind = 0;
    CCH_REQUIRE(out_fmt == CCH_FMT_E4M3 || out_fmt == CCH_FMT_E5M2 || out_fmt == CCH_FMT_E2M1,
                "cch_mx_gmm_swiglu_mx_packed: out_fmt %d (E4M3, E5M2 or E2M1)", out_fmt);
    CCH_REQUIRE(group_sizes != nullptr || t == 0, "cch_mx_gmm_swiglu_mx_packed: null group_sizes");
    CCH_REQUIRE(n % 2 == 0, "cch_mx_gmm_swiglu_mx_packed: n=%lld must be even (gate | up halves)", (long long)n);
    CCH_REQUIRE(out_fmt != CCH_FMT_E2M1 || n % 4 == 0, "cch_mx_gmm_swiglu_mx_packed: n=%lld: FP4 rows hold two codes per byte", (long long)n);
    CCH_REQUIRE(t == 0 || n == 0 || scales != nullptr, "cch_mx_gmm_swiglu_mx_packed: null pointer");
    // a packed row: payload bytes, then the padded E8M0 scales (what cch_mx_quant_scatter_packed writes)
    const int64_t payload_bytes = fmt == CCH_FMT_E2M1 ? (k + 1) / 2 : k, row_bytes = payload_bytes + 2 * ((k + 63) / 64);
    const uint8_t *rows = static_cast<const uint8_t *>(packed_a);
    int rc = mx_problem("cch_mx_gmm_swiglu_mx_packed", p, rows, rows ? rows + payload_bytes : nullptr, b, sb, group_sizes, payload, num_experts, t, n,
                        k, fmt, trans_b, &kind);
    if (rc) return rc;
    p.a_pitch = row_bytes;
    p.sa_pitch = row_bytes;
    p.n_out = (int)(n / 2);
    p.out_scales = static_cast<uint8_t *>(scales);
    p.mx_out = 1;
    p.mx_out_fmt = out_fmt;
    p.mx_out_sld = (int)(2 * ((p.n_out + 63) / 64));
    return run(p, kind, EPI_SWIGLU, static_cast<hipStream_t>(stream));
}

int cch_mx_gmm_mapped(const void *a, const void *sa, const void *b, const void *sb, const int32_t *group_sizes,
                      const int32_t *out_row_map, void *out, int64_t out_rows, int out_dtype, int64_t num_experts, int64_t t,
                      int64_t n, int64_t k, int fmt, int trans_b, void *stream)
{
    GemmProblem p{};
    int kind = 0;
    CCH_REQUIRE(group_sizes != nullptr || t == 0, "cch_mx_gmm_mapped: null group_sizes");
    CCH_REQUIRE(out_rows >= 0 && out_rows < ((int64_t)1 << 31), "cch_mx_gmm_mapped: out_rows=%lld", (long long)out_rows);
    CCH_REQUIRE(out_row_map != nullptr || out_rows == t, "cch_mx_gmm_mapped: without a row map out has t=%lld rows, not %lld",
                (long long)t, (long long)out_rows);
    CCH_REQUIRE(out_dtype == CCH_OUT_BF16 || out_dtype == CCH_OUT_FP16, "cch_mx_gmm_mapped: out_dtype %d", out_dtype);
    int rc = mx_problem("cch_mx_gmm_mapped", p, a, sa, b, sb, group_sizes, out, num_experts, t, n, k, fmt, trans_b, &kind);
    if (rc) return rc;
    p.out_row_map = out_row_map;
    p.out_rows = out_rows;
    p.out_fp16 = out_dtype == CCH_OUT_FP16;
    return run(p, kind, EPI_PLAIN, static_cast<hipStream_t>(stream));
}

}  // extern "C"
