// Tiled MFMA GEMM family for gfx950: which problems the kernels take, and the choice of the instantiation.
// The kernel template is gemm_tile_kernel.h; gemm_tile_<kind>_<layout>.hip instantiate it.
#include <algorithm>

#include "common.h"
#include "gemm_common.h"
#include "gemm_tile_shape.h"

namespace cch {

template <int KIND, int EPI, int FMT, int TB> int launch_tile_t(const GemmProblem &p, hipStream_t stream);
#define CCH_TILE_FAMILY(KIND, EPI, FMT) \
    extern template int launch_tile_t<KIND, EPI, FMT, 0>(const GemmProblem &, hipStream_t); \
    extern template int launch_tile_t<KIND, EPI, FMT, 1>(const GemmProblem &, hipStream_t);
CCH_TILE_FAMILY(KIND_I8, EPI_DEQUANT, 0)
CCH_TILE_FAMILY(KIND_I8, EPI_DEQUANT_SWIGLU, 0)
CCH_TILE_FAMILY(KIND_F8, EPI_PLAIN, CCH_FMT_E4M3)
CCH_TILE_FAMILY(KIND_F8, EPI_PLAIN, CCH_FMT_E5M2)
CCH_TILE_FAMILY(KIND_F8, EPI_SWIGLU, CCH_FMT_E4M3)
CCH_TILE_FAMILY(KIND_F8, EPI_SWIGLU, CCH_FMT_E5M2)
CCH_TILE_FAMILY(KIND_F4, EPI_PLAIN, CCH_FMT_E2M1)
CCH_TILE_FAMILY(KIND_F4, EPI_SWIGLU, CCH_FMT_E2M1)
#undef CCH_TILE_FAMILY

#ifdef CCH_PROF
// Measurement build: counters of the last tiled launch (see gemm_tile_kernel.h).
int (*g_prof_copy)(uint64_t *, int) = nullptr;
extern "C" int cch_prof_read(uint64_t *host) { return g_prof_copy ? g_prof_copy(host, 0) : -1; }
extern "C" int cch_prof_read_tiles(uint64_t *host) { return g_prof_copy ? g_prof_copy(host, 1) : -1; }
extern "C" int cch_prof_read_entry(uint64_t *host) { return g_prof_copy ? g_prof_copy(host, 2) : -1; }
#endif

// nullptr when the tiled kernels take this problem; otherwise the precondition that failed (the
// caller then uses the generic path or reports it).
const char *gemm_tile_unsupported(const GemmProblem &p, int kind, int epi)
{
    const int epb = kind == KIND_F4 ? 2 : 1;
    const int64_t lda = p.K / epb;
    // rows are fetched in 16-byte pieces
    if (p.K < 1 || p.K % (16 * epb) != 0) return "K must be a multiple of 16 bytes per row";
    if (p.n_out % 8 != 0 || !aligned(p.out, 16)) return "output rows must take 16-byte stores (n_out % 8 == 0, out 16-byte aligned)";
    if (p.mx_out && ((epi != EPI_DEQUANT_SWIGLU && epi != EPI_SWIGLU) || p.n_out % 32 != 0 || p.out_fp16)) return "MX-quantised output needs whole 32-column blocks";
    if ((int64_t)BM * p.n_out * 2 >= ((int64_t)1 << 31)) return "output row tile beyond 2 GiB";
    // mapped output rows are addressed from the start of `out` with 32-bit offsets
    if (p.out_row_map && (epi != EPI_PLAIN || p.out_rows * p.n_out * 2 >= ((int64_t)1 << 31) || !aligned(p.out_row_map, 4)))
        return "mapped output beyond 2 GiB or misaligned row map";
    if (p.num_groups > MAX_GROUPS) return "more than 256 groups";
    if ((int64_t)p.N * lda >= ((int64_t)1 << 31)) return "one right-hand operand beyond 2 GiB (32-bit source offsets)";
    if ((int64_t)BM * std::max<int64_t>(lda, p.a_pitch) >= ((int64_t)1 << 31)) return "a row tile of the left-hand operand beyond 2 GiB";
    // (the 16-byte requests need dword alignment only: packed rows of K = 256 are 264 bytes long)
    if (p.a_pitch && (p.a_pitch % 4 != 0 || p.a_pitch < lda)) return "rows of the left-hand operand must start on 4-byte boundaries";
    if (p.sa_pitch && (p.sa_pitch % 2 != 0 || p.sa_pitch < p.sld)) return "scale rows of the left-hand operand must start on even addresses";
    if (!aligned(p.a, 16) || !aligned(p.b, 16) || p.b_stride % 16 != 0) return "operands must be 16-byte aligned";
    if (kind != KIND_I8 && (!aligned(p.sa, 4) || !aligned(p.sb, 4) || p.sb_stride % 2 != 0)) return "scale arrays must be 4-byte aligned";
    if (kind != KIND_I8 && ((int64_t)p.num_groups * p.N * p.sld >= ((int64_t)1 << 31) || (int64_t)p.T * std::max<int64_t>(p.sld, p.sa_pitch) >= ((int64_t)1 << 31)))
        return "scale arrays beyond 2 GiB";
    if (kind != KIND_I8 && p.sb_stride != (int64_t)p.N * p.sld) return "scale arrays of the right-hand operands must be back to back";
    if ((epi == EPI_DEQUANT || epi == EPI_DEQUANT_SWIGLU) && (!aligned(p.per_tok, 4) || !aligned(p.per_ch, 4))) return "dequantisation scales must be 4-byte aligned";
    if (!p.trans_b) {
        // [K, N] operands: rows of B are fetched in 16-byte pieces that start on 4-byte boundaries
        if ((p.N / epb) % 4 != 0) return "[K,N] operands need rows of a multiple of 4 bytes";
        if ((epi == EPI_DEQUANT_SWIGLU || epi == EPI_SWIGLU) && (p.n_out / epb) % 4 != 0) return "[K,N] SwiGLU operands need n/2 to be a multiple of 4";
    }
    return nullptr;
}

int launch_gemm_tile(const GemmProblem &p, int kind, int epi, hipStream_t stream)
{
    const bool tb = p.trans_b != 0;
    if (kind == KIND_I8 && epi == EPI_DEQUANT)
        return tb ? launch_tile_t<KIND_I8, EPI_DEQUANT, 0, 1>(p, stream) : launch_tile_t<KIND_I8, EPI_DEQUANT, 0, 0>(p, stream);
    if (kind == KIND_I8 && epi == EPI_DEQUANT_SWIGLU)
        return tb ? launch_tile_t<KIND_I8, EPI_DEQUANT_SWIGLU, 0, 1>(p, stream) : launch_tile_t<KIND_I8, EPI_DEQUANT_SWIGLU, 0, 0>(p, stream);
    if (kind == KIND_F8 && epi == EPI_PLAIN && p.fmt == CCH_FMT_E4M3)
        return tb ? launch_tile_t<KIND_F8, EPI_PLAIN, CCH_FMT_E4M3, 1>(p, stream) : launch_tile_t<KIND_F8, EPI_PLAIN, CCH_FMT_E4M3, 0>(p, stream);
    if (kind == KIND_F8 && epi == EPI_PLAIN && p.fmt == CCH_FMT_E5M2)
        return tb ? launch_tile_t<KIND_F8, EPI_PLAIN, CCH_FMT_E5M2, 1>(p, stream) : launch_tile_t<KIND_F8, EPI_PLAIN, CCH_FMT_E5M2, 0>(p, stream);
    if (kind == KIND_F4 && epi == EPI_PLAIN)
        return tb ? launch_tile_t<KIND_F4, EPI_PLAIN, CCH_FMT_E2M1, 1>(p, stream) : launch_tile_t<KIND_F4, EPI_PLAIN, CCH_FMT_E2M1, 0>(p, stream);
    if (kind == KIND_F8 && epi == EPI_SWIGLU && p.fmt == CCH_FMT_E4M3)
        return tb ? launch_tile_t<KIND_F8, EPI_SWIGLU, CCH_FMT_E4M3, 1>(p, stream) : launch_tile_t<KIND_F8, EPI_SWIGLU, CCH_FMT_E4M3, 0>(p, stream);
    if (kind == KIND_F8 && epi == EPI_SWIGLU && p.fmt == CCH_FMT_E5M2)
        return tb ? launch_tile_t<KIND_F8, EPI_SWIGLU, CCH_FMT_E5M2, 1>(p, stream) : launch_tile_t<KIND_F8, EPI_SWIGLU, CCH_FMT_E5M2, 0>(p, stream);
    if (kind == KIND_F4 && epi == EPI_SWIGLU)
        return tb ? launch_tile_t<KIND_F4, EPI_SWIGLU, CCH_FMT_E2M1, 1>(p, stream) : launch_tile_t<KIND_F4, EPI_SWIGLU, CCH_FMT_E2M1, 0>(p, stream);
    return fail(CCH_ENOSUP, "no tiled GEMM kernel for kind %d with epilogue %d, trans_b %d", kind, epi, p.trans_b);
}

}  // namespace cch
