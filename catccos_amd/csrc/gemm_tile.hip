// Tiled MFMA GEMM family for gfx950 (B stored K-contiguous, i.e. trans_b = 1):
//   int8 x int8 -> int32   v_mfma_i32_32x32x32_i8          + dequant / dequant+SwiGLU epilogue
//   MXFP8 / MXFP4          v_mfma_scale_f32_32x32x64_f8f6f4 with per-lane E8M0 scale operands
// One persistent workgroup per CU walks a global list of 256x256 output tiles built from the
// prefix sums of the group sizes (a dense problem is one group).  Per K-step of 128 bytes the
// A and B panels go global -> LDS with 16-byte direct-to-LDS loads (no VGPR round trip),
// double buffered; four waves each own a 128x128 quadrant as 4x4 MFMA tiles held in
// registers; epilogues run on the accumulators before the bf16 store.
//
// Stands in for Catlass::Gemm::Block::BlockMmadTla<MmadMx<...>> as instantiated in
// examples/ascend950_fp4_mx_alltoallv_grouped_matmul/ascend950_fp4_mx_alltoallv_grouped_matmul_device.h:59-71,
// FixpipeBlockMmad (include/catccos/dgemm/block/block_mmad_preload_fixpipe.hpp:151-379), the
// tile loop of BlockMmadSchedulerAllToAllVAllGather
// (include/catccos/dgemm/block/block_scheduler_alltoallv_allgather.hpp:122-168) and the epilogues
// include/catccos/epilogue/block/block_epilogue_per_token_dequant[_swiglu].hpp.
#include <type_traits>
#include <utility>

#include "common.h"
#include "gemm_common.h"
#include "mx_formats.h"

namespace cch {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v8i __attribute__((ext_vector_type(8)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v16f __attribute__((ext_vector_type(16)));

constexpr int BM = 256, BN = 256;      // output tile
constexpr int BKB = 128;               // bytes of K per step (per row)
constexpr int TILE_BYTES = BM * BKB;   // one operand panel of one stage: 32 KiB
constexpr int STAGE_BYTES = 2 * TILE_BYTES;
constexpr int NSTAGE = 2;
constexpr int TILE_THREADS = 256;
constexpr int LDS_BYTES = NSTAGE * STAGE_BYTES;  // 128 KiB of the CU's 160 KiB

template <int KIND> struct KindTraits;
template <> struct KindTraits<KIND_I8> { static constexpr int SUBSTEPS = 4, ELEMS_PER_BYTE = 1; using Acc = v16i; };
template <> struct KindTraits<KIND_F8> { static constexpr int SUBSTEPS = 2, ELEMS_PER_BYTE = 1; using Acc = v16f; };
template <> struct KindTraits<KIND_F4> { static constexpr int SUBSTEPS = 4, ELEMS_PER_BYTE = 2; using Acc = v16f; };

extern __shared__ __attribute__((aligned(1024))) uint8_t smem[];

// Calls f(std::integral_constant<int, 0>) ... f(std::integral_constant<int, N-1>): loop indices
// that have to reach the MFMA builtins as immediates.
template <int... I, class F>
__device__ __forceinline__ void static_for_impl(std::integer_sequence<int, I...>, F &&f)
{
    (f(std::integral_constant<int, I>{}), ...);
}
template <int N, class F> __device__ __forceinline__ void static_for(F &&f)
{
    static_for_impl(std::make_integer_sequence<int, N>{}, f);
}

__device__ __forceinline__ void load16_to_lds(const uint8_t *src, uint32_t lds_offset)
{
    __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)src,
                                     (__attribute__((address_space(3))) void *)(smem + lds_offset), 16, 0, 0);
}

__device__ __forceinline__ v4i lds_read16(uint32_t off) { return *reinterpret_cast<const v4i *>(smem + off); }

// One operand panel of a K-step: 256 rows x 128 bytes, row r at r*128, 16-byte chunk c of a row
// stored at chunk position c ^ (r & 7).  A wave moves 8 rows (1 KiB) per instruction: lane l
// lands at row l/8, position l%8, so it must fetch chunk (l%8) ^ (l/8 % 8) of that row.
// `off[j]` holds, per lane, the byte offset of its source row + chunk for instruction j.
template <int NJ>
__device__ __forceinline__ void issue_panel(const uint8_t *base, const uint32_t (&off)[NJ], int kbyte, uint32_t lds_panel,
                                            int wave)
{
#pragma unroll
    for (int j = 0; j < NJ; j++) load16_to_lds(base + off[j] + kbyte, lds_panel + (uint32_t)((wave * NJ + j) * 1024));
}

template <int KIND, int EPI>
__global__ __launch_bounds__(TILE_THREADS, 1) void gemm_tile_kernel(GemmProblem p)
{
    using KT = KindTraits<KIND>;
    using Acc = typename KT::Acc;
    constexpr bool MX = KIND != KIND_I8;
    constexpr bool SWIGLU = EPI == EPI_DEQUANT_SWIGLU;
    constexpr int BN_OUT = SWIGLU ? BN / 2 : BN;  // output columns per tile
    constexpr int SCALE_DW = KIND == KIND_F4 ? 2 : 1;  // scale dwords per row per K-step
    constexpr int NJ = TILE_BYTES / 1024 / 4;     // direct-to-LDS instructions per wave per panel

    __shared__ GroupTable tab;
    if (threadIdx.x == 0) build_group_table(tab, p.group_sizes, p.num_groups, p.T, BM);
    __syncthreads();

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int wm = wave >> 1, wn = wave & 1;
    const int r = lane & 31, g = lane >> 5;

    const int lda = p.K / KT::ELEMS_PER_BYTE;  // bytes per row of A and of B (K-contiguous)
    const int ksteps = lda / BKB;
    const int n_tiles = (p.n_out + BN_OUT - 1) / BN_OUT;
    const int total_tiles = tab.tile_start[p.num_groups + 1] * n_tiles;

    // LDS read offsets of this lane inside a panel: row (quadrant base + r), swizzle r & 7.
    const uint32_t rd_row = (uint32_t)r * BKB;
    const uint32_t swz = (uint32_t)(r & 7);

    for (int t = blockIdx.x; t < total_tiles; t += gridDim.x) {
        const int tr = t / n_tiles, nt = t - tr * n_tiles;
        const int e = find_group(tab, p.num_groups, tr);
        const int m0 = tab.row_start[e] + (tr - tab.tile_start[e]) * BM;
        const int m_end = tab.row_start[e + 1];
        const int j0 = nt * BN_OUT;  // first output column of the tile

        if (e == p.num_groups) {  // rows that belong to no expert: zeros
            for (int i = threadIdx.x; i < BM * BN_OUT; i += TILE_THREADS) {
                const int rr = m0 + i / BN_OUT, cc = j0 + i % BN_OUT;
                if (rr < m_end && cc < p.n_out) p.out[(size_t)rr * p.n_out + cc] = 0;
            }
            continue;
        }

        const uint8_t *a_base = p.a + (size_t)m0 * lda;
        const uint8_t *b_base = p.b + (size_t)e * p.b_stride;

        // Source offsets of the direct-to-LDS loads.  Rows past the edge re-read the last valid
        // row; their products land in accumulators that are never stored.
        uint32_t off_a[NJ], off_b[NJ];
#pragma unroll
        for (int j = 0; j < NJ; j++) {
            const int row = (wave * NJ + j) * 8 + (lane >> 3);
            const uint32_t chunk = (uint32_t)((lane & 7) ^ (row & 7));
            const int arow = min(row, m_end - 1 - m0);
            off_a[j] = (uint32_t)arow * (uint32_t)lda + chunk * 16u;
            int col;  // B row (= logical column) feeding tile row `row`
            if (SWIGLU) {
                const int q = row >> 6;  // 0: gate wn=0, 1: up wn=0, 2: gate wn=1, 3: up wn=1
                col = (q & 1) * p.n_out + j0 + (q >> 1) * 64 + (row & 63);
                col = min(col, (q & 1) * p.n_out + p.n_out - 1);
            } else {
                col = min(j0 + row, p.N - 1);
            }
            off_b[j] = (uint32_t)col * (uint32_t)lda + chunk * 16u;
        }

        // Per-lane scale sources (MX): lane (r, g) supplies the scale of row/column r of each
        // 32-wide MFMA sub-tile for K-block g of the current 64-wide MFMA step.
        const uint8_t *sa_ptr[4], *sb_ptr[4];
        if (MX) {
#pragma unroll
            for (int s = 0; s < 4; s++) {
                const int arow = min(m0 + wm * 128 + s * 32 + r, m_end - 1);
                sa_ptr[s] = p.sa + (size_t)arow * p.sld;
                const int col = min(j0 + wn * 128 + s * 32 + r, p.N - 1);
                sb_ptr[s] = p.sb + (size_t)e * p.sb_stride + (size_t)col * p.sld;
            }
        }

        Acc acc[4][4];
#pragma unroll
        for (int i = 0; i < 4; i++)
#pragma unroll
            for (int j = 0; j < 4; j++)
#pragma unroll
                for (int x = 0; x < 16; x++) acc[i][j][x] = 0;

        uint32_t sca[2][4][SCALE_DW], scb[2][4][SCALE_DW];  // [parity of K-step][sub-tile][dword]
        auto load_scales = [&](int kt, auto parity) {
            constexpr int par = decltype(parity)::value;
            if (!MX) return;
#pragma unroll
            for (int s = 0; s < 4; s++)
#pragma unroll
                for (int d = 0; d < SCALE_DW; d++) {
                    sca[par][s][d] = *reinterpret_cast<const uint32_t *>(sa_ptr[s] + (kt * SCALE_DW + d) * 4) >> (8 * g);
                    scb[par][s][d] = *reinterpret_cast<const uint32_t *>(sb_ptr[s] + (kt * SCALE_DW + d) * 4) >> (8 * g);
                }
        };

        // prologue: stage 0 <- K-step 0
        __syncthreads();  // every wave is done with the previous tile's LDS contents
        issue_panel<NJ>(a_base, off_a, 0, 0, wave);
        issue_panel<NJ>(b_base, off_b, 0, TILE_BYTES, wave);
        load_scales(0, std::integral_constant<int, 0>{});

        auto kstep = [&](int kt, auto parity) {
            constexpr int st = decltype(parity)::value;
            __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): this wave's direct-to-LDS loads have landed
            __syncthreads();                      // ... and everybody else's; stage st^1 is free again
            if (kt + 1 < ksteps) {
                issue_panel<NJ>(a_base, off_a, (kt + 1) * BKB, (uint32_t)((st ^ 1) * STAGE_BYTES), wave);
                issue_panel<NJ>(b_base, off_b, (kt + 1) * BKB, (uint32_t)((st ^ 1) * STAGE_BYTES + TILE_BYTES), wave);
            }
            const uint32_t pa = (uint32_t)(st * STAGE_BYTES) + (uint32_t)(wm * 128) * BKB + rd_row;
            const uint32_t pb = (uint32_t)(st * STAGE_BYTES + TILE_BYTES) + (uint32_t)(wn * 128) * BKB + rd_row;

            if (kt + 1 < ksteps) load_scales(kt + 1, std::integral_constant<int, st ^ 1>{});

            static_for<KT::SUBSTEPS>([&](auto substep) {
                constexpr int ks = decltype(substep)::value;
                if constexpr (KIND == KIND_F8) {
                    v8i fa[4], fb[4];
                    const uint32_t c0 = (((uint32_t)(ks * 4 + g)) ^ swz) << 4, c1 = (((uint32_t)(ks * 4 + 2 + g)) ^ swz) << 4;
#pragma unroll
                    for (int s = 0; s < 4; s++) {
                        const v4i lo = lds_read16(pa + s * 32 * BKB + c0), hi = lds_read16(pa + s * 32 * BKB + c1);
                        fa[s] = (v8i){lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
                        const v4i lo2 = lds_read16(pb + s * 32 * BKB + c0), hi2 = lds_read16(pb + s * 32 * BKB + c1);
                        fb[s] = (v8i){lo2[0], lo2[1], lo2[2], lo2[3], hi2[0], hi2[1], hi2[2], hi2[3]};
                    }
                    const int cb = p.fmt == CCH_FMT_E5M2;
#pragma unroll
                    for (int i = 0; i < 4; i++)
#pragma unroll
                        for (int j = 0; j < 4; j++) {
                            const int sA = (int)sca[st][i][0], sB = (int)scb[st][j][0];
                            if (cb)
                                acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(fa[i], fb[j], acc[i][j], 1, 1, ks * 2, sA, ks * 2, sB);
                            else
                                acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(fa[i], fb[j], acc[i][j], 0, 0, ks * 2, sA, ks * 2, sB);
                        }
                } else {
                    v4i fa[4], fb[4];
                    const uint32_t c0 = (((uint32_t)(ks * 2 + g)) ^ swz) << 4;
#pragma unroll
                    for (int s = 0; s < 4; s++) {
                        fa[s] = lds_read16(pa + s * 32 * BKB + c0);
                        fb[s] = lds_read16(pb + s * 32 * BKB + c0);
                    }
#pragma unroll
                    for (int i = 0; i < 4; i++)
#pragma unroll
                        for (int j = 0; j < 4; j++) {
                            if constexpr (KIND == KIND_I8) {
                                acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[i], fb[j], acc[i][j], 0, 0, 0);
                            } else {
                                const v8i a8 = (v8i){fa[i][0], fa[i][1], fa[i][2], fa[i][3], 0, 0, 0, 0};
                                const v8i b8 = (v8i){fb[j][0], fb[j][1], fb[j][2], fb[j][3], 0, 0, 0, 0};
                                const int sA = (int)sca[st][i][ks >> 1], sB = (int)scb[st][j][ks >> 1];
                                acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a8, b8, acc[i][j], 4, 4, (ks & 1) * 2, sA, (ks & 1) * 2, sB);
                            }
                        }
                }
            });
        };
        for (int kt = 0; kt < ksteps; kt += 2) {
            kstep(kt, std::integral_constant<int, 0>{});
            if (kt + 1 < ksteps) kstep(kt + 1, std::integral_constant<int, 1>{});
        }

        // Epilogue on the accumulators.  Lane (r, g) holds, for sub-tile (i, j), column r and
        // rows (x/4)*8 + g*4 + x%4.
#pragma unroll
        for (int i = 0; i < 4; i++) {
#pragma unroll
            for (int x = 0; x < 16; x++) {
                const int row = m0 + wm * 128 + i * 32 + (x >> 2) * 8 + g * 4 + (x & 3);
                if (row >= m_end) continue;
                float tok = 1.0f;
                if (EPI != EPI_PLAIN) tok = p.per_tok[row];
                uint16_t *orow = p.out + (size_t)row * p.n_out;
                if (SWIGLU) {
#pragma unroll
                    for (int j = 0; j < 2; j++) {
                        const int oc = j0 + wn * 64 + j * 32 + r;
                        if (oc >= p.n_out) continue;
                        const float *pc = p.per_ch + (size_t)e * p.N;
                        const float gate = (float)acc[i][j][x] * pc[oc] * tok;
                        const float up = (float)acc[i][j + 2][x] * pc[oc + p.n_out] * tok;
                        orow[oc] = (uint16_t)f32_to_bf16_bits(gate * (1.0f / (1.0f + expf(-gate))) * up);
                    }
                } else {
#pragma unroll
                    for (int j = 0; j < 4; j++) {
                        const int oc = j0 + wn * 128 + j * 32 + r;
                        if (oc >= p.n_out) continue;
                        float v = (float)acc[i][j][x];
                        if (EPI == EPI_DEQUANT) v = v * tok * p.per_ch[(size_t)e * p.N + oc];
                        orow[oc] = (uint16_t)f32_to_bf16_bits(v);
                    }
                }
            }
        }
    }
}

template <int KIND, int EPI>
static int launch_tile_t(const GemmProblem &p, hipStream_t stream)
{
    static bool attr_set = false;
    auto kern = gemm_tile_kernel<KIND, EPI>;
    if (!attr_set) {
        CCH_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, LDS_BYTES));
        attr_set = true;
    }
    int dev = 0, cus = 0;
    CCH_HIP(hipGetDevice(&dev));
    CCH_HIP(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev));
    constexpr int bn_out = EPI == EPI_DEQUANT_SWIGLU ? BN / 2 : BN;
    const int64_t row_tiles = (p.T + BM - 1) / BM + (p.group_sizes ? p.num_groups : 0);  // upper bound
    const int64_t tiles = row_tiles * ((p.n_out + bn_out - 1) / bn_out);
    const unsigned grid = (unsigned)std::max<int64_t>(1, std::min<int64_t>(tiles, cus));
    hipLaunchKernelGGL(kern, dim3(grid), dim3(TILE_THREADS), LDS_BYTES, stream, p);
    return launch_status("gemm_tile_kernel");
}

// True when the tiled kernels take this problem; otherwise the caller uses the generic path.
bool gemm_tile_supports(const GemmProblem &p, int kind)
{
    const int epb = kind == KIND_F4 ? 2 : 1;
    if (!p.trans_b) return false;
    if (p.K <= 0 || p.K % (BKB * epb) != 0) return false;
    if (p.num_groups > MAX_GROUPS) return false;
    if ((int64_t)p.N * (p.K / epb) >= ((int64_t)1 << 31)) return false;  // 32-bit source offsets
    if (!aligned(p.a, 16) || !aligned(p.b, 16) || p.b_stride % 16 != 0) return false;
    if (kind != KIND_I8 && (!aligned(p.sa, 4) || !aligned(p.sb, 4) || p.sb_stride % 4 != 0 || p.sld % 4 != 0)) return false;
    return true;
}

int launch_gemm_tile(const GemmProblem &p, int kind, int epi, hipStream_t stream)
{
    if (kind == KIND_I8 && epi == EPI_DEQUANT) return launch_tile_t<KIND_I8, EPI_DEQUANT>(p, stream);
    if (kind == KIND_I8 && epi == EPI_DEQUANT_SWIGLU) return launch_tile_t<KIND_I8, EPI_DEQUANT_SWIGLU>(p, stream);
    if (kind == KIND_F8 && epi == EPI_PLAIN) return launch_tile_t<KIND_F8, EPI_PLAIN>(p, stream);
    if (kind == KIND_F4 && epi == EPI_PLAIN) return launch_tile_t<KIND_F4, EPI_PLAIN>(p, stream);
    return fail(CCH_ENOSUP, "no tiled GEMM kernel for kind %d with epilogue %d", kind, epi);
}

}  // namespace cch
