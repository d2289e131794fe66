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
constexpr int TILE_THREADS = 512;      // 8 waves: 2 (M) x 4 (N), each owning 128 x 64 outputs
constexpr int WAVES_N = 4;
constexpr int WM = 128, WN = 64;       // wave tile
constexpr int MT = WM / 32, NT = WN / 32;  // 32x32 MFMA tiles per wave
constexpr int LDS_BYTES = NSTAGE * STAGE_BYTES;  // 128 KiB of the CU's 160 KiB
constexpr int SWZ_SHIFT = 1;           // chunk swizzle uses bits [SWZ_SHIFT, SWZ_SHIFT+3) of the row

// FMT: CCH_FMT_* for the MX kinds (fixes cbsz/blgp of the scaled MFMA), ignored for int8.
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

__device__ __forceinline__ int uniform(int v) { return __builtin_amdgcn_readfirstlane(v); }

// 16 bytes per lane, global -> LDS without passing through registers.  `base` is wave-uniform,
// `off` per lane; lane l of the wave lands at lds_offset + 16*l.
__device__ __forceinline__ void load16_to_lds(const uint8_t *base, uint32_t off, uint32_t lds_offset)
{
    __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)(base + off),
                                     (__attribute__((address_space(3))) void *)(smem + lds_offset), 16, 0, 0);
}

__device__ __forceinline__ v4i lds_read16(uint32_t off) { return *reinterpret_cast<const v4i *>(smem + off); }

__device__ __forceinline__ uint32_t swizzle_of_row(int row) { return (uint32_t)((row >> SWZ_SHIFT) & 7); }

// Two bf16 results that sit in neighbouring lanes (columns c, c+1) are paired so that every
// lane stores 4 bytes: even lanes keep row `lo`, odd lanes row `hi` of the pair of rows.
__device__ __forceinline__ void store_pair(uint16_t *out, size_t ld, int row_lo, int row_hi, int col, int row_end,
                                           int col_end, float v_lo, float v_hi, bool odd)
{
    const uint32_t keep = f32_to_bf16_bits(odd ? v_hi : v_lo);
    const uint32_t send = f32_to_bf16_bits(odd ? v_lo : v_hi);
    const uint32_t recv = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)send, 0xB1, 0xF, 0xF, true);  // swap lane pairs
    const int row = odd ? row_hi : row_lo;
    const int c0 = odd ? col - 1 : col;
    const uint32_t packed = odd ? (recv | (keep << 16)) : (keep | (recv << 16));
    if (row < row_end) {
        uint16_t *dst = out + (size_t)row * ld + c0;
        if (c0 + 1 < col_end && ((reinterpret_cast<uintptr_t>(dst) & 3) == 0)) {
            *reinterpret_cast<uint32_t *>(dst) = packed;
        } else {
            if (c0 < col_end) dst[0] = (uint16_t)packed;
            if (c0 + 1 < col_end) dst[1] = (uint16_t)(packed >> 16);
        }
    }
}

template <int KIND, int EPI, int FMT>
__global__ __launch_bounds__(TILE_THREADS) void gemm_tile_kernel(GemmProblem p)
{
    using KT = KindTraits<KIND>;
    using Acc = typename KT::Acc;
    constexpr bool MX = KIND != KIND_I8;
    constexpr bool SWIGLU = EPI == EPI_DEQUANT_SWIGLU;
    constexpr int BN_OUT = SWIGLU ? BN / 2 : BN;         // output columns per tile
    constexpr int WN_OUT = SWIGLU ? WN / 2 : WN;         // output columns per wave
    constexpr int SCALE_DW = KIND == KIND_F4 ? 2 : 1;    // scale dwords per row per K-step
    constexpr int NJ = TILE_BYTES / 1024 / (TILE_THREADS / 64);  // direct-to-LDS instructions per wave per panel
    constexpr int CBSZ = FMT == CCH_FMT_E2M1 ? 4 : (FMT == CCH_FMT_E5M2 ? 1 : 0);

    __shared__ GroupTable tab;
    if (threadIdx.x == 0) build_group_table(tab, p.group_sizes, p.num_groups, p.T, BM);
    __syncthreads();

    const int lane = threadIdx.x & 63;
    const int wave = uniform(threadIdx.x >> 6);
    const int wm = wave / WAVES_N, wn = wave % WAVES_N;
    const int r = lane & 31, g = lane >> 5;

    const int lda = p.K / KT::ELEMS_PER_BYTE;  // bytes per row of A and of B (K-contiguous)
    const int ksteps = lda / BKB;
    const int n_tiles = (p.n_out + BN_OUT - 1) / BN_OUT;
    const int total_tiles = uniform(tab.tile_start[p.num_groups + 1]) * n_tiles;

    // LDS read offsets of this lane inside a panel: rows (wave base + 32 s + r); the swizzle term
    // depends on r only because wave and sub-tile bases are multiples of 32.
    const uint32_t rd_a = (uint32_t)(wm * WM + r) * BKB, rd_b = (uint32_t)TILE_BYTES + (uint32_t)(wn * WN + r) * BKB;
    const uint32_t swz = swizzle_of_row(r);

    for (int t = blockIdx.x; t < total_tiles; t += gridDim.x) {
        const int tr = t / n_tiles, nt = t - tr * n_tiles;
        const int e = uniform(find_group(tab, p.num_groups, tr));
        const int m0 = uniform(tab.row_start[e] + (tr - tab.tile_start[e]) * BM);
        const int m_end = uniform(tab.row_start[e + 1]);
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

        // Source offsets of the direct-to-LDS loads: instruction j of this wave fills rows
        // (wave*NJ + j)*8 .. +7 of a panel; lane l lands at row l/8, chunk position l%8 and must
        // therefore fetch chunk (l%8) ^ swizzle(row).  Rows past the edge re-read the last valid
        // row; their products land in accumulators that are never stored.
        uint32_t off_a[NJ], off_b[NJ];
#pragma unroll
        for (int j = 0; j < NJ; j++) {
            const int row = (wave * NJ + j) * 8 + (lane >> 3);
            const uint32_t chunk = (uint32_t)(lane & 7) ^ swizzle_of_row(row);
            const int arow = min(row, m_end - 1 - m0);
            off_a[j] = (uint32_t)arow * (uint32_t)lda + chunk * 16u;
            int col;  // B row (= logical column) feeding tile row `row`
            if (SWIGLU) {
                // tile row = wn*64 + h*32 + c: h = 0 gate, 1 up; output column j0 + wn*32 + c
                const int h = (row >> 5) & 1;
                col = h * p.n_out + min(j0 + (row >> 6) * 32 + (row & 31), p.n_out - 1);
            } else {
                col = min(j0 + row, p.N - 1);
            }
            off_b[j] = (uint32_t)col * (uint32_t)lda + chunk * 16u;
        }

        // Per-lane scale sources (MX): lane (r, g) supplies the scale of row/column r of each
        // 32-wide MFMA sub-tile for K-block g of the current 64-wide MFMA step.
        uint32_t sa_off[MT], sb_off[NT];
        const uint8_t *sb_base = p.sb + (size_t)e * p.sb_stride;
        if (MX) {
#pragma unroll
            for (int s = 0; s < MT; s++) sa_off[s] = (uint32_t)min(m0 + wm * WM + s * 32 + r, m_end - 1) * (uint32_t)p.sld;
#pragma unroll
            for (int s = 0; s < NT; s++) sb_off[s] = (uint32_t)min(j0 + wn * WN + s * 32 + r, p.N - 1) * (uint32_t)p.sld;
        }

        Acc acc[MT][NT];
#pragma unroll
        for (int i = 0; i < MT; i++)
#pragma unroll
            for (int j = 0; j < NT; j++)
#pragma unroll
                for (int x = 0; x < 16; x++) acc[i][j][x] = 0;

        uint32_t sca[2][MT][SCALE_DW], scb[2][NT][SCALE_DW];  // [parity of K-step][sub-tile][dword]
        auto load_scales = [&](int kt, auto parity) {
            constexpr int par = decltype(parity)::value;
            if (!MX) return;
#pragma unroll
            for (int d = 0; d < SCALE_DW; d++) {
#pragma unroll
                for (int s = 0; s < MT; s++)
                    sca[par][s][d] = *reinterpret_cast<const uint32_t *>(p.sa + sa_off[s] + (kt * SCALE_DW + d) * 4);
#pragma unroll
                for (int s = 0; s < NT; s++)
                    scb[par][s][d] = *reinterpret_cast<const uint32_t *>(sb_base + sb_off[s] + (kt * SCALE_DW + d) * 4);
            }
        };
        auto issue_stage = [&](int kt, int st) {
            const uint32_t lds_a = (uint32_t)(st * STAGE_BYTES) + (uint32_t)(wave * NJ) * 1024u;
#pragma unroll
            for (int j = 0; j < NJ; j++) load16_to_lds(a_base + (size_t)kt * BKB, off_a[j], lds_a + j * 1024u);
#pragma unroll
            for (int j = 0; j < NJ; j++) load16_to_lds(b_base + (size_t)kt * BKB, off_b[j], lds_a + TILE_BYTES + j * 1024u);
        };

        // prologue: stage 0 <- K-step 0
        __syncthreads();  // every wave is done with the previous tile's LDS contents
        issue_stage(0, 0);
        load_scales(0, std::integral_constant<int, 0>{});

        auto kstep = [&](int kt, auto parity) {
            constexpr int st = decltype(parity)::value;
            __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): this wave's direct-to-LDS loads have landed
            __syncthreads();                      // ... and everybody else's; stage st^1 is free again
            if (kt + 1 < ksteps) {
                issue_stage(kt + 1, st ^ 1);
                load_scales(kt + 1, std::integral_constant<int, st ^ 1>{});
            }
            const uint32_t pa = (uint32_t)(st * STAGE_BYTES) + rd_a;
            const uint32_t pb = (uint32_t)(st * STAGE_BYTES) + rd_b;
            // scale operands of this K-step: byte (2*ks + g) of the row's dword must sit at the
            // position the MFMA's op_sel picks, so group g shifts its dword by 8*g bits.
            int sA[MT][SCALE_DW], sB[NT][SCALE_DW];
            if (MX) {
#pragma unroll
                for (int d = 0; d < SCALE_DW; d++) {
#pragma unroll
                    for (int s = 0; s < MT; s++) sA[s][d] = (int)(sca[st][s][d] >> (8 * g));
#pragma unroll
                    for (int s = 0; s < NT; s++) sB[s][d] = (int)(scb[st][s][d] >> (8 * g));
                }
            }

            static_for<KT::SUBSTEPS>([&](auto substep) {
                constexpr int ks = decltype(substep)::value;
                if constexpr (KIND == KIND_F8) {
                    // lane (r, g) feeds K bytes [16g, 16g+16) of each 32-byte MX block of the step
                    v8i fa[MT], fb[NT];
                    const uint32_t c0 = (((uint32_t)(ks * 4 + g)) ^ swz) << 4, c1 = (((uint32_t)(ks * 4 + 2 + g)) ^ swz) << 4;
#pragma unroll
                    for (int s = 0; s < MT; s++) {
                        const v4i lo = lds_read16(pa + s * 32 * BKB + c0), hi = lds_read16(pa + s * 32 * BKB + c1);
                        fa[s] = (v8i){lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
                    }
#pragma unroll
                    for (int s = 0; s < NT; s++) {
                        const v4i lo = lds_read16(pb + s * 32 * BKB + c0), hi = lds_read16(pb + s * 32 * BKB + c1);
                        fb[s] = (v8i){lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
                    }
#pragma unroll
                    for (int i = 0; i < MT; i++)
#pragma unroll
                        for (int j = 0; j < NT; j++)
                            acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(fa[i], fb[j], acc[i][j], CBSZ, CBSZ, ks * 2,
                                                                                        sA[i][0], ks * 2, sB[j][0]);
                } else {
                    v4i fa[MT], fb[NT];
                    const uint32_t c0 = (((uint32_t)(ks * 2 + g)) ^ swz) << 4;
#pragma unroll
                    for (int s = 0; s < MT; s++) fa[s] = lds_read16(pa + s * 32 * BKB + c0);
#pragma unroll
                    for (int s = 0; s < NT; s++) fb[s] = lds_read16(pb + s * 32 * BKB + c0);
#pragma unroll
                    for (int i = 0; i < MT; i++)
#pragma unroll
                        for (int j = 0; j < NT; j++) {
                            if constexpr (KIND == KIND_I8) {
                                acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[i], fb[j], acc[i][j], 0, 0, 0);
                            } else {
                                const v8i a8 = (v8i){fa[i][0], fa[i][1], fa[i][2], fa[i][3], 0, 0, 0, 0};
                                const v8i b8 = (v8i){fb[j][0], fb[j][1], fb[j][2], fb[j][3], 0, 0, 0, 0};
                                acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a8, b8, acc[i][j], 4, 4, (ks & 1) * 2,
                                                                                            sA[i][ks >> 1], (ks & 1) * 2, sB[j][ks >> 1]);
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
        // rows (x/4)*8 + g*4 + x%4, x = 0..15.  Rows x and x+1 (x even) are exchanged between
        // neighbouring lanes so that each lane writes two adjacent bf16 values.
        const bool odd = lane & 1;
        const float *pc = (EPI != EPI_PLAIN) ? p.per_ch + (size_t)e * p.N : nullptr;
#pragma unroll
        for (int i = 0; i < MT; i++) {
#pragma unroll
            for (int x = 0; x < 16; x += 2) {
                const int row = m0 + wm * WM + i * 32 + (x >> 2) * 8 + g * 4 + (x & 3);
                float tok0 = 1.0f, tok1 = 1.0f;
                if (EPI != EPI_PLAIN) {
                    tok0 = p.per_tok[min(row, m_end - 1)];
                    tok1 = p.per_tok[min(row + 1, m_end - 1)];
                }
                if (SWIGLU) {
                    const int oc = j0 + wn * WN_OUT + r;
                    const int occ = min(oc, p.n_out - 1);
                    const float cg = pc[occ], cu = pc[occ + p.n_out];
                    float v[2];
#pragma unroll
                    for (int h = 0; h < 2; h++) {
                        const float tok = h ? tok1 : tok0;
                        const float gate = (float)acc[i][0][x + h] * cg * tok;
                        const float up = (float)acc[i][1][x + h] * cu * tok;
                        v[h] = gate * (1.0f / (1.0f + expf(-gate))) * up;
                    }
                    store_pair(p.out, (size_t)p.n_out, row, row + 1, oc, m_end, p.n_out, v[0], v[1], odd);
                } else {
#pragma unroll
                    for (int j = 0; j < NT; j++) {
                        const int oc = j0 + wn * WN + j * 32 + r;
                        float v0 = (float)acc[i][j][x], v1 = (float)acc[i][j][x + 1];
                        if (EPI == EPI_DEQUANT) {
                            const float ch = pc[min(oc, p.N - 1)];
                            v0 = v0 * tok0 * ch;
                            v1 = v1 * tok1 * ch;
                        }
                        store_pair(p.out, (size_t)p.n_out, row, row + 1, oc, m_end, p.n_out, v0, v1, odd);
                    }
                }
            }
        }
    }
}

template <int KIND, int EPI, int FMT>
static int launch_tile_t(const GemmProblem &p, hipStream_t stream)
{
    static bool attr_set = false;
    auto kern = gemm_tile_kernel<KIND, EPI, FMT>;
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
    if (kind == KIND_I8 && epi == EPI_DEQUANT) return launch_tile_t<KIND_I8, EPI_DEQUANT, 0>(p, stream);
    if (kind == KIND_I8 && epi == EPI_DEQUANT_SWIGLU) return launch_tile_t<KIND_I8, EPI_DEQUANT_SWIGLU, 0>(p, stream);
    if (kind == KIND_F8 && epi == EPI_PLAIN && p.fmt == CCH_FMT_E4M3) return launch_tile_t<KIND_F8, EPI_PLAIN, CCH_FMT_E4M3>(p, stream);
    if (kind == KIND_F8 && epi == EPI_PLAIN && p.fmt == CCH_FMT_E5M2) return launch_tile_t<KIND_F8, EPI_PLAIN, CCH_FMT_E5M2>(p, stream);
    if (kind == KIND_F4 && epi == EPI_PLAIN) return launch_tile_t<KIND_F4, EPI_PLAIN, CCH_FMT_E2M1>(p, stream);
    return fail(CCH_ENOSUP, "no tiled GEMM kernel for kind %d with epilogue %d", kind, epi);
}

}  // namespace cch
