// Tiled MFMA GEMM family for gfx950 (B stored K-contiguous, i.e. trans_b = 1):
//   int8 x int8 -> int32   v_mfma_i32_32x32x32_i8          + dequant / dequant+SwiGLU epilogue
//   MXFP8 / MXFP4          v_mfma_scale_f32_32x32x64_f8f6f4 with per-lane E8M0 scale operands
//
// One persistent workgroup (8 waves) per CU walks a global list of 256x256 output tiles built
// from the prefix sums of the group sizes (a dense problem is one group).
//   * K advances in steps of 64 bytes per row.  The A and B panels of a step (256 rows x 64 B
//     each) and, for MX, one dword of E8M0 scales per row go global -> LDS with direct-to-LDS
//     loads (no VGPR round trip) into a ring of four stages, so three steps are in flight
//     while one is consumed.
//   * Each wave owns 128 x 64 outputs as 4 x 2 MFMA tiles of 32 x 32.  A step is two MFMA
//     groups (rows 0-63, rows 64-127 of the wave tile); the LDS reads of one group are issued
//     before the MFMAs of the previous one, and the single workgroup barrier of a step sits
//     between the two groups, behind already issued MFMAs.
//   * The next tile's first four steps are requested before the current tile's epilogue.
//   * Epilogues (dequant, SwiGLU, bf16 rounding) run on the accumulators; results pass through
//     a wave-private 2 KiB LDS buffer so that every lane stores 16 contiguous bytes.
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
typedef float v4f __attribute__((ext_vector_type(4)));
typedef float v16f __attribute__((ext_vector_type(16)));

constexpr int BM = 256, BN = 256;        // output tile
constexpr int BKB = 64;                  // bytes of K per step (per row)
constexpr int PANEL_BYTES = BM * BKB;    // one operand panel of one stage: 16 KiB
constexpr int STAGE_BYTES = 2 * PANEL_BYTES;
constexpr int NSTAGE = 4;
constexpr int TILE_THREADS = 512;        // 8 waves: 2 (M) x 4 (N), each owning 128 x 64 outputs
constexpr int NWAVES = TILE_THREADS / 64;
constexpr int WAVES_N = 4;
constexpr int WM = 128, WN = 64;         // wave tile
constexpr int MT = WM / 32, NT = WN / 32;  // 32x32 MFMA tiles per wave
constexpr int NJ = PANEL_BYTES / 1024 / NWAVES;  // direct-to-LDS instructions per wave per panel (2)

// dynamic LDS map
constexpr int RING_OFF = 0;
constexpr int SCALE_OFF = RING_OFF + NSTAGE * STAGE_BYTES;   // per stage: 256 A dwords, 256 B dwords
constexpr int SCALE_STAGE = 2048;
constexpr int EPI_OFF = SCALE_OFF + NSTAGE * SCALE_STAGE;    // per wave: 16 rows x 64 bf16
constexpr int EPI_WAVE = 2048;
constexpr int PARAM_OFF = EPI_OFF + NWAVES * EPI_WAVE;       // per tile parity: 256 per_tok + 256 per_ch floats
constexpr int PARAM_SET = 2048;
constexpr int LDS_BYTES = PARAM_OFF + 2 * PARAM_SET;         // 156 KiB of the CU's 160 KiB

template <int KIND> struct KindTraits;
template <> struct KindTraits<KIND_I8> { static constexpr int ELEMS_PER_BYTE = 1; using Acc = v16i; };
template <> struct KindTraits<KIND_F8> { static constexpr int ELEMS_PER_BYTE = 1; using Acc = v16f; };
template <> struct KindTraits<KIND_F4> { static constexpr int ELEMS_PER_BYTE = 2; using Acc = v16f; };

extern __shared__ __attribute__((aligned(1024))) uint8_t smem[];

template <int N> using IC = std::integral_constant<int, N>;

// Calls f(IC<0>) ... f(IC<N-1>): loop indices that must be compile-time constants.
template <int... I, class F>
__device__ __forceinline__ void static_for_impl(std::integer_sequence<int, I...>, F &&f)
{
    (f(IC<I>{}), ...);
}
template <int N, class F> __device__ __forceinline__ void static_for(F &&f)
{
    static_for_impl(std::make_integer_sequence<int, N>{}, f);
}

__device__ __forceinline__ int uniform(int v) { return __builtin_amdgcn_readfirstlane(v); }

// s_waitcnt vmcnt(n) lgkmcnt(0) on gfx9: vmcnt in bits [3:0] and [15:14], expcnt [6:4], lgkmcnt [11:8].
#define CCH_WAIT_VM_LGKM0(n) __builtin_amdgcn_s_waitcnt(((n) & 15) | (((n) >> 4) << 14) | (7 << 4))

// 16 / 4 bytes per lane, global -> LDS without passing through registers, as raw buffer loads:
// the descriptor holds the wave-uniform base, `voff` is the per-lane byte offset, `soff` a
// wave-uniform byte offset (the K position).  Lane l of the wave lands at LDS address
// lds_addr + size*l.  Issued as inline assembly on purpose: the compiler's wait-count pass
// would otherwise drain every outstanding direct-to-LDS load before each LDS read, which
// defeats the multi-stage ring; completion is tracked by the explicit vmcnt waits instead.
typedef int Rsrc __attribute__((ext_vector_type(4)));
__device__ __forceinline__ Rsrc make_rsrc(const void *base)
{
    const uint64_t b = reinterpret_cast<uint64_t>(base);
    Rsrc rs;
    rs[0] = __builtin_amdgcn_readfirstlane((int)(uint32_t)b);
    rs[1] = __builtin_amdgcn_readfirstlane((int)(uint32_t)(b >> 32));  // stride 0, no swizzle
    rs[2] = 0x7FFFFFFF;                                                // num_records (bytes)
    rs[3] = 0x00020000;                                                // raw 32-bit data format
    return rs;
}
__device__ __forceinline__ void load16_to_lds(Rsrc rs, uint32_t voff, uint32_t soff, uint32_t lds_addr)
{
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
                 :
                 : "s"(lds_addr), "v"(voff), "s"(rs), "s"(soff)
                 : "memory", "m0");
}
__device__ __forceinline__ void load4_to_lds(Rsrc rs, uint32_t voff, uint32_t soff, uint32_t lds_addr)
{
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dword %1, %2, %3 offen lds"
                 :
                 : "s"(lds_addr), "v"(voff), "s"(rs), "s"(soff)
                 : "memory", "m0");
}

__device__ __forceinline__ v4i lds_read16(uint32_t off) { return *reinterpret_cast<const v4i *>(smem + off); }
__device__ __forceinline__ uint32_t lds_read4(uint32_t off) { return *reinterpret_cast<const uint32_t *>(smem + off); }

// Panel layout: row pitch 64 B; 16-byte chunk c of row `row` sits at chunk position
// c ^ ((row >> 2) & 3), which spreads 16 consecutive rows over all 64 banks for 16-byte reads.
__device__ __forceinline__ uint32_t swizzle_of_row(int row) { return (uint32_t)((row >> 2) & 3); }

// What one tile needs, all wave-uniform except the per-lane source offsets.
template <int NSRC> struct TileCtx {
    int valid, e, m0, m_end, j0;
    Rsrc rs_a, rs_b, rs_sc;             // buffer descriptors: A rows from m0, B of the expert, scales
    uint32_t off_a[NSRC], off_b[NSRC];  // per lane: source row * pitch + chunk * 16
    uint32_t off_sc;                    // per lane: scale row * sld (A rows for waves 0-3, B columns for 4-7)
};

template <int KIND, int EPI, int FMT>
__global__ __launch_bounds__(TILE_THREADS) void gemm_tile_kernel(GemmProblem p)
{
    using KT = KindTraits<KIND>;
    using Acc = typename KT::Acc;
    constexpr bool MX = KIND != KIND_I8;
    constexpr bool SWIGLU = EPI == EPI_DEQUANT_SWIGLU;
    constexpr int BN_OUT = SWIGLU ? BN / 2 : BN;   // output columns per tile
    constexpr int WN_OUT = SWIGLU ? WN / 2 : WN;   // output columns per wave
    constexpr int NV = 2 * NJ + (MX ? 1 : 0);      // vector-memory instructions per wave per step
    constexpr int CBSZ = FMT == CCH_FMT_E2M1 ? 4 : (FMT == CCH_FMT_E5M2 ? 1 : 0);

    __shared__ GroupTable tab;
    if (threadIdx.x == 0) build_group_table(tab, p.group_sizes, p.num_groups, p.T, BM);
    __syncthreads();

    const int lane = threadIdx.x & 63;
    const int wave = uniform(threadIdx.x >> 6);
    const int wm = wave / WAVES_N, wn = wave % WAVES_N;
    // LDS byte address of the dynamic segment, for the direct-to-LDS destinations
    const uint32_t lds_base = (uint32_t)uniform((int)(uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint8_t *)smem);
    const int r = lane & 31, g = lane >> 5;

    const int lda = p.K / KT::ELEMS_PER_BYTE;  // bytes per row of A and of B (K-contiguous)
    const int ksteps = lda / BKB;
    const int n_tiles = (p.n_out + BN_OUT - 1) / BN_OUT;
    const int total_tiles = uniform(tab.tile_start[p.num_groups]) * n_tiles;  // rows past the groups are not ours

    // LDS read offsets of this lane inside a stage.
    const uint32_t swz = swizzle_of_row(r);
    const uint32_t rd_a = (uint32_t)(wm * WM + r) * BKB, rd_b = (uint32_t)PANEL_BYTES + (uint32_t)(wn * WN + r) * BKB;
    const uint32_t ch0 = (((uint32_t)g) ^ swz) << 4, ch1 = (((uint32_t)(2 + g)) ^ swz) << 4;
    const uint32_t rd_sa = (uint32_t)(wm * WM + r) * 4, rd_sb = 1024u + (uint32_t)(wn * WN + r) * 4;
    // DMA lane roles: lane l fills row l/4, chunk position l%4 of a 16-row segment.
    const uint32_t dma_chunk = ((uint32_t)(lane & 3) ^ (uint32_t)((lane >> 4) & 3)) * 16u;

    auto decode = [&](int t, TileCtx<NJ> &c) {
        c.valid = t < total_tiles;
        if (!c.valid) return;
        const int tr = t / n_tiles, nt = t - tr * n_tiles;
        c.e = uniform(find_group(tab, p.num_groups, tr));
        c.m0 = uniform(tab.row_start[c.e] + (tr - tab.tile_start[c.e]) * BM);
        c.m_end = uniform(tab.row_start[c.e + 1]);
        c.j0 = nt * BN_OUT;
        c.rs_a = make_rsrc(p.a + (size_t)c.m0 * lda);
        c.rs_b = make_rsrc(p.b + (size_t)c.e * p.b_stride);
        // Rows past the edge re-read the last valid row; their products land in accumulators
        // that are never stored.
#pragma unroll
        for (int j = 0; j < NJ; j++) {
            const int row = (wave * NJ + j) * 16 + (lane >> 2);
            c.off_a[j] = (uint32_t)min(row, c.m_end - 1 - c.m0) * (uint32_t)lda + dma_chunk;
            int col;  // B row (= logical column) feeding tile row `row`
            if (SWIGLU) {
                // tile row = wn*64 + h*32 + c: h = 0 gate, 1 up; output column j0 + wn*32 + c
                col = ((row >> 5) & 1) * p.n_out + min(c.j0 + (row >> 6) * 32 + (row & 31), p.n_out - 1);
            } else {
                col = min(c.j0 + row, p.N - 1);
            }
            c.off_b[j] = (uint32_t)col * (uint32_t)lda + dma_chunk;
        }
        if (MX) {
            const int idx = (wave & 3) * 64 + lane;
            if (wave < 4) {
                c.rs_sc = make_rsrc(p.sa + (size_t)c.m0 * p.sld);
                c.off_sc = (uint32_t)min(idx, c.m_end - 1 - c.m0) * (uint32_t)p.sld;
            } else {
                c.rs_sc = make_rsrc(p.sb + (size_t)c.e * p.sb_stride);
                c.off_sc = (uint32_t)min(c.j0 + idx, p.N - 1) * (uint32_t)p.sld;
            }
        }
    };

    // Requests K-step kt of tile c into ring slot kt % NSTAGE: NV instructions per wave, which
    // can be issued one at a time (piece 0..NV-1) so that they interleave with MFMAs instead of
    // arriving at the texture addresser as one burst from all eight waves.
    auto issue_piece = [&](const TileCtx<NJ> &c, int kt, auto piece_c) {
        constexpr int piece = decltype(piece_c)::value;
        const int slot = kt & (NSTAGE - 1);
        const uint32_t lds = lds_base + (uint32_t)(RING_OFF + slot * STAGE_BYTES) + (uint32_t)(wave * NJ) * 1024u;
        if constexpr (piece < NJ) {
            load16_to_lds(c.rs_a, c.off_a[piece], (uint32_t)kt * BKB, lds + piece * 1024u);
        } else if constexpr (piece < 2 * NJ) {
            load16_to_lds(c.rs_b, c.off_b[piece - NJ], (uint32_t)kt * BKB, lds + PANEL_BYTES + (piece - NJ) * 1024u);
        } else if constexpr (MX) {
            // one dword = 4 scale bytes per row: FP8 covers steps 2q and 2q+1, FP4 exactly one step
            const int dw = KIND == KIND_F8 ? (kt >> 1) : kt;
            load4_to_lds(c.rs_sc, c.off_sc, (uint32_t)dw * 4u,
                         lds_base + (uint32_t)(SCALE_OFF + slot * SCALE_STAGE) + (uint32_t)(wave >= 4) * 1024u + (uint32_t)(wave & 3) * 256u);
        }
    };
    auto issue_step = [&](const TileCtx<NJ> &c, int kt) {
        issue_piece(c, kt, IC<0>{});
        issue_piece(c, kt, IC<1>{});
        issue_piece(c, kt, IC<2>{});
        issue_piece(c, kt, IC<3>{});
        if (MX) issue_piece(c, kt, IC<4>{});
    };

    // Tile set-up: epilogue parameters of the tile (per-token / per-channel scales) and its
    // first NSTAGE steps.  Every wave issues the same number of instructions.
    auto setup = [&](const TileCtx<NJ> &c, int parity) {
        if (EPI != EPI_PLAIN) {
            const int idx = (wave & 3) * 64 + lane;
            // destination of lane 0 of this wave; lane l lands 4*l bytes further
            const uint32_t dst = lds_base + (uint32_t)(PARAM_OFF + parity * PARAM_SET) + (uint32_t)(wave & 3) * 256u;
            load4_to_lds(make_rsrc(p.per_tok + c.m0), (uint32_t)min(idx, c.m_end - 1 - c.m0) * 4u, 0u, dst);
            int col;
            if (SWIGLU) col = ((idx >> 5) & 1) * p.n_out + min(c.j0 + (idx >> 6) * 32 + (idx & 31), p.n_out - 1);
            else col = min(c.j0 + idx, p.N - 1);
            load4_to_lds(make_rsrc(p.per_ch + (size_t)c.e * p.N), (uint32_t)col * 4u, 0u, dst + 1024u);
        }
        for (int kt = 0; kt < min(NSTAGE, ksteps); kt++) issue_step(c, kt);
    };

    TileCtx<NJ> cur, nxt;
    int t = blockIdx.x, parity = 0;
    decode(t, cur);
    if (cur.valid) setup(cur, 0);

    while (cur.valid) {

        Acc acc[MT][NT];
#pragma unroll
        for (int i = 0; i < MT; i++)
#pragma unroll
            for (int j = 0; j < NT; j++)
#pragma unroll
                for (int x = 0; x < 16; x++) acc[i][j][x] = 0;

        v8i fb[NT], fa[MT];              // B and A fragments of the current step
        uint32_t sc[MT + NT];            // raw scale dwords of the current step

        auto read_frag = [&](uint32_t row_off) {
#ifdef DBG_NO_LDSREAD
            if (ksteps > 0) { const int q = (int)row_off; return (v8i){q, q, q, q, q, q, q, q}; }
#endif
            const v4i lo = lds_read16(row_off + ch0), hi = lds_read16(row_off + ch1);
            return (v8i){lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
        };
        // all fragments and scales of step kt
        auto read_step = [&](int kt) {
            const uint32_t st = (uint32_t)(RING_OFF + (kt & (NSTAGE - 1)) * STAGE_BYTES);
#pragma unroll
            for (int s = 0; s < NT; s++) fb[s] = read_frag(st + rd_b + s * 32 * BKB);
#pragma unroll
            for (int s = 0; s < MT; s++) fa[s] = read_frag(st + rd_a + s * 32 * BKB);
            if (MX) {
                const uint32_t ss = (uint32_t)(SCALE_OFF + (kt & (NSTAGE - 1)) * SCALE_STAGE);
#pragma unroll
                for (int s = 0; s < MT; s++) sc[s] = lds_read4(ss + rd_sa + s * 128);
#pragma unroll
                for (int s = 0; s < NT; s++) sc[MT + s] = lds_read4(ss + rd_sb + s * 128);
            }
        };
        // One MFMA group: A sub-tiles (2h, 2h+1) against both B sub-tiles.
        // DMA: after each MFMA issue one piece of the request for step kt + NSTAGE.
        auto mfma_group = [&](int kt, auto half_c, auto dma_c) {
            constexpr int h = decltype(half_c)::value;
            constexpr bool DMA = decltype(dma_c)::value;
            if (DMA && MX) issue_piece(cur, kt + NSTAGE, IC<4>{});
#ifndef DBG_NO_MFMA
            // scale operands: lane group g must present byte (2*(kt&1) + g) [FP8] or bytes g and
            // 2+g [FP4] of the row's dword where op_sel looks for it
            const int sh = KIND == KIND_F8 ? 8 * (2 * (kt & 1) + g) : 8 * g;
            static_for<2 * NT>([&](auto idx_c) {
                constexpr int ii = decltype(idx_c)::value / NT, j = decltype(idx_c)::value % NT;
                {
                    const int i = 2 * h + ii;
                    if constexpr (KIND == KIND_F8) {
                        acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(fa[2 * h + ii], fb[j], acc[i][j], CBSZ, CBSZ, 0,
                                                                                    (int)(sc[i] >> sh), 0, (int)(sc[MT + j] >> sh));
                    } else if constexpr (KIND == KIND_F4) {
                        const int sA = (int)(sc[i] >> sh), sB = (int)(sc[MT + j] >> sh);
                        const v8i alo = (v8i){fa[2 * h + ii][0], fa[2 * h + ii][1], fa[2 * h + ii][2], fa[2 * h + ii][3], 0, 0, 0, 0};
                        const v8i blo = (v8i){fb[j][0], fb[j][1], fb[j][2], fb[j][3], 0, 0, 0, 0};
                        const v8i ahi = (v8i){fa[2 * h + ii][4], fa[2 * h + ii][5], fa[2 * h + ii][6], fa[2 * h + ii][7], 0, 0, 0, 0};
                        const v8i bhi = (v8i){fb[j][4], fb[j][5], fb[j][6], fb[j][7], 0, 0, 0, 0};
                        acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(alo, blo, acc[i][j], 4, 4, 0, sA, 0, sB);
                        acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(ahi, bhi, acc[i][j], 4, 4, 2, sA, 2, sB);
                    } else {
                        const v4i alo = (v4i){fa[2 * h + ii][0], fa[2 * h + ii][1], fa[2 * h + ii][2], fa[2 * h + ii][3]}, ahi = (v4i){fa[2 * h + ii][4], fa[2 * h + ii][5], fa[2 * h + ii][6], fa[2 * h + ii][7]};
                        const v4i blo = (v4i){fb[j][0], fb[j][1], fb[j][2], fb[j][3]};
                        const v4i bhi = (v4i){fb[j][4], fb[j][5], fb[j][6], fb[j][7]};
                        acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(alo, blo, acc[i][j], 0, 0, 0);
                        acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(ahi, bhi, acc[i][j], 0, 0, 0);
                    }
                }
                if constexpr (DMA) {
                    __builtin_amdgcn_sched_barrier(0);
                    issue_piece(cur, kt + NSTAGE, idx_c);
                    __builtin_amdgcn_sched_barrier(0);
                }
            });
#endif
        };

        // Step 0 of this tile was requested before at most min(NSTAGE, ksteps) - 1 later steps.
        {
            const int later = min(NSTAGE, ksteps) - 1;
            if (later >= 3) CCH_WAIT_VM_LGKM0(3 * NV);
            else if (later == 2) CCH_WAIT_VM_LGKM0(2 * NV);
            else if (later == 1) CCH_WAIT_VM_LGKM0(NV);
            else CCH_WAIT_VM_LGKM0(0);
            __syncthreads();
        }

        // One K-step.  STEADY: at least NSTAGE more steps follow, so every branch is decided
        // at compile time and the body is one straight block around the barrier.
        auto kstep = [&](int kt, auto steady_c) {
            constexpr bool STEADY = decltype(steady_c)::value;
            read_step(kt);
            mfma_group(kt, IC<0>{}, std::false_type{});
            // Before the barrier: this wave's reads of stage kt are complete and its requests for
            // step kt+1 have landed (steps kt+2, kt+3 may still be in flight).
            if (STEADY) {
                CCH_WAIT_VM_LGKM0(2 * NV);
            } else {
                const int ahead = min(2, ksteps - 2 - kt);
                if (ahead >= 2) CCH_WAIT_VM_LGKM0(2 * NV);
                else if (ahead == 1) CCH_WAIT_VM_LGKM0(NV);
                else CCH_WAIT_VM_LGKM0(0);
            }
#ifndef DBG_NO_BARRIER
            __syncthreads();
#endif
            // After the barrier: stage kt is dead for every wave, step kt+1 is visible to all.
#ifndef DBG_NO_LOADS
            if (STEADY) {
                mfma_group(kt, IC<1>{}, std::true_type{});
            } else {
                if (kt + NSTAGE < ksteps) {
                    issue_step(cur, kt + NSTAGE);
                } else if (kt == ksteps - 1) {
                    decode(t + gridDim.x, nxt);
                    if (nxt.valid) setup(nxt, parity ^ 1);
                }
                mfma_group(kt, IC<1>{}, std::false_type{});
            }
#else
            if (!STEADY && kt == ksteps - 1) decode(t + gridDim.x, nxt);
            mfma_group(kt, IC<1>{}, std::false_type{});
#endif
        };
        int kt = 0;
        for (; kt + NSTAGE < ksteps; kt++) kstep(kt, std::true_type{});
        for (; kt < ksteps; kt++) kstep(kt, std::false_type{});

#ifdef DBG_NO_EPI
        if (acc[0][0][0] != 12345) { cur = nxt; t += gridDim.x; parity ^= 1; continue; }
#endif
        // Epilogue.  Lane (r, g) holds, for sub-tile (i, j), column r and rows
        // (x/4)*8 + g*4 + x%4, x = 0..15.  Sixteen rows at a time go through the wave's private
        // LDS buffer: neighbouring lanes exchange one value so that each writes two adjacent
        // bf16, then every lane reads back 16 contiguous bytes and stores them.
        {
            const uint32_t epi = (uint32_t)(EPI_OFF + wave * EPI_WAVE);
            const uint32_t prm = (uint32_t)(PARAM_OFF + parity * PARAM_SET);
            constexpr int ROWB = WN_OUT * 2;              // bytes per staged row
            constexpr int CPR = ROWB / 16;                // 16-byte chunks per staged row
            constexpr int RPI = 64 / CPR;                 // rows covered by one read-back instruction
            const bool odd = lane & 1;
            float chs[NT];
            if (EPI != EPI_PLAIN) {
#pragma unroll
                for (int j = 0; j < NT; j++) chs[j] = __uint_as_float(lds_read4(prm + 1024u + (uint32_t)(wn * WN + j * 32 + r) * 4u));
            }
            const bool vec_ok = (p.n_out % 8 == 0) && ((reinterpret_cast<uintptr_t>(p.out) & 15) == 0);
#pragma unroll
            for (int i = 0; i < MT; i++) {
#pragma unroll
                for (int hh = 0; hh < 2; hh++) {
                    float tok[2][4];
                    if (EPI != EPI_PLAIN) {
#pragma unroll
                        for (int xq = 0; xq < 2; xq++) {
                            const v4i tv = lds_read16(prm + (uint32_t)(wm * WM + i * 32 + hh * 16 + xq * 8 + g * 4) * 4u);
#pragma unroll
                            for (int xr = 0; xr < 4; xr++) tok[xq][xr] = __int_as_float(tv[xr]);
                        }
                    }
#pragma unroll
                    for (int xq = 0; xq < 2; xq++)
#pragma unroll
                        for (int xr = 0; xr < 4; xr += 2)
#pragma unroll
                            for (int j = 0; j < (SWIGLU ? 1 : NT); j++) {
                                const int x = (2 * hh + xq) * 4 + xr;
                                float v[2];
#pragma unroll
                                for (int d = 0; d < 2; d++) {
                                    if (SWIGLU) {
                                        const float gate = (float)acc[i][0][x + d] * chs[0] * tok[xq][xr + d];
                                        const float up = (float)acc[i][1][x + d] * chs[1] * tok[xq][xr + d];
                                        v[d] = gate * (1.0f / (1.0f + expf(-gate))) * up;
                                    } else if (EPI == EPI_DEQUANT) {
                                        v[d] = (float)acc[i][j][x + d] * tok[xq][xr + d] * chs[j];
                                    } else {
                                        v[d] = (float)acc[i][j][x + d];
                                    }
                                }
                                const uint32_t keep = f32_to_bf16_bits(odd ? v[1] : v[0]);
                                const uint32_t send = f32_to_bf16_bits(odd ? v[0] : v[1]);
                                const uint32_t recv = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)send, 0xB1, 0xF, 0xF, true);
                                const uint32_t packed = odd ? (recv | (keep << 16)) : (keep | (recv << 16));
                                const int lrow = xq * 8 + g * 4 + xr + (odd ? 1 : 0);
                                const int lcol = j * 32 + (r & ~1);
                                *reinterpret_cast<uint32_t *>(smem + epi + (uint32_t)(lrow * ROWB + lcol * 2)) = packed;
                            }
                    const int row0 = cur.m0 + wm * WM + i * 32 + hh * 16;
                    const int col0 = cur.j0 + wn * WN_OUT;
#pragma unroll
                    for (int q = 0; q < 16 / RPI; q++) {
                        const int lrow = q * RPI + lane / CPR, chunk = lane % CPR;
                        const v4i val = lds_read16(epi + (uint32_t)(lrow * ROWB + chunk * 16));
                        const int row = row0 + lrow, col = col0 + chunk * 8;
                        if (row < cur.m_end) {
                            uint16_t *dst = p.out + (size_t)row * p.n_out + col;
                            if (vec_ok && col + 8 <= p.n_out) {
                                *reinterpret_cast<v4i *>(dst) = val;
                            } else {
#pragma unroll
                                for (int c = 0; c < 8; c++)
                                    if (col + c < p.n_out) dst[c] = (uint16_t)((uint32_t)val[c >> 1] >> ((c & 1) * 16));
                            }
                        }
                    }
                }
            }
        }
        cur = nxt;
        t += gridDim.x;
        parity ^= 1;
    }
}

// Rows that belong to no group are written as zeros (the reference's golden pads them,
// examples/utils/gen_data_fp4_mx_alltoallv_gmm.py:788-790).
__global__ __launch_bounds__(256) void zero_tail_rows_kernel(uint16_t *out, const int32_t *group_sizes, int num_groups, int T,
                                                             int n_out)
{
    int used = 0;
    for (int gidx = 0; gidx < num_groups; gidx++) used += max(0, min(group_sizes[gidx], T - used));
    const size_t begin = (size_t)used * n_out, end = (size_t)T * n_out;
    for (size_t i = begin + (size_t)blockIdx.x * 256 + threadIdx.x; i < end; i += (size_t)gridDim.x * 256) out[i] = 0;
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
    int rc = launch_status("gemm_tile_kernel");
    if (rc || !p.group_sizes) return rc;
    hipLaunchKernelGGL(zero_tail_rows_kernel, dim3(64), dim3(256), 0, stream, p.out, p.group_sizes, p.num_groups, p.T, p.n_out);
    return launch_status("zero_tail_rows_kernel");
}

// True when the tiled kernels take this problem; otherwise the caller uses the generic path.
bool gemm_tile_supports(const GemmProblem &p, int kind)
{
    const int epb = kind == KIND_F4 ? 2 : 1;
    if (!p.trans_b) return false;
    // whole 64-byte K-steps; MX additionally whole scale dwords (4 blocks of 32) per row
    if (p.K <= 0 || p.K % (kind == KIND_I8 ? 64 : 128) != 0) return false;
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
