// Tiled MFMA GEMM family for gfx950 (B stored K-contiguous, i.e. trans_b = 1):
//   int8 x int8 -> int32   v_mfma_i32_32x32x32_i8          + dequant / dequant+SwiGLU epilogue
//   MXFP8 / MXFP4          v_mfma_scale_f32_32x32x64_f8f6f4 with per-lane E8M0 scale operands
//
// One persistent workgroup (8 waves) per CU walks a global list of 256x256 output tiles built
// from the prefix sums of the group sizes (a dense problem is one group).
//   * K advances in steps of 128 bytes per row, the size of an L2 line: direct-to-LDS loads
//     that cover whole lines reach about 1.5x the L2 throughput of half-line requests.  The A
//     and B panels of a step (256 rows x 128 B each) and, for MX, the E8M0 scales of the step
//     go global -> LDS without a VGPR round trip into a ring of two stages; the requests for
//     step k+1 are issued one instruction at a time between the MFMAs of step k.
//   * Each wave owns 128 x 64 outputs as 4 x 2 MFMA tiles of 32 x 32 and reads its fragments
//     with 16-byte LDS reads from an XOR-swizzled panel layout (no bank conflicts).
//   * The next tile's first step is requested before the current tile's epilogue.
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
typedef unsigned int v4u __attribute__((ext_vector_type(4)));
typedef float v16f __attribute__((ext_vector_type(16)));

constexpr int BM = 256, BN = 256;        // output tile
constexpr int BKB = 128;                 // bytes of K per step (per row) = one L2 line
constexpr int PANEL_BYTES = BM * BKB;    // one operand panel of one stage: 32 KiB
constexpr int STAGE_BYTES = 2 * PANEL_BYTES;
constexpr int NSTAGE = 2;
constexpr int TILE_THREADS = 512;        // 8 waves: 2 (M) x 4 (N), each owning 128 x 64 outputs
constexpr int NWAVES = TILE_THREADS / 64;
constexpr int WAVES_N = 4;
constexpr int WM = 128, WN = 64;         // wave tile
constexpr int MT = WM / 32, NT = WN / 32;  // 32x32 MFMA tiles per wave
constexpr int NJ = PANEL_BYTES / 1024 / NWAVES;  // direct-to-LDS instructions per wave per panel (4)

// dynamic LDS map
constexpr int RING_OFF = 0;
constexpr int SCALE_OFF = RING_OFF + NSTAGE * STAGE_BYTES;   // per stage: up to 2 x (256 A + 256 B) dwords
constexpr int SCALE_STAGE = 4096;
constexpr int EPI_OFF = SCALE_OFF + NSTAGE * SCALE_STAGE;    // per wave: 16 rows x 64 bf16
constexpr int EPI_WAVE = 2048;
constexpr int PARAM_OFF = EPI_OFF + NWAVES * EPI_WAVE;       // per tile parity: 256 per_tok + 256 per_ch floats
constexpr int PARAM_SET = 2048;
constexpr int LDS_BYTES = PARAM_OFF + 2 * PARAM_SET;         // 156 KiB of the CU's 160 KiB

template <int KIND> struct KindTraits;
template <> struct KindTraits<KIND_I8> { static constexpr int ELEMS_PER_BYTE = 1, SCALE_DW = 0; using Acc = v16i; };
template <> struct KindTraits<KIND_F8> { static constexpr int ELEMS_PER_BYTE = 1, SCALE_DW = 1; using Acc = v16f; };
template <> struct KindTraits<KIND_F4> { static constexpr int ELEMS_PER_BYTE = 2, SCALE_DW = 2; using Acc = v16f; };

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
// s_waitcnt lgkmcnt(0) only (vmcnt left at its maximum of 63)
#define CCH_WAIT_LGKM0() __builtin_amdgcn_s_waitcnt(0xC07F)

// 16 / 4 bytes per lane, global -> LDS without passing through registers, as raw buffer loads:
// the descriptor holds the wave-uniform base, `voff` is the per-lane byte offset, `soff` a
// wave-uniform byte offset (the K position).  Lane l of the wave lands at LDS address
// lds_addr + size*l.  Issued as inline assembly on purpose: the compiler's wait-count pass
// would otherwise drain every outstanding direct-to-LDS load before each LDS read;
// completion is tracked by the explicit vmcnt waits instead.
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
// Descriptors are wave-uniform by construction; this pins them to scalar registers where the
// compiler has lost track of that.
__device__ __forceinline__ Rsrc scalar_rsrc(Rsrc rs)
{
    Rsrc u;
    u[0] = __builtin_amdgcn_readfirstlane(rs[0]);
    u[1] = __builtin_amdgcn_readfirstlane(rs[1]);
    u[2] = 0x7FFFFFFF;
    u[3] = 0x00020000;
    return u;
}
__device__ __forceinline__ void load16_to_lds(Rsrc rs, uint32_t voff, uint32_t soff, uint32_t lds_addr)
{
    rs = scalar_rsrc(rs);
    soff = (uint32_t)__builtin_amdgcn_readfirstlane((int)soff);
    lds_addr = (uint32_t)__builtin_amdgcn_readfirstlane((int)lds_addr);
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
                 :
                 : "s"(lds_addr), "v"(voff), "s"(rs), "s"(soff)
                 : "memory", "m0");
}
__device__ __forceinline__ void load4_to_lds(Rsrc rs, uint32_t voff, uint32_t soff, uint32_t lds_addr)
{
    rs = scalar_rsrc(rs);
    soff = (uint32_t)__builtin_amdgcn_readfirstlane((int)soff);
    lds_addr = (uint32_t)__builtin_amdgcn_readfirstlane((int)lds_addr);
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dword %1, %2, %3 offen lds"
                 :
                 : "s"(lds_addr), "v"(voff), "s"(rs), "s"(soff)
                 : "memory", "m0");
}

__device__ __forceinline__ v4i lds_read16(uint32_t off) { return *reinterpret_cast<const v4i *>(smem + off); }
__device__ __forceinline__ uint32_t lds_read4(uint32_t off) { return *reinterpret_cast<const uint32_t *>(smem + off); }

// Panel layout: row pitch 128 B; 16-byte chunk c of row `row` sits at chunk position
// c ^ ((row >> 1) & 7), which spreads 16 consecutive rows over all 64 banks for 16-byte reads.
__device__ __forceinline__ uint32_t swizzle_of_row(int row) { return (uint32_t)((row >> 1) & 7); }

// What one tile needs, all wave-uniform except the per-lane source offsets.
struct TileCtx {
    int valid, e, m0, m_end, j0;
    Rsrc rs_a, rs_b, rs_sc;             // buffer descriptors: A rows from m0, B of the expert, scales
    uint32_t off_a[NJ], off_b[NJ];      // per lane: source row * pitch + chunk * 16
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
    constexpr int SCALE_DW = KT::SCALE_DW;         // scale dwords per row per step
    constexpr int NV = 2 * NJ + SCALE_DW;          // direct-to-LDS instructions per wave per step
    constexpr int CBSZ = FMT == CCH_FMT_E2M1 ? 4 : (FMT == CCH_FMT_E5M2 ? 1 : 0);
    constexpr int ROWB = WN_OUT * 2;               // epilogue staging: bytes per row
    constexpr int CPR = ROWB / 16;                 // 16-byte chunks per staged row
    constexpr int RPI = 64 / CPR;                  // rows covered by one read-back instruction
    constexpr int NSTORES = MT * 2 * (16 / RPI);   // 16-byte stores per lane per tile
    constexpr int NP = EPI != EPI_PLAIN ? 2 : 0;   // extra requests in a tile's first batch (epilogue parameters)

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
    const uint32_t rd_sa = (uint32_t)(wm * WM + r) * 4, rd_sb = 1024u + (uint32_t)(wn * WN + r) * 4;

    auto decode = [&](int t, TileCtx &c) {
        c.valid = t < total_tiles;
        if (!c.valid) return;
        const int tr = t / n_tiles, nt = t - tr * n_tiles;
        c.e = uniform(find_group(tab, p.num_groups, tr));
        c.m0 = uniform(tab.row_start[c.e] + (tr - tab.tile_start[c.e]) * BM);
        c.m_end = uniform(tab.row_start[c.e + 1]);
        c.j0 = nt * BN_OUT;
        c.rs_a = make_rsrc(p.a + (size_t)c.m0 * lda);
        c.rs_b = make_rsrc(p.b + (size_t)c.e * p.b_stride);
        // Instruction j of this wave fills rows (wave*NJ + j)*8 .. +7 of a panel; lane l lands at
        // row l/8, chunk position l%8 and must therefore fetch chunk (l%8) ^ swizzle(row).  Rows
        // past the edge re-read the last valid row; their products land in accumulators that are
        // never stored.
#pragma unroll
        for (int j = 0; j < NJ; j++) {
            const int row = (wave * NJ + j) * 8 + (lane >> 3);
            const uint32_t chunk = ((uint32_t)(lane & 7) ^ swizzle_of_row(row)) * 16u;
            c.off_a[j] = (uint32_t)min(row, c.m_end - 1 - c.m0) * (uint32_t)lda + chunk;
            int col;  // B row (= logical column) feeding tile row `row`
            if (SWIGLU) {
                // tile row = wn*64 + h*32 + c: h = 0 gate, 1 up; output column j0 + wn*32 + c
                col = ((row >> 5) & 1) * p.n_out + min(c.j0 + (row >> 6) * 32 + (row & 31), p.n_out - 1);
            } else {
                col = min(c.j0 + row, p.N - 1);
            }
            c.off_b[j] = (uint32_t)col * (uint32_t)lda + chunk;
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

    // Requests K-step kt of tile c into ring stage `stage`: NV instructions per wave, issued one
    // at a time (piece 0..NV-1) so that they interleave with MFMAs instead of reaching the
    // texture addresser as one burst from all eight waves.
    auto issue_piece = [&](const TileCtx &c, int kt, int stage, auto piece_c) {
        constexpr int piece = decltype(piece_c)::value;
        const uint32_t lds = lds_base + (uint32_t)(RING_OFF + stage * STAGE_BYTES) + (uint32_t)(wave * NJ) * 1024u;
        if constexpr (piece < NJ) {
            load16_to_lds(c.rs_a, c.off_a[piece], (uint32_t)kt * BKB, lds + piece * 1024u);
        } else if constexpr (piece < 2 * NJ) {
            load16_to_lds(c.rs_b, c.off_b[piece - NJ], (uint32_t)kt * BKB, lds + PANEL_BYTES + (piece - NJ) * 1024u);
        } else if constexpr (piece < NV) {
            // dword d of the step's scales: 4 E8M0 bytes per row
            constexpr int d = piece - 2 * NJ;
            load4_to_lds(c.rs_sc, c.off_sc, (uint32_t)(kt * SCALE_DW + d) * 4u,
                         lds_base + (uint32_t)(SCALE_OFF + stage * SCALE_STAGE + d * 2048) + (uint32_t)(wave >= 4) * 1024u +
                             (uint32_t)(wave & 3) * 256u);
        }
    };
    auto issue_step = [&](const TileCtx &c, int kt, int stage) {
        static_for<NV>([&](auto piece_c) { issue_piece(c, kt, stage, piece_c); });
    };

    // Tile set-up: epilogue parameters of the tile (per-token / per-channel scales) and its
    // first step.  Every wave issues the same number of instructions.
    auto setup = [&](const TileCtx &c, int parity, int stage) {
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
        issue_step(c, 0, stage);
    };

    TileCtx cur, nxt;
    int t = blockIdx.x, parity = 0;
    int gstep = 0;        // K-steps executed by this workgroup so far; ring stage = gstep & 1
    bool first = true;
    decode(t, cur);
    nxt.valid = 0;
    if (cur.valid) setup(cur, 0, 0);

#ifdef DBG_TIMING
#define TSTAMP(slot) do { if (t == 2 * (int)gridDim.x && blockIdx.x == 0 && kt >= 16 && kt < 32) { \
        unsigned long long ts_ = __builtin_readcyclecounter(); \
        if (lane == 0) *reinterpret_cast<unsigned long long *>(smem + EPI_OFF + ((wave * 16 + (kt - 16)) * 4 + (slot)) * 8) = ts_; } } while (0)
#else
#define TSTAMP(slot) do { } while (0)
#endif
    while (cur.valid) {
        Acc acc[MT][NT];
#pragma unroll
        for (int i = 0; i < MT; i++)
#pragma unroll
            for (int j = 0; j < NT; j++)
#pragma unroll
                for (int x = 0; x < 16; x++) acc[i][j][x] = 0;

        v8i fb[NT], fa[MT];              // B and A fragments of the current 64-byte substep
        uint32_t sc[SCALE_DW > 0 ? SCALE_DW : 1][MT + NT];  // raw scale dwords of the current step

        auto read_frag = [&](uint32_t row_off, int ks) {
            // lane (r, g) feeds K bytes [16g, 16g+16) of each 32-byte half of the 64-byte substep
            const uint32_t c0 = (((uint32_t)(ks * 4 + g)) ^ swz) << 4, c1 = (((uint32_t)(ks * 4 + 2 + g)) ^ swz) << 4;
            const v4i lo = lds_read16(row_off + c0), hi = lds_read16(row_off + c1);
            return (v8i){lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
        };
        auto read_substep = [&](int stage, int ks) {
            const uint32_t st = (uint32_t)(RING_OFF + stage * STAGE_BYTES);
#pragma unroll
            for (int s = 0; s < NT; s++) fb[s] = read_frag(st + rd_b + s * 32 * BKB, ks);
#pragma unroll
            for (int s = 0; s < MT; s++) fa[s] = read_frag(st + rd_a + s * 32 * BKB, ks);
        };
        auto read_scales = [&](int stage) {
            if (!MX) return;
#pragma unroll
            for (int d = 0; d < SCALE_DW; d++) {
                const uint32_t ss = (uint32_t)(SCALE_OFF + stage * SCALE_STAGE + d * 2048);
#pragma unroll
                for (int s = 0; s < MT; s++) sc[d][s] = lds_read4(ss + rd_sa + s * 128);
#pragma unroll
                for (int s = 0; s < NT; s++) sc[d][MT + s] = lds_read4(ss + rd_sb + s * 128);
            }
        };
        // The MFMAs of one 64-byte substep.  DMA: between them, issue the requests of the next
        // step (pieces PIECE0 .. PIECE0 + count - 1 of tile cur, step kt_next).
        auto mfma_substep = [&](auto ks_c, auto dma_c, int kt_next, int stage_next) {
            constexpr int ks = decltype(ks_c)::value;
            constexpr bool DMA = decltype(dma_c)::value;
            constexpr int PER = (NV + 1) / 2;            // pieces issued during one substep
            constexpr int PIECE0 = ks * PER;
            static_for<MT * NT>([&](auto idx_c) {
                constexpr int idx = decltype(idx_c)::value;
                constexpr int i = idx / NT, j = idx % NT;
#ifndef DBG_NO_MFMA
                if constexpr (KIND == KIND_F8) {
                    // scale operands: lane group g presents byte 2*ks + g of the row's dword
                    const int sh = 8 * (2 * ks) + 8 * g;
                    acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(fa[i], fb[j], acc[i][j], CBSZ, CBSZ, 0, (int)(sc[0][i] >> sh), 0,
                                                                                (int)(sc[0][MT + j] >> sh));
                } else if constexpr (KIND == KIND_F4) {
                    // substep = 128 elements = scale dword ks; MFMA lo uses byte g, MFMA hi byte 2+g
                    const int sA = (int)(sc[ks][i] >> (8 * g)), sB = (int)(sc[ks][MT + j] >> (8 * g));
                    const v8i alo = (v8i){fa[i][0], fa[i][1], fa[i][2], fa[i][3], 0, 0, 0, 0};
                    const v8i blo = (v8i){fb[j][0], fb[j][1], fb[j][2], fb[j][3], 0, 0, 0, 0};
                    const v8i ahi = (v8i){fa[i][4], fa[i][5], fa[i][6], fa[i][7], 0, 0, 0, 0};
                    const v8i bhi = (v8i){fb[j][4], fb[j][5], fb[j][6], fb[j][7], 0, 0, 0, 0};
                    acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(alo, blo, acc[i][j], 4, 4, 0, sA, 0, sB);
                    acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(ahi, bhi, acc[i][j], 4, 4, 2, sA, 2, sB);
                } else {
                    const v4i alo = (v4i){fa[i][0], fa[i][1], fa[i][2], fa[i][3]}, ahi = (v4i){fa[i][4], fa[i][5], fa[i][6], fa[i][7]};
                    const v4i blo = (v4i){fb[j][0], fb[j][1], fb[j][2], fb[j][3]}, bhi = (v4i){fb[j][4], fb[j][5], fb[j][6], fb[j][7]};
                    acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(alo, blo, acc[i][j], 0, 0, 0);
                    acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(ahi, bhi, acc[i][j], 0, 0, 0);
                }
#endif
                if constexpr (DMA && idx < PER && PIECE0 + idx < NV) {
                    __builtin_amdgcn_sched_barrier(0);
                    issue_piece(cur, kt_next, stage_next, IC<PIECE0 + idx>{});
                    __builtin_amdgcn_sched_barrier(0);
                }
#ifdef DBG_TIMING
                if constexpr (ks == 0 && idx == 3) { const int kt = kt_next - 1; TSTAMP(2); }
#endif
            });
        };

        // The requests of step 0 were the last direct-to-LDS loads this wave issued; only the
        // previous tile's epilogue stores may have been issued after them.
        if (first) CCH_WAIT_VM_LGKM0(0);
        else CCH_WAIT_VM_LGKM0(NSTORES);
        __syncthreads();
        // Steady state: right after the barrier that retires step kt-1, request step kt+1 into
        // the stage it vacated, then compute step kt.  No branches.
        for (int kt = 0; kt + 1 < ksteps; kt++, gstep++) {
            const int stage = gstep & 1;
            TSTAMP(0);
#ifndef DBG_NO_LOADS
            issue_step(cur, kt + 1, stage ^ 1);
#endif
            read_scales(stage);
            read_substep(stage, 0);
            TSTAMP(1);
            mfma_substep(IC<0>{}, std::false_type{}, 0, 0);
            TSTAMP(3);
            read_substep(stage, 1);
            mfma_substep(IC<1>{}, std::false_type{}, 0, 0);
            CCH_WAIT_VM_LGKM0(0);  // this wave's requests for step kt+1 have landed
#ifndef DBG_NO_BARRIER
            __syncthreads();        // ... everybody's have, and everybody is done reading step kt
#endif
        }
        // Last step: the other stage is free for the next tile's first step.
        {
            const int stage = gstep & 1;
            decode(t + gridDim.x, nxt);
#ifndef DBG_NO_LOADS
            if (nxt.valid) setup(nxt, parity ^ 1, stage ^ 1);
#endif
            read_scales(stage);
            read_substep(stage, 0);
            mfma_substep(IC<0>{}, std::false_type{}, 0, 0);
            read_substep(stage, 1);
            mfma_substep(IC<1>{}, std::false_type{}, 0, 0);
            gstep++;
        }
#ifdef DBG_TIMING
        if (t == 2 * (int)gridDim.x && blockIdx.x == 0) {
            __syncthreads();
            for (int i = threadIdx.x; i < 8 * 16 * 4; i += TILE_THREADS)
                reinterpret_cast<unsigned long long *>(const_cast<uint8_t *>(p.sa))[i] =
                    *reinterpret_cast<unsigned long long *>(smem + EPI_OFF + i * 8);
            __syncthreads();
        }
#endif
        first = false;

#ifdef DBG_NO_EPI
        if (acc[0][0][0] != 12345) { cur = nxt; t += gridDim.x; parity ^= 1; continue; }
#endif
        // Epilogue.  Lane (r, g) holds, for sub-tile (i, j), column r and rows
        // (x/4)*8 + g*4 + x%4, x = 0..15.  Sixteen rows at a time go through the wave's private
        // LDS buffer: neighbouring lanes exchange one value so that each writes two adjacent
        // bf16, then every lane reads back 16 contiguous bytes and stores them.  Stores are raw
        // buffer stores whose out-of-range lanes are dropped by the bounds check, so that every
        // lane issues exactly NSTORES of them.
        {
            const uint32_t epi = (uint32_t)(EPI_OFF + wave * EPI_WAVE);
            const uint32_t prm = (uint32_t)(PARAM_OFF + parity * PARAM_SET);
            const bool odd = lane & 1;
            const __amdgpu_buffer_rsrc_t rs_out =
                __builtin_amdgcn_make_buffer_rsrc(p.out + (size_t)cur.m0 * p.n_out, 0, 0x7FFFFFFF, 0x00020000);
            float chs[NT];
            if (EPI != EPI_PLAIN) {
#pragma unroll
                for (int j = 0; j < NT; j++) chs[j] = __uint_as_float(lds_read4(prm + 1024u + (uint32_t)(wn * WN + j * 32 + r) * 4u));
            }
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
                    const int row0 = wm * WM + i * 32 + hh * 16;  // relative to m0
                    const int col0 = cur.j0 + wn * WN_OUT;
#pragma unroll
                    for (int q = 0; q < 16 / RPI; q++) {
                        const int lrow = q * RPI + lane / CPR, chunk = lane % CPR;
                        const v4i val = lds_read16(epi + (uint32_t)(lrow * ROWB + chunk * 16));
                        const int row = row0 + lrow, col = col0 + chunk * 8;
                        const bool ok = (cur.m0 + row < cur.m_end) && (col + 8 <= p.n_out);
                        const uint32_t off = ok ? ((uint32_t)row * (uint32_t)p.n_out + (uint32_t)col) * 2u : 0xFFFFFFF0u;
                        __builtin_amdgcn_raw_buffer_store_b128((v4u){(uint32_t)val[0], (uint32_t)val[1], (uint32_t)val[2], (uint32_t)val[3]},
                                                               rs_out, (int)off, 0, 0);
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
    // whole 128-byte K-steps; output rows must take 16-byte stores
    if (p.K <= 0 || p.K % (BKB * epb) != 0) return false;
    if (p.n_out % 8 != 0 || !aligned(p.out, 16)) return false;
    if ((int64_t)BM * p.n_out * 2 >= ((int64_t)1 << 31)) return false;
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
