// Tiled MFMA GEMM family for gfx950 (B stored K-contiguous, i.e. trans_b = 1):
//   int8 x int8 -> int32   v_mfma_i32_32x32x32_i8          + dequant / dequant+SwiGLU epilogue
//   MXFP8 / MXFP4          v_mfma_scale_f32_32x32x64_f8f6f4 with per-lane E8M0 scale operands
//
// One persistent workgroup (8 waves) per CU walks a global list of 256x256 output tiles built
// from the prefix sums of the group sizes (a dense problem is one group).
//   * K advances in steps of 128 bytes per row, the size of an L2 line: direct-to-LDS loads
//     that cover whole lines reach about 1.5x the L2 throughput of half-line requests.  The A
//     and B panels of a step (256 rows x 128 B each) go global -> LDS without a VGPR round
//     trip into a ring of two stages.  A stage is read for the last time about 5/8 through
//     its step; the requests that refill it (two steps ahead of use) follow the step's one
//     barrier and are threaded between the remaining MFMAs.
//   * MX scales travel 16 bytes per row at a time (4 MXFP8 steps, 2 MXFP4 steps) into a pair of
//     scale buffers: a per-step 4-byte fetch touches one L2 line per lane and costs as many
//     line requests as the whole data panel.
//   * Each wave owns 128 x 64 outputs as 4 x 2 MFMA tiles of 32 x 32 and reads its fragments
//     with 16-byte LDS reads from an XOR-swizzled panel layout (no bank conflicts).  Fragment
//     registers are refilled as soon as the MFMAs that read them have been issued, so LDS
//     latency hides behind the other MFMAs of the step.
//   * The K loop is a single basic block without compiler-visible memory loads; the last two
//     steps of a tile are peeled and request the next tile's first two steps, with empty
//     buffer descriptors when there is no next tile, so they are branch-free as well.
//   * Epilogues (dequant, SwiGLU, bf16 rounding) run on the accumulators; results pass through
//     a wave-private 1 KiB LDS buffer so that every lane stores 16 contiguous bytes.
//
// Stands in for Catlass::Gemm::Block::BlockMmadTla<MmadMx<...>> as instantiated in
// examples/ascend950_fp4_mx_alltoallv_grouped_matmul/ascend950_fp4_mx_alltoallv_grouped_matmul_device.h:59-71,
// FixpipeBlockMmad (include/catccos/dgemm/block/block_mmad_preload_fixpipe.hpp:151-379), the
// tile loop of BlockMmadSchedulerAllToAllVAllGather
// (include/catccos/dgemm/block/block_scheduler_alltoallv_allgather.hpp:122-168) and the epilogues
// include/catccos/epilogue/block/block_epilogue_per_token_dequant[_swiglu].hpp.
#include <atomic>
#include <type_traits>
#include <utility>

#include "common.h"
#include "gemm_common.h"
#include "mx_formats.h"

namespace cch {

typedef int v2i __attribute__((ext_vector_type(2)));
typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v8i __attribute__((ext_vector_type(8)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef unsigned int v4u __attribute__((ext_vector_type(4)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));

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

// dynamic LDS map.  The small areas come first so that every read of them is one base register
// plus a 16-bit instruction offset; behind the 128 KiB ring each distinct offset would need an
// address register of its own.
constexpr int SCALE_OFF = 0;                                 // two buffers of (256 A + 256 B rows) x 16 scale bytes
constexpr int SCALE_BUF = 8192;
constexpr int EPI_OFF = SCALE_OFF + 2 * SCALE_BUF;           // per wave: 1 KiB of output staging
constexpr int EPI_WAVE = 1024;
constexpr int PARAM_OFF = EPI_OFF + NWAVES * EPI_WAVE;       // per tile parity: 256 per_tok + 256 per_ch floats
constexpr int PARAM_SET = 2048;
constexpr int RING_OFF = PARAM_OFF + 2 * PARAM_SET;          // NSTAGE stages of an A panel and a B panel
constexpr int LDS_BYTES = RING_OFF + NSTAGE * STAGE_BYTES;   // 156 KiB of the CU's 160 KiB

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
__device__ __forceinline__ Rsrc make_rsrc(const void *base, uint32_t bytes = 0x7FFFFFFFu)
{
    const uint64_t b = reinterpret_cast<uint64_t>(base);
    Rsrc rs;
    rs[0] = __builtin_amdgcn_readfirstlane((int)(uint32_t)b);
    rs[1] = __builtin_amdgcn_readfirstlane((int)(uint32_t)(b >> 32));  // stride 0, no swizzle
    rs[2] = __builtin_amdgcn_readfirstlane((int)bytes);                // num_records (bytes); reads past it return 0
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
    u[2] = __builtin_amdgcn_readfirstlane(rs[2]);
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
// The same load with the non-temporal hint: the line is not kept in L2 after use (weight panels of
// experts so small that no other workgroup reads them again).
__device__ __forceinline__ void load16_to_lds_nt(Rsrc rs, uint32_t voff, uint32_t soff, uint32_t lds_addr)
{
    rs = scalar_rsrc(rs);
    soff = (uint32_t)__builtin_amdgcn_readfirstlane((int)soff);
    lds_addr = (uint32_t)__builtin_amdgcn_readfirstlane((int)lds_addr);
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen nt lds"
                 :
                 : "s"(lds_addr), "v"(voff), "s"(rs), "s"(soff)
                 : "memory", "m0");
}
// The same 16-byte load, performed only when `enable` (wave-uniform) is non-zero, without a
// branch: the load is issued with an empty EXEC mask otherwise.  Keeps the K loop one basic
// block, which the register allocator handles far better than a loop with a diamond in it.
__device__ __forceinline__ void load16_to_lds_if(int enable, Rsrc rs, uint32_t voff, uint32_t soff, uint32_t lds_addr)
{
    rs = scalar_rsrc(rs);
    soff = (uint32_t)__builtin_amdgcn_readfirstlane((int)soff);
    lds_addr = (uint32_t)__builtin_amdgcn_readfirstlane((int)lds_addr);
    enable = __builtin_amdgcn_readfirstlane(enable);
    uint64_t saved;
    asm volatile("s_mov_b64 %0, exec\n\ts_cmp_lg_u32 %1, 0\n\ts_cselect_b64 exec, %0, 0\n\ts_mov_b32 m0, %2\n\ts_nop 0\n\t"
                 "buffer_load_dwordx4 %3, %4, %5 offen lds\n\ts_mov_b64 exec, %0"
                 : "=&s"(saved)
                 : "s"(enable), "s"(lds_addr), "v"(voff), "s"(rs), "s"(soff)
                 : "memory", "m0", "scc");
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
    uint32_t lim;                       // descriptor size: 0 for a tile past the end, whose requests then fetch nothing
    Rsrc rs_a, rs_b, rs_sc;             // buffer descriptors: A rows from m0, B of the expert, scales
    uint32_t off_a[NJ], off_b[NJ];      // per lane: source row * pitch + chunk * 16
    uint32_t off_sc;                    // per lane: scale row * sld (A rows for waves 0-3, B columns for 4-7)
};

// TB = 1: B is stored [N, K] (K contiguous) and its panel is staged like A's.  TB = 0 (int8 and
// MXFP8): B is stored [K, N]; a step's panel is staged as 128 K-rows of 256 bytes and the MFMA
// operand, which wants K-contiguous bytes per column, is read with the transposing LDS load
// ds_read_b64_tr_b8.  Inside a group of 16 lanes that load treats the lanes' addresses as 16
// row segments of 8 bytes and returns to lane j byte (j & 7) of segments (j >> 3), (j >> 3) + 2,
// ..., (j >> 3) + 14.  Lane i of a group therefore addresses K-row i/2 at columns 8*(i & 1) ..
// +7, and lane j receives 8 consecutive K bytes of column j.
template <int KIND, int EPI, int FMT, int TB>
__global__ __launch_bounds__(TILE_THREADS) void gemm_tile_kernel(GemmProblem p)
{
    using KT = KindTraits<KIND>;
    using Acc = typename KT::Acc;
    constexpr bool MX = KIND != KIND_I8;
    constexpr bool SWIGLU = EPI == EPI_DEQUANT_SWIGLU;
    constexpr int BN_OUT = SWIGLU ? BN / 2 : BN;   // output columns per tile
    constexpr int WN_OUT = SWIGLU ? WN / 2 : WN;   // output columns per wave
    constexpr int SCALE_DW = KT::SCALE_DW;         // scale dwords per row per step
    constexpr int NV = 2 * NJ;                     // direct-to-LDS instructions per wave per step
    // MX scales travel 16 bytes per row at a time: one request per wave covers SPG steps
    constexpr int SPG = SCALE_DW > 0 ? 4 / SCALE_DW : 1;
    constexpr int CBSZ = FMT == CCH_FMT_E2M1 ? 4 : (FMT == CCH_FMT_E5M2 ? 1 : 0);
    constexpr int ROWB = WN_OUT * 2;               // epilogue staging: bytes per row
    constexpr int CPR = ROWB / 16;                 // 16-byte chunks per staged row
    constexpr int PASS_ROWS = 64 / CPR;            // rows staged per pass: 1 KiB, one read-back instruction
    constexpr int NPASS = 32 / PASS_ROWS;          // passes per 32-row MFMA tile

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
    const uint32_t rd_sa = (uint32_t)(wm * WM + r) * 16;
    // B scales: TB = 1 like A's, 16 bytes per column; TB = 0 eight 512-byte rows per group,
    // [K64 block][column][2]
    const uint32_t rd_sb = TB ? 4096u + (uint32_t)(wn * WN + r) * 16 : 4096u + (((uint32_t)(wn * WN + r) * 2) & ~3u);
    const uint32_t sb_sel = (r & 1) ? 0x07060302u : 0x05040100u;   // TB = 0: which half of the dwords holds this column
    // TB = 0 fragment reads: lane (q = lane / 16, i = lane % 16) addresses K-row 16*(q/2) + i/2 of
    // the substep part and the 8-byte half (i & 1) of 16-byte chunk wn*4 + j*2 + (q & 1), whose
    // position in the row is swizzled by twice the row's low bits (i / 2): the 32 lanes of one pass
    // of the load address 8 K-rows x 2 neighbouring chunks, and chunk ^ 2*(row & 7) puts those 16
    // pieces on 16 different chunk positions of the 256-byte row, i.e. on all 64 banks once
    // For FP4 the panel has 256 K-rows of 128 bytes (two columns per byte) and the 4-bit form of
    // the load is a 16 x 16 nibble transpose: lane i addresses K-row i at 16 columns (8 bytes) and
    // lane j receives 16 consecutive K nibbles of column j; the chunk swizzle uses row bits 1..3.
    constexpr bool FP4K = KIND == KIND_F4;
    constexpr int EPB = KT::ELEMS_PER_BYTE;
    constexpr int BROW = BN / EPB;               // bytes per K-row of the TB = 0 panel
    constexpr int BCPR = BROW / 16;              // 16-byte chunks per K-row
    constexpr int BRPI = 64 / BCPR;              // K-rows filled by one direct-to-LDS instruction
    const int tq = lane >> 4, ti = lane & 15;
    const uint32_t rd_bt = FP4K ? (uint32_t)PANEL_BYTES + (uint32_t)(32 * (tq >> 1) + ti) * 128u +
                                      ((uint32_t)((wn * 2) ^ (ti >> 1)) << 4) + (uint32_t)(tq & 1) * 8u
                                : (uint32_t)PANEL_BYTES + (uint32_t)(16 * (tq >> 1) + (ti >> 1)) * 256u +
                                      ((uint32_t)((wn * 4 + (tq & 1)) ^ ((ti >> 1) << 1)) << 4) + (uint32_t)(ti & 1) * 8u;
    const int ldb = TB ? lda : p.N / EPB;   // bytes between consecutive rows of B as stored
    // Rows that belong to no group are written as zeros (the reference's golden pads them,
    // examples/utils/gen_data_fp4_mx_alltoallv_gmm.py:788-790): all workgroups share the range,
    // 16 bytes per thread and pass; usually it is empty.
    const bool has_map = EPI == EPI_PLAIN && p.out_row_map != nullptr;   // rows go where the map says
    if (p.group_sizes && !has_map) {
        const size_t begin = (size_t)uniform(tab.row_start[p.num_groups]) * p.n_out / 8, end = (size_t)p.T * p.n_out / 8;
        v4u *o16 = reinterpret_cast<v4u *>(p.out);
        for (size_t i = begin + (size_t)blockIdx.x * TILE_THREADS + threadIdx.x; i < end; i += (size_t)gridDim.x * TILE_THREADS)
            o16[i] = (v4u){0, 0, 0, 0};
    }

    // Workgroups that take tiles: all of them, or (balance) just enough for the same number of
    // rounds, in whole groups of eight so that every XCD keeps the same share.
    int nwg = gridDim.x;
    if (p.balance_rounds && total_tiles > 0) {
        const int rounds = (total_tiles + (int)gridDim.x - 1) / (int)gridDim.x;
        nwg = min((int)gridDim.x, (((total_tiles + rounds - 1) / rounds) + 7) & ~7);
    }
    nwg = uniform(nwg);

    int gi = 0;           // scale groups requested so far; group n lives in scale buffer n & 1
    int gbase = 0;        // value of gi when the current tile's group 0 was requested

    auto decode = [&](int t, TileCtx &c) {
        // A tile index past the end decodes to the last tile with empty descriptors: its requests
        // can then be issued unconditionally (they read nothing and write zeros into LDS areas
        // that are never used), which keeps the peeled steps free of branches.
        c.valid = t < total_tiles;
        c.lim = c.valid ? 0x7FFFFFFFu : 0u;
        t = max(min(t, total_tiles - 1), 0);
        if (p.tile_order == 1 && (nwg & 7) == 0 && t < total_tiles - total_tiles % nwg) {
            // Workgroup w of a round runs on XCD w % 8: give each XCD a run of gridDim.x / 8
            // consecutive tiles of the round (whole row tiles next to each other), so that its L2
            // fetches one or two A panels and the B panels of one or two experts per round.
            const int G = nwg, j = t / G, w = t - j * G;
            t = j * G + (w & 7) * (G >> 3) + (w >> 3);
        }
        const int tr = t / n_tiles, nt = t - tr * n_tiles;
        c.e = uniform(find_group(tab, p.num_groups, tr));
        c.m0 = uniform(tab.row_start[c.e] + (tr - tab.tile_start[c.e]) * BM);
        c.m_end = uniform(tab.row_start[c.e + 1]);
        c.j0 = nt * BN_OUT;
        // A's descriptor ends with the group: requests for tile rows past it are dropped by the
        // bounds check (LDS receives zeros), and their products land in accumulators that are
        // never stored.
        c.rs_a = make_rsrc(p.a + (size_t)c.m0 * lda, min((uint32_t)min(c.m_end - c.m0, BM) * (uint32_t)lda, c.lim));
        c.rs_b = make_rsrc(p.b + (size_t)c.e * p.b_stride, c.lim);
        // Instruction j of this wave fills rows (wave*NJ + j)*8 .. +7 of a panel; lane l lands at
        // row l/8, chunk position l%8 and must therefore fetch chunk (l%8) ^ swizzle(row).
#pragma unroll
        for (int j = 0; j < NJ; j++) {
            const int row = (wave * NJ + j) * 8 + (lane >> 3);
            const uint32_t chunk = ((uint32_t)(lane & 7) ^ swizzle_of_row(row)) * 16u;
            c.off_a[j] = (uint32_t)row * (uint32_t)lda + chunk;
            if (TB) {
                int col;  // B row (= logical column) feeding tile row `row`
                if (SWIGLU) {
                    // tile row = wn*64 + h*32 + c: h = 0 gate, 1 up; output column j0 + wn*32 + c
                    col = ((row >> 5) & 1) * p.n_out + min(c.j0 + (row >> 6) * 32 + (row & 31), p.n_out - 1);
                } else {
                    col = min(c.j0 + row, p.N - 1);
                }
                c.off_b[j] = (uint32_t)col * (uint32_t)lda + chunk;
            } else {
                // Instruction j fills K-rows (wave*NJ + j)*4 .. +3 of the panel, 256 bytes each;
                // lane l lands at row l/16, chunk position l%16 and fetches tile chunk
                // (l%16) ^ 2*(row & 7): 16 tile columns, clamped to stay inside the row of B.
                const int kr = (wave * NJ + j) * BRPI + lane / BCPR;
                const int tc = (lane % BCPR) ^ (FP4K ? (kr >> 1) & 7 : (kr & 7) << 1);
                constexpr int CPC = 16 * EPB;  // columns per chunk
                int col;
                if (SWIGLU) col = ((tc >> 1) & 1) * p.n_out + min(c.j0 + (tc >> 2) * 32 + (tc & 1) * 16, p.n_out - 16);
                else col = min(c.j0 + tc * CPC, p.N - CPC);
                c.off_b[j] = (uint32_t)kr * (uint32_t)ldb + (uint32_t)(col / EPB);
            }
        }
        if (MX) {
            const int idx = (wave & 3) * 64 + lane;
            if (wave < 4) {
                c.rs_sc = make_rsrc(p.sa + (size_t)c.m0 * p.sld, (uint32_t)min((int64_t)(p.T - c.m0) * p.sld, (int64_t)c.lim));
                c.off_sc = (uint32_t)min(idx, c.m_end - 1 - c.m0) * (uint32_t)p.sld;
            } else if (TB) {
                c.rs_sc = make_rsrc(p.sb + (size_t)c.e * p.sb_stride, (uint32_t)min((int64_t)p.N * p.sld, (int64_t)c.lim));
                c.off_sc = (uint32_t)min(c.j0 + idx, p.N - 1) * (uint32_t)p.sld;
            } else {
                // [K/64][N][2]: a scale group is 8 rows of K64 blocks (4 MXFP8 steps, 2 MXFP4 steps)
                // x 256 columns x 2 bytes; wave 4+i fetches rows 2i, 2i+1, lane l 16 bytes of row l/32
                c.rs_sc = make_rsrc(p.sb + (size_t)c.e * p.sb_stride, (uint32_t)min((int64_t)p.N * p.sld, (int64_t)c.lim));
                c.off_sc = (uint32_t)((lane >> 5) + 2 * (wave - 4)) * (uint32_t)p.N * 2u + (uint32_t)c.j0 * 2u + (uint32_t)(lane & 31) * 16u;
            }
        }
    };

    // Requests K-step kt of tile c into ring stage `stage`: NV instructions per wave, issued one
    // at a time (piece 0..NV-1) so that they interleave with MFMAs instead of reaching the
    // texture addresser as one burst from all eight waves.
    auto issue_piece = [&](const TileCtx &c, int kt, int stage, auto piece_c, auto ntb_c) {
        constexpr int piece = decltype(piece_c)::value;
        constexpr bool NTB = decltype(ntb_c)::value != 0;
        const uint32_t lds = lds_base + (uint32_t)(RING_OFF + stage * STAGE_BYTES) + (uint32_t)(wave * NJ) * 1024u;
        if constexpr (piece < NJ) {
            load16_to_lds(c.rs_a, c.off_a[piece], (uint32_t)kt * BKB, lds + piece * 1024u);
        } else if constexpr (piece < 2 * NJ) {
            if constexpr (NTB)
                load16_to_lds_nt(c.rs_b, c.off_b[piece - NJ], TB ? (uint32_t)kt * BKB : (uint32_t)kt * (BKB * EPB) * (uint32_t)ldb,
                                 lds + PANEL_BYTES + (piece - NJ) * 1024u);
            else
                load16_to_lds(c.rs_b, c.off_b[piece - NJ], TB ? (uint32_t)kt * BKB : (uint32_t)kt * (BKB * EPB) * (uint32_t)ldb,
                              lds + PANEL_BYTES + (piece - NJ) * 1024u);
        }
    };
    // Scale group `grp` of tile c (steps grp*SPG .. grp*SPG+SPG-1) into scale buffer `buf`: waves
    // 0-3 fetch 16 bytes of each A row, one row per lane; waves 4-7 the same for the B rows
    // (TB = 1) or 1 KiB each of the group's eight [column][2] rows (TB = 0).
    auto issue_scales = [&](int newgrp, const TileCtx &c, int grp, int buf) {
        if constexpr (MX)
            load16_to_lds_if(newgrp, c.rs_sc, c.off_sc, (TB || wave < 4) ? (uint32_t)grp * 16u : (uint32_t)grp * 16u * (uint32_t)p.N,
                             lds_base + (uint32_t)(SCALE_OFF + buf * SCALE_BUF) + (uint32_t)(wave >= 4) * 4096u + (uint32_t)(wave & 3) * 1024u);
    };
    auto issue_step = [&](const TileCtx &c, int kt, int stage) {
        static_for<NV>([&](auto piece_c) { issue_piece(c, kt, stage, piece_c, IC<0>{}); });
    };

    // Tile set-up: epilogue parameters of the tile (per-token / per-channel scales) and its
    // first step.  Every wave issues the same number of instructions.
    auto setup = [&](const TileCtx &c, int parity, int stage) {
        if (EPI != EPI_PLAIN) {
            const int idx = (wave & 3) * 64 + lane;
            // destination of lane 0 of this wave; lane l lands 4*l bytes further
            const uint32_t dst = lds_base + (uint32_t)(PARAM_OFF + parity * PARAM_SET) + (uint32_t)(wave & 3) * 256u;
            load4_to_lds(make_rsrc(p.per_tok + c.m0, c.lim), (uint32_t)min(idx, c.m_end - 1 - c.m0) * 4u, 0u, dst);
            int col;
            if (SWIGLU) col = ((idx >> 5) & 1) * p.n_out + min(c.j0 + (idx >> 6) * 32 + (idx & 31), p.n_out - 1);
            else col = min(c.j0 + idx, p.N - 1);
            load4_to_lds(make_rsrc(p.per_ch + (size_t)c.e * p.N, c.lim), (uint32_t)col * 4u, 0u, dst + 1024u);
        } else {
            // destination rows of the tile's 256 rows, where the per-token scales of the other
            // epilogues go; without a map the descriptor is empty and nothing is fetched
            const int idx = (wave & 3) * 64 + lane;
            const uint32_t dst = lds_base + (uint32_t)(PARAM_OFF + parity * PARAM_SET) + (uint32_t)(wave & 3) * 256u;
            load4_to_lds(make_rsrc(p.out_row_map + c.m0, has_map ? c.lim : 0u), (uint32_t)min(idx, c.m_end - 1 - c.m0) * 4u, 0u, dst);
        }
        issue_scales(1, c, 0, gi & 1);
        gi++;
        issue_step(c, 0, stage);
    };

    TileCtx cur, nxt;
    int t = (int)blockIdx.x < nwg ? (int)blockIdx.x : total_tiles, parity = 0;
    int gstep = 0;        // K-steps executed by this workgroup so far; ring stage = gstep & 1
    bool first = true;
    decode(t, cur);
    nxt.valid = 0;
    if (cur.valid) {
        setup(cur, 0, 0);
        issue_step(cur, 1, 1);
    }
    while (cur.valid) {
        Acc acc[MT][NT];
#pragma unroll
        for (int i = 0; i < MT; i++)
#pragma unroll
            for (int j = 0; j < NT; j++)
#pragma unroll
                for (int x = 0; x < 16; x++) acc[i][j][x] = 0;

        int nbase = 0;  // gi when the next tile's scale group 0 is requested
        // Fragment registers.  fa[i] and fb0 hold the first 64-byte substep of the current
        // step, fb1 the second; fa[i] is refilled with its next contents as soon as the MFMAs
        // that read it have been issued, so that LDS latency hides behind the other MFMAs.
        v8i fa[MT], fb0[NT], fb1[NT];
        constexpr int NSC = SCALE_DW > 0 ? SCALE_DW : 1;
        uint32_t sc[NSC][MT + NT];  // raw scale dwords of the current step

        auto read_frag = [&](uint32_t row_off, int ks) {
            // lane (r, g) feeds K bytes [16g, 16g+16) of each 32-byte half of the 64-byte substep
            const uint32_t c0 = (((uint32_t)(ks * 4 + g)) ^ swz) << 4, c1 = (((uint32_t)(ks * 4 + 2 + g)) ^ swz) << 4;
            const v4i lo = lds_read16(row_off + c0), hi = lds_read16(row_off + c1);
            return (v8i){lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
        };
        auto frag_a = [&](int stage, int ks, int i) { return read_frag((uint32_t)(RING_OFF + stage * STAGE_BYTES) + rd_a + i * 32 * BKB, ks); };
        auto frag_b = [&](int stage, int ks, int j) {
            if constexpr (TB) {
                return read_frag((uint32_t)(RING_OFF + stage * STAGE_BYTES) + rd_b + j * 32 * BKB, ks);
            } else {
                typedef __attribute__((address_space(3))) v2i *LdsV2;
                v2i t0, t1, t2, t3;
                if constexpr (FP4K) {
                    // four nibble transposes: K elements 32g+0..15, 32g+16..31, 64+32g+0..15, 64+32g+16..31 of the substep
                    const uint32_t base = (uint32_t)(RING_OFF + stage * STAGE_BYTES) + (rd_bt ^ ((uint32_t)j << 4)) + (uint32_t)ks * (128u * 128u);
                    t0 = __builtin_amdgcn_ds_read_tr4_b64_v2i32((LdsV2)(uintptr_t)(lds_base + base));
                    t1 = __builtin_amdgcn_ds_read_tr4_b64_v2i32((LdsV2)(uintptr_t)(lds_base + base + 16u * 128u));
                    t2 = __builtin_amdgcn_ds_read_tr4_b64_v2i32((LdsV2)(uintptr_t)(lds_base + base + 64u * 128u));
                    t3 = __builtin_amdgcn_ds_read_tr4_b64_v2i32((LdsV2)(uintptr_t)(lds_base + base + 80u * 128u));
                } else {
                    // four byte transposes: K bytes 16g+0..7, 16g+8..15, 32+16g+0..7, 32+16g+8..15 of the substep
                    const uint32_t base = (uint32_t)(RING_OFF + stage * STAGE_BYTES) + (rd_bt ^ ((uint32_t)j << 5)) + (uint32_t)ks * (64u * 256u);
                    t0 = __builtin_amdgcn_ds_read_tr8_b64_v2i32((LdsV2)(uintptr_t)(lds_base + base));
                    t1 = __builtin_amdgcn_ds_read_tr8_b64_v2i32((LdsV2)(uintptr_t)(lds_base + base + 8u * 256u));
                    t2 = __builtin_amdgcn_ds_read_tr8_b64_v2i32((LdsV2)(uintptr_t)(lds_base + base + 32u * 256u));
                    t3 = __builtin_amdgcn_ds_read_tr8_b64_v2i32((LdsV2)(uintptr_t)(lds_base + base + 40u * 256u));
                }
                return (v8i){t0[0], t0[1], t1[0], t1[1], t2[0], t2[1], t3[0], t3[1]};
            }
        };
        // Scale dwords of K-step kt of the current tile
        auto read_scales = [&](int kt, uint32_t (&dst)[NSC][MT + NT]) {
            if (!MX) return;
            const uint32_t ss = (uint32_t)(SCALE_OFF + ((gbase + kt / SPG) & 1) * SCALE_BUF) + (uint32_t)(kt % SPG) * (SCALE_DW * 4u);
#pragma unroll
            for (int d = 0; d < SCALE_DW; d++) {
#pragma unroll
                for (int s = 0; s < MT; s++) dst[d][s] = lds_read4(ss + rd_sa + s * 512 + d * 4);
#pragma unroll
                for (int s = 0; s < NT; s++) {
                    if constexpr (TB) {
                        dst[d][MT + s] = lds_read4(ss + rd_sb + s * 512 + d * 4);
                    } else {
                        // The two K32 scales of K64 row 2x and of row 2x+1, for this column: bytes
                        // 2*ks + g of the step's dword as in the TB = 1 layout.  Each row holds two
                        // columns per dword; the permute keeps this column's half of both.
                        const uint32_t sb0 = (uint32_t)(SCALE_OFF + ((gbase + kt / SPG) & 1) * SCALE_BUF) + rd_sb + s * 64 +
                                             (uint32_t)((kt % SPG) * (2 * SCALE_DW) + d * 2) * 512u;
                        dst[d][MT + s] = __builtin_amdgcn_perm(lds_read4(sb0 + 512), lds_read4(sb0), sb_sel);
                    }
                }
            }
        };
        // One MFMA of row block i of a 64-byte substep; m = 0 .. MPR-1 walks the row: all
        // column blocks on the low 32 bytes, then (int8 and FP4, which take two MFMAs per
        // 64 bytes) all on the high 32 bytes, so that consecutive MFMAs never share an accumulator.
        constexpr int MPR = KIND == KIND_F8 ? NT : 2 * NT;  // MFMAs per row block
        auto mfma_one = [&](auto ks_c, auto i_c, auto m_c, const v8i &a, const v8i (&b)[NT]) {
            constexpr int ks = decltype(ks_c)::value, i = decltype(i_c)::value, m = decltype(m_c)::value;
            constexpr int j = m % NT, half = m / NT;
            if constexpr (KIND == KIND_F8) {
                // scale operands: lane group g presents byte 2*ks + g of the row's dword
                const int sh = 8 * (2 * ks) + 8 * g;
                acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a, b[j], acc[i][j], CBSZ, CBSZ, 0, (int)(sc[0][i] >> sh), 0,
                                                                            (int)(sc[0][MT + j] >> sh));
            } else if constexpr (KIND == KIND_F4) {
                // substep = 128 elements = scale dword ks; the low MFMA uses byte g, the high one byte 2+g
                const int sA = (int)(sc[ks][i] >> (8 * g)), sB = (int)(sc[ks][MT + j] >> (8 * g));
                const v8i ah = (v8i){a[4 * half], a[4 * half + 1], a[4 * half + 2], a[4 * half + 3], 0, 0, 0, 0};
                const v8i bh = (v8i){b[j][4 * half], b[j][4 * half + 1], b[j][4 * half + 2], b[j][4 * half + 3], 0, 0, 0, 0};
                acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(ah, bh, acc[i][j], 4, 4, 2 * half, sA, 2 * half, sB);
            } else {
                const v4i ah = (v4i){a[4 * half], a[4 * half + 1], a[4 * half + 2], a[4 * half + 3]};
                const v4i bh = (v4i){b[j][4 * half], b[j][4 * half + 1], b[j][4 * half + 2], b[j][4 * half + 3]};
                acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(ah, bh, acc[i][j], 0, 0, 0);
            }
        };
        auto mfma_row = [&](auto ks_c, auto i_c, const v8i &a, const v8i (&b)[NT]) {
            static_for<MPR>([&](auto m_c) { mfma_one(ks_c, i_c, m_c, a, b); });
        };

        // One K-step.  On entry fa / fb0 / sc hold the step's first substep.  MODE 0: steady
        // state, requests step kt+2 of this tile; 1: second to last step, requests the next
        // tile's set-up and first step; 2: last step, requests the next tile's second step and
        // prefetches no fragments.  The ring stage a step occupies is read for the last time
        // just before the step's barrier, and the requests issued after that barrier refill
        // it, two steps ahead of its use.  Everything that follows the barrier is threaded
        // between the step's remaining MFMAs, one or two instructions at a time, so that the
        // matrix pipe keeps running while the wave issues them.
        auto step = [&](auto mode_c, auto mta_c, auto ntb_c, int kt) {
            constexpr int MODE = decltype(mode_c)::value;
            constexpr int MTA = decltype(mta_c)::value;   // row blocks of this wave that hold rows of the group
            const int stage = gstep & 1, nstage = stage ^ 1;
            static_for<MT>([&](auto i_c) {
                constexpr int i = decltype(i_c)::value;
                if constexpr (i < MTA) mfma_row(IC<0>{}, i_c, fa[i], fb0);
                __builtin_amdgcn_sched_barrier(0);
                if constexpr (i < MTA) fa[i] = frag_a(stage, 1, i);
                if constexpr (i < NT && MTA > 0) fb1[i] = frag_b(stage, 1, i);
                __builtin_amdgcn_sched_barrier(0);
            });
            if constexpr (MTA > 0) mfma_row(IC<1>{}, IC<0>{}, fa[0], fb1);
            __builtin_amdgcn_sched_barrier(0);
            // Every LDS read of this step has been issued; once they have returned and the
            // requests of step kt+1 have landed, for all waves, the stage can be refilled.
            CCH_WAIT_VM_LGKM0(0);
            __syncthreads();
            constexpr int SLOTS = MTA > 0 ? (MTA - 1) * MPR : 0;   // MFMAs left in this step
            constexpr int NREQ = NV + (MX ? 1 : 0);                // requests of a steady step
            constexpr int PER_SLOT = SLOTS >= 2 ? (NREQ + SLOTS - 2) / (SLOTS - 1) : NREQ;
            const int newgrp = ((kt + 2) & (SPG - 1)) == 0;
            // what follows the first MFMA after the barrier: the next step's first fragments, and
            // in the peeled steps the next tile's requests
            auto after_barrier = [&]() {
                if constexpr (MODE != 2 && MTA > 0) {
#pragma unroll
                    for (int j = 0; j < NT; j++) fb0[j] = frag_b(nstage, 0, j);
                    fa[0] = frag_a(nstage, 0, 0);
                }
                if constexpr (MODE == 1) {
                    nbase = gi;
                    setup(nxt, parity ^ 1, stage);
                } else if constexpr (MODE == 2) {
                    issue_step(nxt, 1, stage);
                }
            };
            auto requests = [&](auto first_c) {
                constexpr int first_piece = decltype(first_c)::value;
                if constexpr (MODE == 0) {
                    static_for<PER_SLOT>([&](auto q_c) {
                        constexpr int piece = first_piece + decltype(q_c)::value;
                        if constexpr (piece < NV) issue_piece(cur, kt + 2, stage, IC<piece>{}, ntb_c);
                        else if constexpr (piece == NV && MX) {
                            issue_scales(newgrp, cur, (kt + 2) / SPG, gi & 1);
                        }
                    });
                }
            };
            if constexpr (SLOTS == 0) {
                // a wave with at most one row block to compute: nothing to hide the requests behind
                after_barrier();
                requests(IC<0>{});
            }
            static_for<SLOTS>([&](auto slot_c) {
                constexpr int slot = decltype(slot_c)::value;
                constexpr int i = 1 + slot / MPR, m = slot % MPR;
                mfma_one(IC<1>{}, IC<i>{}, IC<m>{}, fa[i], fb1);
                __builtin_amdgcn_sched_barrier(0);
                // The SwiGLU kernel measured 3 % faster with the requests ahead of the next step's
                // first fragment reads, the others 1 % slower.
                if constexpr (SWIGLU) {
                    if constexpr (slot == SLOTS - 1) after_barrier();
                    else requests(IC<slot * PER_SLOT>{});
                } else {
                    if constexpr (slot == 0) after_barrier();
                    else requests(IC<(slot - 1) * PER_SLOT>{});
                }
                if constexpr (MODE != 2 && m == MPR - 1) fa[i] = frag_a(nstage, 0, i);
                __builtin_amdgcn_sched_barrier(0);
            });
            if constexpr (MODE == 0) gi += MX ? newgrp : 0;
            if constexpr (MODE != 2) read_scales(kt + 1, sc);
            if constexpr (MODE != 0) {
                // Pin the accumulators here: otherwise the compiler sinks the MFMAs of the
                // peeled steps into the epilogue and spills their fragments to get them there.
#pragma unroll
                for (int i = 0; i < MT; i++)
#pragma unroll
                    for (int j = 0; j < NT; j++) asm volatile("" : "+v"(acc[i][j]));
            }
            gstep++;
        };
        // Tile prologue.  In flight, oldest first: this tile's set-up and first step, its
        // second step (NV requests), then the previous tile's epilogue stores.
        constexpr int NSTORES = MT * NPASS;
        constexpr int NSTEP1 = NV;  // requests of the tile's second step
        if (first) CCH_WAIT_VM_LGKM0(NSTEP1);
        else CCH_WAIT_VM_LGKM0(NSTEP1 + NSTORES);
        __syncthreads();
        // Row blocks of this wave that hold rows of the group: the K loop is instantiated for
        // each count, and a wave whose rows lie wholly past the end of a short group issues its
        // requests and barriers but no matrix instruction (its SIMD then belongs to the other
        // wave it hosts, which covers the other half of the tile's rows).
        auto k_loop = [&](auto mta_c, auto ntb_c) {
            constexpr int MTA = decltype(mta_c)::value;
            const int stage = gstep & 1;
            if constexpr (MTA > 0) {
                read_scales(0, sc);
#pragma unroll
                for (int j = 0; j < NT; j++) fb0[j] = frag_b(stage, 0, j);
#pragma unroll
                for (int i = 0; i < MTA; i++) fa[i] = frag_a(stage, 0, i);
            }
            // The step count is made opaque per tile: addresses that depend on it (the scale
            // reads of the peeled steps) would otherwise be hoisted out of the tile loop and
            // held in registers through the K loop.
            int nk = ksteps;
            asm volatile("" : "+s"(nk));
            for (int kt = 0; kt + 2 < nk; kt++) step(IC<0>{}, mta_c, ntb_c, kt);
            decode(t + nwg, nxt);
            step(IC<1>{}, mta_c, ntb_c, nk - 2);
            step(IC<2>{}, mta_c, ntb_c, nk - 1);
        };
        const int mta = uniform(min(max((cur.m_end - cur.m0 - wm * WM + 31) >> 5, 0), MT));
        // Weight panels of an expert with at most nt_b_max_tiles row tiles are read by that many
        // workgroups and never again: their steady-state requests carry the non-temporal hint.
        const bool ntb = uniform(p.nt_b_max_tiles > 0 && tab.tile_start[cur.e + 1] - tab.tile_start[cur.e] <= p.nt_b_max_tiles);
        if (ntb) {
            if (mta == MT) k_loop(IC<MT>{}, IC<1>{});
            else if (mta == 0) k_loop(IC<0>{}, IC<1>{});
            else if (mta == 1) k_loop(IC<1>{}, IC<1>{});
            else if (mta == 2) k_loop(IC<2>{}, IC<1>{});
            else k_loop(IC<3>{}, IC<1>{});
        } else {
            if (mta == MT) k_loop(IC<MT>{}, IC<0>{});
            else if (mta == 0) k_loop(IC<0>{}, IC<0>{});
            else if (mta == 1) k_loop(IC<1>{}, IC<0>{});
            else if (mta == 2) k_loop(IC<2>{}, IC<0>{});
            else k_loop(IC<3>{}, IC<0>{});
        }
        first = false;

        // Epilogue.  Lane (r, g) holds, for sub-tile (i, j), column r and rows
        // q*8 + g*4 + xr at accumulator index 4q + xr.  PASS_ROWS rows at a time go through the
        // wave's private 1 KiB LDS buffer: neighbouring lanes exchange one value so that each
        // writes two adjacent bf16, then every lane reads back 16 contiguous bytes and stores
        // them.  Stores are raw buffer stores whose out-of-range lanes are dropped by the
        // bounds check.
        {
            const uint32_t epi = (uint32_t)(EPI_OFF + wave * EPI_WAVE);
            const uint32_t prm = (uint32_t)(PARAM_OFF + parity * PARAM_SET);
            const bool odd = lane & 1;
            // The lane number as the store addresses see it is made opaque per tile: otherwise
            // the sixteen per-pass row offsets are hoisted out of the tile loop and occupy
            // registers that the K loop needs.
            int lane_e = lane;
            asm volatile("" : "+v"(lane_e));
            const __amdgpu_buffer_rsrc_t rs_out =
                __builtin_amdgcn_make_buffer_rsrc(p.out + (has_map ? (size_t)0 : (size_t)cur.m0 * p.n_out), 0, 0x7FFFFFFF, 0x00020000);
            float chs[NT];
            if (EPI != EPI_PLAIN) {
#pragma unroll
                for (int j = 0; j < NT; j++) chs[j] = __uint_as_float(lds_read4(prm + 1024u + (uint32_t)(wn * WN + j * 32 + r) * 4u));
            }
#pragma unroll
            for (int i = 0; i < MT; i++) {
#pragma unroll
                for (int ps = 0; ps < NPASS; ps++) {
#pragma unroll
                    for (int qq = 0; qq < PASS_ROWS / 8; qq++) {
                        const int q = ps * (PASS_ROWS / 8) + qq;
                        float tok[4];
                        if (EPI != EPI_PLAIN) {
                            const v4i tv = lds_read16(prm + (uint32_t)(wm * WM + i * 32 + q * 8 + g * 4) * 4u);
#pragma unroll
                            for (int xr = 0; xr < 4; xr++) tok[xr] = __int_as_float(tv[xr]);
                        }
#pragma unroll
                        for (int xr = 0; xr < 4; xr += 2)
#pragma unroll
                            for (int j = 0; j < (SWIGLU ? 1 : NT); j++) {
                                const int x = q * 4 + xr;
                                float v[2];
#pragma unroll
                                for (int d = 0; d < 2; d++) {
                                    if (SWIGLU) {
                                        const float gate = (float)acc[i][0][x + d] * chs[0] * tok[xr + d];
                                        const float up = (float)acc[i][1][x + d] * chs[1] * tok[xr + d];
                                        // hardware exp2 and reciprocal: relative error ~1e-6, far inside the bf16 result
                                        v[d] = gate * __builtin_amdgcn_rcpf(1.0f + __expf(-gate)) * up;
                                    } else if (EPI == EPI_DEQUANT) {
                                        v[d] = (float)acc[i][j][x + d] * tok[xr + d] * chs[j];
                                    } else {
                                        v[d] = (float)acc[i][j][x + d];
                                    }
                                }
                                // hardware RNE to bf16, both rows in one dword; then the neighbour's dword
                                // and one byte permute: even lanes keep the low halves (row x), odd lanes
                                // the high halves (row x+1), own column in its place
                                const uint32_t pk_bf = __builtin_bit_cast(uint32_t, __builtin_convertvector((f32x2){v[0], v[1]}, bf16x2));
                                const uint32_t pk_h = __builtin_bit_cast(uint32_t, __builtin_convertvector((f32x2){v[0], v[1]}, f16x2));
                                const uint32_t pk = p.out_fp16 ? pk_h : pk_bf;   // wave-uniform choice of the output type
                                const uint32_t nb = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)pk, 0xB1, 0xF, 0xF, true);
                                const uint32_t packed = __builtin_amdgcn_perm(nb, pk, odd ? 0x03020706u : 0x05040100u);
                                const int lrow = qq * 8 + g * 4 + xr + (odd ? 1 : 0);
                                const int lcol = j * 32 + (r & ~1);
                                *reinterpret_cast<uint32_t *>(smem + epi + (uint32_t)(lrow * ROWB + lcol * 2)) = packed;
                            }
                    }
                    const int lrow = lane_e / CPR, chunk = lane_e % CPR;
                    const v4i val = lds_read16(epi + (uint32_t)(lrow * ROWB + chunk * 16));
                    const int row = wm * WM + i * 32 + ps * PASS_ROWS + lrow;  // relative to m0
                    const int col = cur.j0 + wn * WN_OUT + chunk * 8;
                    bool ok = (cur.m0 + row < cur.m_end) && (col + 8 <= p.n_out);
                    uint32_t out_row = (uint32_t)row;
                    if constexpr (EPI == EPI_PLAIN) {
                        const int mapped = (int)lds_read4(prm + (uint32_t)row * 4u);
                        ok = ok && (!has_map || (mapped >= 0 && mapped < (int)p.out_rows));   // dropped or out of range: not written
                        out_row = has_map ? (uint32_t)mapped : out_row;
                    }
                    const uint32_t off = ok ? (out_row * (uint32_t)p.n_out + (uint32_t)col) * 2u : 0xFFFFFFF0u;
                    const v4u sv = (v4u){(uint32_t)val[0], (uint32_t)val[1], (uint32_t)val[2], (uint32_t)val[3]};
                    if (p.nt_out) __builtin_amdgcn_raw_buffer_store_b128(sv, rs_out, (int)off, 0, 2);   // non-temporal
                    else __builtin_amdgcn_raw_buffer_store_b128(sv, rs_out, (int)off, 0, 0);
                }
            }
        }
        cur = nxt;
        gbase = nbase;
        t += nwg;
        parity ^= 1;
    }
}

template <int KIND, int EPI, int FMT, int TB>
static int launch_tile_t(const GemmProblem &p, hipStream_t stream)
{
    // the LDS size attribute is set once per device and kernel; setting it twice from two threads is harmless
    static std::atomic<uint64_t> attr_set{0};
    auto kern = gemm_tile_kernel<KIND, EPI, FMT, TB>;
    int dev = 0, cus = 0;
    CCH_HIP(hipGetDevice(&dev));
    const uint64_t dev_bit = (uint64_t)1 << (dev & 63);
    if (dev >= 64 || !(attr_set.load(std::memory_order_acquire) & dev_bit)) {
        CCH_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, LDS_BYTES));
        attr_set.fetch_or(dev_bit, std::memory_order_release);
    }
    CCH_HIP(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev));
    constexpr int bn_out = EPI == EPI_DEQUANT_SWIGLU ? BN / 2 : BN;
    const int64_t row_tiles = (p.T + BM - 1) / BM + (p.group_sizes ? p.num_groups : 0);  // upper bound
    const int64_t tiles = row_tiles * ((p.n_out + bn_out - 1) / bn_out);
    const unsigned grid = (unsigned)std::max<int64_t>(1, std::min<int64_t>(tiles, cus));
    hipLaunchKernelGGL(kern, dim3(grid), dim3(TILE_THREADS), LDS_BYTES, stream, p);
    return launch_status("gemm_tile_kernel");
}

// nullptr when the tiled kernels take this problem; otherwise the precondition that failed (the
// caller then uses the generic path or reports it).
const char *gemm_tile_unsupported(const GemmProblem &p, int kind, int epi)
{
    const int epb = kind == KIND_F4 ? 2 : 1;
    if (p.K < 2 * BKB * epb || p.K % (BKB * epb) != 0) return "K must be a whole number of 128-byte steps, at least two";
    if (p.n_out % 8 != 0 || !aligned(p.out, 16)) return "output rows must take 16-byte stores (n_out % 8 == 0, out 16-byte aligned)";
    if ((int64_t)BM * p.n_out * 2 >= ((int64_t)1 << 31)) return "output row tile beyond 2 GiB";
    // mapped output rows are addressed from the start of `out` with 32-bit offsets
    if (p.out_row_map && (epi != EPI_PLAIN || p.out_rows * p.n_out * 2 >= ((int64_t)1 << 31) || !aligned(p.out_row_map, 4)))
        return "mapped output beyond 2 GiB or misaligned row map";
    if (p.num_groups > MAX_GROUPS) return "more than 256 groups";
    if ((int64_t)p.N * (p.K / epb) >= ((int64_t)1 << 31)) return "one right-hand operand beyond 2 GiB (32-bit source offsets)";
    if (!aligned(p.a, 16) || !aligned(p.b, 16) || p.b_stride % 16 != 0) return "operands must be 16-byte aligned";
    if (kind != KIND_I8 && (!aligned(p.sa, 4) || !aligned(p.sb, 4) || p.sb_stride % 4 != 0 || p.sld % 4 != 0))
        return "scale arrays must be 4-byte aligned with a row length that is a multiple of 4";
    if (!p.trans_b) {
        // [K, N] operands: 16-byte pieces of a row of B must not straddle its end
        const int cpc = 16 * epb;  // columns per 16-byte piece
        if ((epi == EPI_DEQUANT_SWIGLU ? p.n_out : p.N) % cpc != 0 || (epi == EPI_DEQUANT_SWIGLU ? p.n_out : p.N) < cpc)
            return "[K,N] operands need N to be a multiple of 16 bytes";
        if (kind != KIND_I8 && p.K % 64 != 0) return "[K,N] MX operands need K % 64 == 0";
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
    return fail(CCH_ENOSUP, "no tiled GEMM kernel for kind %d with epilogue %d, trans_b %d", kind, epi, p.trans_b);
}

}  // namespace cch
