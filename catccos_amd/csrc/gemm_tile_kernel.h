// Tiled MFMA GEMM family for gfx950 (kernel template; the translation units gemm_tile_*.hip instantiate it):
//   int8 x int8 -> int32   v_mfma_i32_32x32x32_i8          + dequant / dequant+SwiGLU epilogue
//   MXFP8 / MXFP4          v_mfma_scale_f32_32x32x64_f8f6f4 with per-lane E8M0 scale operands
//
// One persistent workgroup (8 waves) per CU walks a global list of output tiles, up to 256 rows x 256 columns
// each, built from the prefix sums of the group sizes (a dense problem is one group).
//   * K advances in steps of 128 bytes per row, the size of an L2 line.  The A and B panels of a
//     step (256 rows x 128 B each) go global -> LDS without a VGPR round trip (buffer_load ... lds)
//     into a ring of two stages.
//   * The eight waves form two groups of four, one wave of each group per SIMD; each wave owns 128 x 64
//     outputs as four row blocks of 32 rows by two column blocks.  The row blocks of the two groups are
//     interleaved: group w (0: waves 0-3, 1: waves 4-7) owns tile rows 64*i + 32*w .. +31, i = 0..3, so a tile
//     that holds R rows leaves both groups ceil(R/64) (or one fewer) blocks of matrix work, and the K loop is
//     instantiated on that count: a short tile costs matrix instructions and fragment reads in proportion to
//     its rows.  In LDS a group's 128 rows stay contiguous (panel position p = 128*w + 32*i + r holds tile row
//     64*i + 32*w + r); only the global side of the requests and of the stores knows the interleaving.
//   * A wave alternates between a memory slot (LDS fragment reads, global -> LDS requests) and a
//     matrix slot (MFMAs only), the slots are separated by workgroup barriers, and the second
//     group runs one slot behind the first: while one wave of a SIMD issues matrix instructions
//     its neighbour fetches, and the next slot they swap.  A K-step is four slots per wave.  A wave issues in
//     order: a matrix slot holds nothing that can wait (no LDS read, no wait for data), and what it prepares for
//     the coming slots sits between its first matrix instructions, so that the wave is at the slot's barrier
//     before the matrix pipe falls free and the other group's first instruction finds it so.
//     B stored [K, N] (a step's panel is 128 K-rows, so its two 64-byte halves of K are separate rows):
//       L0  read the first half of the step: B fragments and the A fragments of the wave's row blocks;
//           request the second-half K-rows of B of step k+1
//       C0  MFMAs of the first half (all row blocks)
//       L1  read the second half into the same registers; request the first-half K-rows of B of step k+2
//           (the other group read them one slot ago) and the scales
//       C1  MFMAs of the second half; request this group's A rows of step k+2 between them
//     so both memory slots read the same amount (48 KiB per group) and fit under a matrix slot, and a
//     request has four to six slots to land.  B stored [N, K] (every panel row holds both halves, nothing
//     of a stage is free before both are read) splits the step by row blocks, which leaves its requests
//     more time:
//       L0  read all B fragments of the step and the A fragments of row blocks 0-1;
//           request the A rows of row blocks 2-3 of step k+1
//       C0  MFMAs of row blocks 0-1 (both 64-byte halves of the step)
//       L1  read the A fragments of row blocks 2-3 (into the same registers);
//           request B and the A rows of row blocks 0-1 of step k+2 - their place in the ring is the
//           stage being computed, whose B panel and first A rows nobody reads any more
//       C1  MFMAs of row blocks 2-3
//     (five slots, 1.25 steps, from a request to the barrier that publishes it).
//   * MX scales travel 16 bytes per row at a time (4 MXFP8 steps, 2 MXFP4 steps) into a pair of
//     scale buffers: a per-step 4-byte fetch touches one L2 line per lane and costs as many
//     line requests as the whole data panel.
//   * The K loop has no compiler-visible global loads (the requests are inline assembly tracked by
//     explicit vmcnt waits with fixed counts; a request that is not due is issued against an empty
//     buffer descriptor instead of being skipped); the last two steps of a tile are peeled and
//     request the next tile's first two steps.  K needs no particular length: the last step is
//     cut off per row (lanes past the row end fetch nothing), scale bytes past it are masked.
//   * Epilogues (dequant, SwiGLU, bf16 rounding) run on the accumulators between a wave's last
//     matrix slot of a tile and its first memory slot of the next; both groups do it in the same
//     slot.  Results pass through a wave-private 1 KiB LDS buffer so that every lane stores 16
//     contiguous bytes.
//
// Stands in for Catlass::Gemm::Block::BlockMmadTla<MmadMx<...>> as instantiated in
// examples/ascend950_fp4_mx_alltoallv_grouped_matmul/ascend950_fp4_mx_alltoallv_grouped_matmul_device.h:59-71,
// FixpipeBlockMmad (include/catccos/dgemm/block/block_mmad_preload_fixpipe.hpp:151-379), the
// tile loop of BlockMmadSchedulerAllToAllVAllGather
// (include/catccos/dgemm/block/block_scheduler_alltoallv_allgather.hpp:122-168) and the epilogues
// include/catccos/epilogue/block/block_epilogue_per_token_dequant[_swiglu].hpp.
#pragma once
#include <atomic>
#include <type_traits>
#include <utility>

#include "common.h"
#include "gemm_common.h"
#include "gemm_tile_shape.h"
#include "mx_formats.h"
#include "mx_quant_block.h"

namespace cch {

typedef int v2i __attribute__((ext_vector_type(2)));
typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v8i __attribute__((ext_vector_type(8)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef unsigned int v4u __attribute__((ext_vector_type(4)));
typedef unsigned int v2u __attribute__((ext_vector_type(2)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));

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
constexpr int SINK_OFF = PARAM_OFF + 2 * PARAM_SET;          // 1 KiB where requests that are not due land (zeros)
constexpr int RING_OFF = SINK_OFF + 1024;                    // NSTAGE stages of an A panel and a B panel
constexpr int RING_B_OFF = RING_OFF + NSTAGE * PANEL_BYTES;  // the ring holds the A panels of both stages, then the B panels
constexpr int LDS_BYTES = RING_OFF + NSTAGE * STAGE_BYTES;   // 157 KiB of the CU's 160 KiB (the group table is static LDS)

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

// s_waitcnt on gfx9: vmcnt in bits [3:0] and [15:14], expcnt [6:4], lgkmcnt [11:8].
#define CCH_WAIT_VM_LGKM0(n) __builtin_amdgcn_s_waitcnt(((n) & 15) | (((n) >> 4) << 14) | (7 << 4))
// vmcnt only (lgkmcnt left at its maximum of 15)
#define CCH_WAIT_VM(n) __builtin_amdgcn_s_waitcnt(((n) & 15) | (((n) >> 4) << 14) | (7 << 4) | (15 << 8))
// s_waitcnt lgkmcnt(0) only (vmcnt left at its maximum of 63)
#define CCH_WAIT_LGKM0() __builtin_amdgcn_s_waitcnt(0xC07F)

// Workgroup barrier that the compiler moves no memory access across (the intrinsic alone is not a
// memory barrier to the optimiser) and that the instruction scheduler leaves where it is.
#define CCH_BARRIER()                                  \
    do {                                               \
        __builtin_amdgcn_sched_barrier(0);             \
        asm volatile("s_barrier" ::: "memory");        \
        __builtin_amdgcn_sched_barrier(0);             \
    } while (0)

// 16 / 4 bytes per lane, global -> LDS without passing through registers, as raw buffer loads:
// the descriptor holds the wave-uniform base, `voff` is the per-lane byte offset, `soff` a
// wave-uniform byte offset (the K position).  Lane l of the wave lands at LDS address
// lds_addr + size*l.  A lane whose offset lies at or past the descriptor's size fetches nothing
// and receives zeros.  Issued as inline assembly on purpose: the compiler's wait-count pass
// would otherwise drain every outstanding direct-to-LDS load before each LDS read;
// completion is tracked by the explicit vmcnt waits instead.
typedef int Rsrc __attribute__((ext_vector_type(4)));
__device__ __forceinline__ Rsrc make_rsrc(const void *base, uint32_t bytes)
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
// compiler has lost track of that (the 16-byte requests of the K loop take theirs as built).
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
    soff = (uint32_t)__builtin_amdgcn_readfirstlane((int)soff);
    lds_addr = (uint32_t)__builtin_amdgcn_readfirstlane((int)lds_addr);
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
                 :
                 : "s"(lds_addr), "v"(voff), "s"(rs), "s"(soff)
                 : "memory", "m0");
}
// The same with the LDS address given as a scalar base plus a compile-time displacement (one scalar add
// straight into M0).
template <int DISP>
__device__ __forceinline__ void load16_to_lds_at(Rsrc rs, uint32_t voff, uint32_t soff, uint32_t lds_sbase)
{
    soff = (uint32_t)__builtin_amdgcn_readfirstlane((int)soff);
    lds_sbase = (uint32_t)__builtin_amdgcn_readfirstlane((int)lds_sbase);
    asm volatile("s_add_u32 m0, %0, %4\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
                 :
                 : "s"(lds_sbase), "v"(voff), "s"(rs), "s"(soff), "i"(DISP)
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
// The same reads from an absolute LDS address (a base that already holds the segment's start plus a
// compile-time displacement, which becomes the instruction's offset field).
__device__ __forceinline__ v4i lds_read16_abs(uint32_t addr)
{
    return *reinterpret_cast<const __attribute__((address_space(3))) v4i *>((uintptr_t)addr);
}
__device__ __forceinline__ uint32_t lds_read4_abs(uint32_t addr)
{
    return *reinterpret_cast<const __attribute__((address_space(3))) uint32_t *>((uintptr_t)addr);
}

// Tile row held at panel position p of the A panel (and of everything staged per row: scales, per-token
// factors, destination rows): position 128*w + 32*i + r is row block i of wave group w, tile row 64*i + 32*w + r.
__device__ __forceinline__ int tile_row_of(int p) { return ((p & 0x60) << 1) | ((p & 0x80) >> 2) | (p & 31); }

// Panel layout: row pitch 128 B; 16-byte chunk c of row `row` sits at chunk position
// c ^ ((row >> 1) & 7), which spreads 16 consecutive rows over all 64 banks for 16-byte reads.
__device__ __forceinline__ uint32_t swizzle_of_row(int row) { return (uint32_t)((row >> 1) & 7); }

// Measurement builds of this file (never the shipped library; results are wrong or slower):
//   -DCCH_PROF       every wave counts the shader cycles it spends in each wait and barrier of the
//                    K loop, and the first wave of either group notes for each of its tiles the tile's
//                    number, rows and group and the clock at the start and the end of the K loop and at
//                    the end of the epilogue; cch_prof_read() / cch_prof_read_tiles() copy them out;
//   -DCCH_V_NOLOAD   no panel requests: matrix instructions and LDS reads alone (the MFMA-side ceiling);
//   -DCCH_V_NOMFMA   no matrix instructions after a tile's first step: requests, LDS reads, waits and
//                    barriers alone (the memory-side ceiling).
// `python -m catccos_amd.build --only lib --define NAME --out DIR` builds one.
#ifdef CCH_PROF
constexpr int PROF_TILES = 12;   // tiles noted per workgroup and wave group
// (device symbols are private to a translation unit: each keeps its own counters, and a launch leaves behind the
// function that copies out the counters of the unit whose kernel ran)
namespace {
__device__ uint64_t cch_prof[256 * 8 * 8];
__device__ uint64_t cch_prof_tiles[256 * 2 * PROF_TILES * 6];
__device__ uint64_t cch_prof_entry[256 * 8];   // per workgroup: clock at entry, after the group table, before the first decode, after it, after the first requests, at the first step
int prof_copy(uint64_t *host, int tiles)
{
    if (tiles == 2) return (int)hipMemcpyFromSymbol(host, HIP_SYMBOL(cch_prof_entry), sizeof(uint64_t) * 256 * 8);
    return tiles ? (int)hipMemcpyFromSymbol(host, HIP_SYMBOL(cch_prof_tiles), sizeof(uint64_t) * 256 * 2 * PROF_TILES * 6)
                 : (int)hipMemcpyFromSymbol(host, HIP_SYMBOL(cch_prof), sizeof(uint64_t) * 256 * 8 * 8);
}
}  // namespace
extern int (*g_prof_copy)(uint64_t *, int);
#define PROF_BEGIN(t) const uint64_t t = __builtin_readcyclecounter()
#define PROF_END(t, acc) acc += __builtin_readcyclecounter() - t
#else
#define PROF_BEGIN(t)
#define PROF_END(t, acc)
#endif

constexpr uint32_t NO_FETCH = 0xFFFFFFF0u;   // a lane offset past every descriptor: the lane fetches nothing

// Inclusive prefix sum over the 64 lanes of a wave with saturating unsigned adds (associative, and exact
// while no partial sum passes 2^32 - 1): four shifts inside each row of 16 lanes, then the last lane of row 0
// into row 1 and of row 2 into row 3, then the last lane of row 1 into rows 2 and 3 (data-parallel
// primitives of gfx9: no trip through LDS).
__device__ __forceinline__ uint32_t sat_add(uint32_t a, uint32_t b) { const uint32_t s = a + b; return s < a ? 0xFFFFFFFFu : s; }
__device__ __forceinline__ uint32_t wave_scan_sat(uint32_t v)
{
    v = sat_add(v, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x111, 0xF, 0xF, true));   // row_shr:1
    v = sat_add(v, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x112, 0xF, 0xF, true));   // row_shr:2
    v = sat_add(v, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x114, 0xF, 0xF, true));   // row_shr:4
    v = sat_add(v, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x118, 0xF, 0xF, true));   // row_shr:8
    v = sat_add(v, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x142, 0xA, 0xF, false));  // row_bcast:15 into rows 1 and 3
    v = sat_add(v, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x143, 0xC, 0xF, false));  // row_bcast:31 into rows 2 and 3
    return v;
}

// The group table (row ranges and row-tile prefix sums, gemm_common.h) built by one wave (all 64 lanes of the
// caller's first wave): lane l holds groups l, 64 + l, 128 + l, 192 + l.  The running row after group g is
// min(T, sum of the non-negative sizes so far): once the rows are used up every later group is empty, before
// that nothing is clipped (the reference's golden zero-pads the remainder,
// examples/utils/gen_data_fp4_mx_alltoallv_gmm.py:788-790).
__device__ inline void build_group_table_dpp(GroupTable &tab, const int32_t *group_sizes, int num_groups, int T)
{
    constexpr int NB = MAX_GROUPS / 64;
    const int lane = threadIdx.x & 63;
    const int nb = (num_groups + 63) >> 6;   // batches of 64 groups in use (wave-uniform)
    uint32_t sz[NB];
#pragma unroll
    for (int b = 0; b < NB; b++) {
        const int g = b * 64 + lane;
        sz[b] = 0;
        if (b < nb && g < num_groups) sz[b] = group_sizes ? (uint32_t)min(max(group_sizes[g], 0), T) : (uint32_t)T;
    }
    uint32_t raw_before = 0;   // saturating sum of the sizes of the groups before this batch
    int tile_before = 0;
#pragma unroll
    for (int b = 0; b < NB; b++) {
        if (b < nb) {
            const int g = b * 64 + lane;
            const uint32_t incl = sat_add(raw_before, wave_scan_sat(sz[b]));
            const int row_hi = (int)min(incl, (uint32_t)T);
            // (the exclusive sum is the neighbour's inclusive one: incl - sz would be wrong once the sum has saturated)
            const uint32_t prev = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)incl, 0x138, 0xF, 0xF, false);   // wave_shr:1
            const int row_lo = lane == 0 ? (int)min(raw_before, (uint32_t)T) : (int)min(prev, (uint32_t)T);
            const int tiles = (row_hi - row_lo + BM - 1) / BM;
            const int tincl = (int)wave_scan_sat((uint32_t)tiles);
            if (g < num_groups) {
                tab.row_start[g] = row_lo;
                tab.tile_start[g] = tile_before + tincl - tiles;
            }
            raw_before = (uint32_t)__builtin_amdgcn_readlane((int)incl, 63);
            tile_before += __builtin_amdgcn_readlane(tincl, 63);
        }
    }
    if (lane == 0) {
        const int row = (int)min(raw_before, (uint32_t)T);
        tab.row_start[num_groups] = row;   // pseudo group: rows that belong to no expert
        tab.tile_start[num_groups] = tile_before;
        tab.row_start[num_groups + 1] = T;
        tab.tile_start[num_groups + 1] = tile_before + (T - row + BM - 1) / BM;
    }
}

// What one tile needs, all wave-uniform except the per-lane source offsets.
struct TileCtx {
    int valid, e, m0, rows, j0;         // group, first row, rows of the tile that exist (1..256), first output column
    Rsrc rs_a, rs_b, rs_sc;             // buffer descriptors: A rows from m0, B of the expert from the tile's first column, scales
    uint32_t off_sc;                    // per lane: byte offset of its scale row (A rows for waves 0-3, B columns for 4-7), rounded down to 4
    uint32_t sel_a, sel_b;              // per lane: byte selectors that bring this lane's two scale bytes of a step to bytes 0 and 2
};

// TB = 1: B is stored [N, K] (K contiguous) and its panel is staged like A's.  TB = 0 (int8 and
// MXFP8): B is stored [K, N]; a step's panel is staged as 128 K-rows of 256 bytes and the MFMA
// operand, which wants K-contiguous bytes per column, is read with the transposing LDS load
// ds_read_b64_tr_b8.  Inside a group of 16 lanes that load treats the lanes' addresses as 16
// row segments of 8 bytes and returns to lane j byte (j & 7) of segments (j >> 3), (j >> 3) + 2,
// ..., (j >> 3) + 14.  Lane i of a group therefore addresses K-row i/2 at columns 8*(i & 1) ..
// +7, and lane j receives 8 consecutive K bytes of column j.
// UA = 1: MX scale rows (sld bytes each) do not all start on 4-byte boundaries (sld % 4 == 2).
template <int KIND, int EPI, int FMT, int TB, int UA>
__global__ __launch_bounds__(TILE_THREADS) void gemm_tile_kernel(GemmProblem p)
{
    using KT = KindTraits<KIND>;
    using Acc = typename KT::Acc;
    constexpr bool MX = KIND != KIND_I8;
    constexpr bool SWIGLU = EPI == EPI_DEQUANT_SWIGLU || EPI == EPI_SWIGLU;
    constexpr bool DEQ = EPI == EPI_DEQUANT || EPI == EPI_DEQUANT_SWIGLU;   // per-token x per-channel scales in the epilogue
    constexpr int BN_OUT = SWIGLU ? BN / 2 : BN;   // output columns per tile
    constexpr int WN_OUT = SWIGLU ? WN / 2 : WN;   // output columns per wave
    constexpr int SCALE_DW = KT::SCALE_DW;         // scale dwords per row per step
    // MX scales travel 16 bytes per row at a time: one request per wave covers SPG steps
    constexpr int SPG = SCALE_DW > 0 ? 4 / SCALE_DW : 1;
    constexpr int CBSZ = FMT == CCH_FMT_E2M1 ? 4 : (FMT == CCH_FMT_E5M2 ? 1 : 0);
    constexpr int ROWB = WN_OUT * 2;               // epilogue staging: bytes per row
    constexpr int CPR = ROWB / 16;                 // 16-byte chunks per staged row
    constexpr int PASS_ROWS = 64 / CPR;            // rows staged per pass: 1 KiB, one read-back instruction
    constexpr int NPASS = 32 / PASS_ROWS;          // passes per 32-row MFMA tile
    // Output stores per wave and tile that the first step's request counts allow for: one per pass, always issued
    // (out-of-range lanes are dropped by the bounds check).  The MX-quantised activation issues two or three per pass
    // (payload, scale byte, padding byte); requests complete in order, so the waits that count NSTORES younger stores
    // are then merely stricter than they need to be.
    constexpr int NSTORES = MT * NPASS;
    constexpr int NPARAM = DEQ ? 2 : 1;   // epilogue parameter requests per wave and tile
    // requests per wave in the four slots of a step, split by row blocks (the split by halves of K counts its own in `step`)
    constexpr int NL0 = 2;                          // A rows of row blocks 2-3 of the next step
    constexpr int NC0 = 2;                          // A rows of row blocks 0-1 of the step after the next
    constexpr int NL1 = NJ / 2 + (MX ? 1 : 0);      // half of the B panel share, scales (or a request that fetches nothing)
    constexpr int NC1 = NJ / 2;                     // the other half of the B panel share
    // How a step's work is split over the two slot pairs (see `step`): by 64-byte halves of K for [K, N] operands, by row
    // blocks for [N, K] ones.
    constexpr bool KSPLIT = !TB;
    // MXFP4 [K, N] kernels whose scale rows all start on 4-byte boundaries read the scale dword of a step's second half
    // in the step's second memory slot (see `step`)
    constexpr bool SPLIT_SC = KIND == KIND_F4 && KSPLIT && !UA;

#ifdef CCH_PROF
    const uint64_t pf_entry = __builtin_readcyclecounter();
#endif
    __shared__ GroupTable tab;
    if (p.group_sizes == nullptr && p.num_groups == 1) {
        // a dense problem: one group of all rows, no rows past it
        if (threadIdx.x == 0) {
            const int tiles = (p.T + BM - 1) / BM;
            tab.row_start[0] = 0; tab.row_start[1] = p.T; tab.row_start[2] = p.T;
            tab.tile_start[0] = 0; tab.tile_start[1] = tiles; tab.tile_start[2] = tiles;
        }
    } else if (threadIdx.x < 64) {
        build_group_table_dpp(tab, p.group_sizes, p.num_groups, p.T);
    }
    __syncthreads();

#ifdef CCH_PROF
    const uint64_t pf_table = __builtin_readcyclecounter();
#endif
    const int lane = threadIdx.x & 63;
    const int wave = uniform(threadIdx.x >> 6);
    const int wm = wave / WAVES_N, wn = wave % WAVES_N;
    // LDS byte address of the dynamic segment, for the direct-to-LDS destinations
    const uint32_t lds_base = (uint32_t)uniform((int)(uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint8_t *)smem);
    const int r = lane & 31, g = lane >> 5;

    const int lda = p.K / KT::ELEMS_PER_BYTE;  // bytes per row of A and of B (K-contiguous)
    const int pa = p.a_pitch ? (int)p.a_pitch : lda;     // bytes between rows of A (packed rows carry their scales behind the payload)
    const int psa = p.sa_pitch ? (int)p.sa_pitch : p.sld;   // bytes between scale rows of A
    // an even number of steps per tile, so that a step's ring stage is its parity: an odd count runs one
    // more, empty step (its requests fetch nothing, its products are zero)
    const int ksteps = max(((lda + BKB - 1) / BKB + 1) & ~1, 2);
    const int n_tiles = (p.n_out + BN_OUT - 1) / BN_OUT;
    const int total_tiles = uniform(tab.tile_start[p.num_groups]) * n_tiles;  // rows past the groups are not ours

    // ---- LDS addresses of this lane's fragment reads.  Ring: stage s of the A panel at RING_OFF +
    // s * PANEL_BYTES, of the B panel at RING_B_OFF + s * PANEL_BYTES; row pitch 128 B, 16-byte chunk c
    // of row `row` at chunk position c ^ swizzle(row).  Lane (r, g) feeds K bytes [16g, 16g+16) of each
    // 32-byte half of a 64-byte substep: chunks ks*4 + g and ks*4 + 2 + g.  The stage, the row block
    // and the substep are compile-time displacements of the reads, so no address is computed in the
    // K loop.
    const uint32_t swz = swizzle_of_row(r);
    uint32_t fr_a[4], fr_b[4];
#pragma unroll
    for (int x = 0; x < 4; x++) {   // x = 2*ks + half
        const uint32_t chunk = (((uint32_t)((x >> 1) * 4 + (x & 1) * 2 + g)) ^ swz) << 4;
        fr_a[x] = lds_base + (uint32_t)RING_OFF + (uint32_t)(wm * WM + r) * BKB + chunk;
        fr_b[x] = lds_base + (uint32_t)RING_B_OFF + (uint32_t)(wn * WN + r) * BKB + chunk;
    }
    // (absolute LDS addresses, like the fragment bases)
    const uint32_t rd_sa = lds_base + (uint32_t)(wm * WM + r) * 16;
    // B scales: TB = 1 like A's, 16 bytes per column; TB = 0 eight 512-byte rows per group,
    // [K64 block][column][2]
    const uint32_t rd_sb = lds_base + (TB ? 4096u + (uint32_t)(wn * WN + r) * 16 : 4096u + (((uint32_t)(wn * WN + r) * 2) & ~3u));
    // TB = 0 fragment reads: lane (q = lane / 16, i = lane % 16) addresses K-row 16*(q/2) + i/2 of
    // the substep part and the 8-byte half (i & 1) of 16-byte chunk wn*4 + j*2 + (q & 1), whose
    // position in the row is swizzled by twice the row's low bits (i / 2): the 32 lanes of one pass
    // of the load address 8 K-rows x 2 neighbouring chunks, and chunk ^ 2*(row & 7) puts those 16
    // pieces on 16 different chunk positions of the 256-byte row, i.e. on all 64 banks once
    // For FP4 the panel has 256 K-rows of 128 bytes (two columns per byte) and the 4-bit form of
    // the load is a 16 x 16 nibble transpose: lane i addresses K-row i at 16 columns (8 bytes) and
    // lane j receives 16 consecutive K nibbles of column j; the chunk swizzle uses row bits 1..3.
    // The column block j enters the address by an exclusive or: one base per column block.
    constexpr bool FP4K = KIND == KIND_F4;
    constexpr int EPB = KT::ELEMS_PER_BYTE;
    constexpr int BROW = BN / EPB;               // bytes per K-row of the TB = 0 panel
    constexpr int BCPR = BROW / 16;              // 16-byte chunks per K-row
    constexpr int BRPI = 64 / BCPR;              // K-rows filled by one direct-to-LDS instruction
    const int tq = lane >> 4, ti = lane & 15;
    const uint32_t rd_bt = FP4K ? (uint32_t)(32 * (tq >> 1) + ti) * 128u + ((uint32_t)((wn * 2) ^ (ti >> 1)) << 4) + (uint32_t)(tq & 1) * 8u
                                : (uint32_t)(16 * (tq >> 1) + (ti >> 1)) * 256u + ((uint32_t)((wn * 4 + (tq & 1)) ^ ((ti >> 1) << 1)) << 4) +
                                      (uint32_t)(ti & 1) * 8u;
    uint32_t fr_bt[NT];
#pragma unroll
    for (int j = 0; j < NT; j++) fr_bt[j] = lds_base + (uint32_t)RING_B_OFF + (rd_bt ^ ((uint32_t)j << (FP4K ? 4 : 5)));
    // wave-uniform LDS addresses of the first panel request of this wave (stage 0)
    const uint32_t lds_req_a = lds_base + (uint32_t)RING_OFF + (uint32_t)(wm * WM + wn * 16) * BKB;
    // (K-half split, TB = 0: requests 0-1 of a wave land in the K-rows of the first 64-byte half, KiB 2*wave + j of the
    // panel, requests 2-3 in those of the second half, KiB 16 + 2*wave + j - 2)
    const uint32_t lds_req_b = lds_base + (uint32_t)RING_B_OFF + (uint32_t)(wave * (TB ? NJ : 2)) * 1024u;
    const int ldb = TB ? lda : p.N / EPB;   // bytes between consecutive rows of B as stored
    const uint32_t b_bytes = (uint32_t)min((int64_t)p.N * lda, (int64_t)0x7FFFFFFF);   // one right-hand operand
    const uint32_t b_step = (uint32_t)(BKB * EPB) * (uint32_t)ldb;                      // TB = 0: bytes of B between K-steps
    // Byte position inside its 128-byte row piece that this lane fetches in the K-contiguous panels
    // (even / odd request of a wave), for cutting the last step off at the row end.
    const int cb0 = (int)(((lane & 7) ^ (lane >> 4)) << 4), cb1 = cb0 ^ 64;
    // Rows that belong to no group are written as zeros (the reference's golden pads them,
    // examples/utils/gen_data_fp4_mx_alltoallv_gmm.py:788-790): all workgroups share the range,
    // 16 bytes per thread and pass; usually it is empty.
    const bool has_map = EPI == EPI_PLAIN && p.out_row_map != nullptr;   // rows go where the map says
    const bool mx_out = SWIGLU && p.mx_out;
    const int out_row_bytes = mx_out ? (p.mx_out_fmt == CCH_FMT_E2M1 ? p.n_out / 2 : p.n_out) : p.n_out * 2;
    if (p.group_sizes && !has_map) {
        const int first = uniform(tab.row_start[p.num_groups]);
        const size_t begin = (size_t)first * out_row_bytes / 16, end = (size_t)p.T * out_row_bytes / 16;
        v4u *o16 = reinterpret_cast<v4u *>(p.out);
        for (size_t i = begin + (size_t)blockIdx.x * TILE_THREADS + threadIdx.x; i < end; i += (size_t)gridDim.x * TILE_THREADS)
            o16[i] = (v4u){0, 0, 0, 0};
        if (mx_out) {
            // a block of zeros has the scale 2^0
            const size_t sb0 = (size_t)first * p.mx_out_sld, sb1 = (size_t)p.T * p.mx_out_sld;
            for (size_t i = sb0 + (size_t)blockIdx.x * TILE_THREADS + threadIdx.x; i < sb1; i += (size_t)gridDim.x * TILE_THREADS)
                p.out_scales[i] = 127;
        }
    }

    const int nwg = gridDim.x;

    // Per-lane source offsets of the panel requests, relative to the descriptors' starts: the same
    // for every tile.
    //   A: request q = 2*h + jj fills panel positions wm*128 + h*64 + (wn*2 + jj)*8 .. +7 (this wave
    //   fetches rows that its own group computes) from the tile rows that live there (tile_row_of);
    //   lane l lands at row l/8, chunk position l%8 and must therefore fetch chunk (l%8) ^ swizzle(row).
    //   B, TB = 1: request j fills rows (wave*NJ + j)*8 .. +7 in the same way; with SwiGLU tile row
    //   wn*64 + h*32 + c is the gate (h = 0) or up (h = 1) column j0 + wn*32 + c.
    //   B, TB = 0: request j fills K-rows (wave*NJ + j)*BRPI .. of the panel, BROW bytes each; lane l
    //   lands at row l/BCPR, chunk position l%BCPR and fetches tile chunk (l%BCPR) ^ swizzle, 16 bytes
    //   of columns; with SwiGLU chunk tc holds gate or up ((tc >> 1) & 1) columns j0 + (tc >> 2)*32 +
    //   (tc & 1)*16 .. +15.
    uint32_t off_a[NJ], off_b[NJ];
#pragma unroll
    for (int q = 0; q < NJ; q++) {
        const int row = wm * WM + (q >> 1) * 64 + (wn * 2 + (q & 1)) * 8 + (lane >> 3);
        off_a[q] = (uint32_t)tile_row_of(row) * (uint32_t)pa + ((uint32_t)(lane & 7) ^ swizzle_of_row(row)) * 16u;
        if (TB) {
            const int brow = (wave * NJ + q) * 8 + (lane >> 3);
            const uint32_t chunk = ((uint32_t)(lane & 7) ^ swizzle_of_row(brow)) * 16u;
            const int col = SWIGLU ? ((brow >> 5) & 1) * p.n_out + (brow >> 6) * 32 + (brow & 31) : brow;   // relative to j0
            off_b[q] = (uint32_t)col * (uint32_t)lda + chunk;
        } else {
            const int kr = ((q >> 1) * 16 + wave * 2 + (q & 1)) * BRPI + lane / BCPR;
            const int tc = (lane % BCPR) ^ (FP4K ? (kr >> 1) & 7 : (kr & 7) << 1);
            // relative to j0 (FP4: a chunk is 32 columns, one whole gate or up block)
            const int col = !SWIGLU ? tc * 16 * EPB : FP4K ? (tc & 1) * p.n_out + (tc >> 1) * 32 : ((tc >> 1) & 1) * p.n_out + (tc >> 2) * 32 + (tc & 1) * 16;
            off_b[q] = (uint32_t)kr * (uint32_t)ldb + (uint32_t)(col / EPB);
        }
    }

    const int nk_tile = ksteps;
#ifdef CCH_PROF
    uint64_t pf_wa = 0, pf_wb = 0, pf_b0 = 0, pf_b1 = 0, pf_b2 = 0, pf_b3 = 0, pf_l0 = 0;
    uint64_t pf_dec = 0;   // clocks in the decode of the next tile
    int pf_nt = 0;
    const uint64_t pf_start = __builtin_readcyclecounter();
#endif
    int gi = 0;           // scale groups requested so far; group n lives in scale buffer n & 1
    int gbase = 0;        // value of gi when the current tile's group 0 was requested

    auto decode = [&](int t, TileCtx &c) {
        // A tile index past the end decodes to the last tile with empty descriptors: its requests
        // can then be issued unconditionally (they read nothing and write zeros into LDS areas
        // that are never used), which keeps the peeled steps free of branches.
        // Workgroup w takes, in round j, place pi(w) of the round's nwg tiles.  The list of tiles is in group order, a
        // group's short last row tile right behind its whole ones: tiles that stream the same weights run side by side.
        const int G = nwg, j = t / G, w = t - j * G;
        const bool whole_round = t < total_tiles - total_tiles % G;   // the last, partial round stays row-major
        int place = w;
        if (whole_round && p.tile_order == 2 && G == 256 && (n_tiles == 8 || n_tiles == 16 || n_tiles == 32 || n_tiles == 64)) {
            // Workgroup w of a round runs on XCD w % 8.  Each XCD takes a block of 4 row tiles x 8
            // column tiles of the round (256 / n_tiles row tiles by n_tiles column tiles): a weight
            // panel then has up to four users in one L2 and a token panel eight.
            const int x = w & 7, i = w >> 3, lcb = __builtin_ctz(n_tiles >> 3);   // 1, 2, 4 or 8 blocks of 8 column tiles
            place = ((x >> lcb) * 4 + (i >> 3)) * n_tiles + (x & ((1 << lcb) - 1)) * 8 + (i & 7);
        } else if (whole_round && (p.tile_order == 1 || (p.tile_order == 2 && p.group_sizes != nullptr && p.num_groups > 1)) && (G & 7) == 0) {
            // Each XCD takes a run of nwg / 8 consecutive tiles of the round (whole row tiles next
            // to each other), so that its L2 fetches one or two A panels and the B panels of one or
            // two experts per round.
            place = (w & 7) * (G >> 3) + (w >> 3);
        }
        t = j * G + place;
        c.valid = t < total_tiles;
        const uint32_t lim = c.valid ? 0x7FFFFFFFu : 0u;
        t = max(min(t, total_tiles - 1), 0);
        const int tr = t / n_tiles, nt = t - tr * n_tiles;
        c.e = uniform(find_group(tab, p.num_groups, tr));
        c.m0 = uniform(tab.row_start[c.e] + (tr - tab.tile_start[c.e]) * BM);
        c.rows = uniform(max(min(tab.row_start[c.e + 1] - c.m0, BM), 1));   // (no tile at all: a placeholder for requests that fetch nothing)
        c.j0 = nt * BN_OUT;
        // A's descriptor starts at the tile's first row and ends with the group: requests for tile
        // rows past it are dropped by the bounds check (LDS receives zeros), and their products land
        // in accumulators that are never stored.  B's descriptor starts at the tile's first column
        // (TB = 1: row j0 of the expert's [N, K]; TB = 0: column j0 of its [K, N]) and ends with the
        // expert's operand: what a request finds past the tile's last valid column - other columns'
        // or the next expert's bytes, or nothing past the end - feeds columns that are never stored.
        // (with a pitch the last row ends lda bytes into its slot)
        c.rs_a = make_rsrc(p.a + (size_t)c.m0 * pa, min((uint32_t)(c.rows - 1) * (uint32_t)pa + (uint32_t)lda, lim));
        const uint32_t b_first = TB ? (uint32_t)c.j0 * (uint32_t)lda : (uint32_t)(c.j0 / EPB);
        c.rs_b = make_rsrc(p.b + (size_t)c.e * p.b_stride + b_first, min(b_bytes - min(b_first, b_bytes), lim));
        if (MX) {
            // Scale rows are sld bytes long, an even number that need not be a multiple of 4, while the
            // 16-byte fetches must start on 4-byte boundaries: a row that starts 2 bytes past one is
            // fetched from 2 bytes earlier and the reader shifts (ph_a, ph_b).  The descriptors
            // therefore start at the (aligned) beginning of the whole scale array.
            const int idx = (wave & 3) * 64 + lane;
            if (wave < 4) {
                c.rs_sc = make_rsrc(p.sa, (uint32_t)min((int64_t)(p.T - 1) * psa + p.sld, (int64_t)lim));
                c.off_sc = ((uint32_t)(c.m0 + min(tile_row_of(idx), c.rows - 1)) * (uint32_t)psa) & ~3u;
            } else if (TB) {
                c.rs_sc = make_rsrc(p.sb, (uint32_t)min((int64_t)p.num_groups * p.N * p.sld, (int64_t)lim));
                // (SwiGLU: tile column w*64 + h*32 + c is gate (h = 0) or up (h = 1) column j0 + w*32 + c)
                const int col = SWIGLU ? ((idx >> 5) & 1) * p.n_out + min(c.j0 + (idx >> 6) * 32 + (idx & 31), p.n_out - 1) : min(c.j0 + idx, p.N - 1);
                c.off_sc = ((uint32_t)(c.e * p.N + col) * (uint32_t)p.sld) & ~3u;
            } else {
                // [K/64][N][2]: a scale group is 8 rows of K64 blocks (4 MXFP8 steps, 2 MXFP4 steps)
                // x 256 columns x 2 bytes; wave 4+i fetches rows 2i, 2i+1, lane l 16 bytes of row l/32
                c.rs_sc = make_rsrc(p.sb + (size_t)c.e * p.sb_stride, (uint32_t)min((int64_t)p.N * p.sld, (int64_t)lim));
                // (SwiGLU: the lane's 8 tile columns lie inside one gate or up block of 32)
                const int tcol = (lane & 31) * 8;
                const int col = SWIGLU ? ((tcol >> 5) & 1) * p.n_out + c.j0 + (tcol >> 6) * 32 + (tcol & 31) : c.j0 + tcol;
                c.off_sc = (uint32_t)((lane >> 5) + 2 * (wave - 4)) * (uint32_t)p.N * 2u + (uint32_t)col * 2u;
            }
            // Rows 64*s + 32*wm + r of A and columns j0 + wn*64 + s*32 + r of B: only r, m0, j0 and the
            // expert decide by how many bytes (0 or 2) a scale row starts past a 4-byte boundary (the
            // other terms are multiples of 4 rows).  The reader holds the 8 bytes from the fetched
            // dword of a step on (lo, hi); lane group g wants the step's bytes g and 2 + g in bytes 0
            // and 2 of one register (the matrix instruction picks either with its byte selector).
            const uint32_t ph_a = ((uint32_t)(c.m0 + r) * (uint32_t)psa) & 3u;
            const uint32_t ph_b = ((uint32_t)(c.e * p.N + c.j0 + r) * (uint32_t)p.sld) & 3u;
            c.sel_a = 0x0c000c00u | (ph_a + g) | ((ph_a + g + 2) << 16);
            // TB = 0: lo / hi are the dwords of K64 rows 2x and 2x+1, two columns of two bytes each
            c.sel_b = TB ? 0x0c000c00u | (ph_b + g) | ((ph_b + g + 2) << 16)
                         : 0x0c000c00u | (uint32_t)((r & 1) * 2 + g) | ((uint32_t)(4 + (r & 1) * 2 + g) << 16);
        }
    };

    // ---- requests.  Panel requests of K-step `kstep` (byte offset kstep*128 in a row) into ring stage
    // STG.  Lanes whose 16 bytes start at or past the end of the row fetch nothing (LDS gets zeros):
    // `tail` holds what is left of the row from the step's start, worked out once per pair of requests.
    struct Tail {
        int koff;
        bool ok0, ok1;   // per lane: even / odd requests of this wave fetch
    };
    auto tail_of = [&](int kstep) {
        // (the K position is made opaque: for the fixed steps of the peeled requests the lane offsets
        // would otherwise be worked out once and held in registers through the whole kernel)
        Tail tl;
        tl.koff = kstep * BKB;
        asm volatile("" : "+s"(tl.koff));
        const int rem = lda - tl.koff;
        tl.ok0 = cb0 < rem;
        tl.ok1 = cb1 < rem;
        return tl;
    };
    auto issue_a = [&](const TileCtx &c, const Tail &tl, auto stg_c, auto q_c) {
        constexpr int q = decltype(q_c)::value, STG = decltype(stg_c)::value;
#ifdef CCH_V_NOLOAD
        return;
#endif
        const uint32_t voff = ((q & 1) ? tl.ok1 : tl.ok0) ? off_a[q] : NO_FETCH;
        load16_to_lds_at<STG * PANEL_BYTES + ((q >> 1) * 64 + (q & 1) * 8) * BKB>(c.rs_a, voff, (uint32_t)tl.koff, lds_req_a);
    };
    // TB = 0: the K position of a request is part of the lane offset, which the bounds check covers:
    // K-rows past the operand's last one lie past its descriptor
    auto issue_b = [&](const TileCtx &c, const Tail &tl, uint32_t boff, auto stg_c, auto j_c) {
        constexpr int j = decltype(j_c)::value, STG = decltype(stg_c)::value;
#ifdef CCH_V_NOLOAD
        return;
#endif
        if constexpr (TB) {
            const uint32_t voff = ((j & 1) ? tl.ok1 : tl.ok0) ? off_b[j] : NO_FETCH;
            load16_to_lds_at<STG * PANEL_BYTES + j * 1024>(c.rs_b, voff, (uint32_t)tl.koff, lds_req_b);
        } else {
            load16_to_lds_at<STG * PANEL_BYTES + ((j >> 1) * 16 + (j & 1)) * 1024>(c.rs_b, off_b[j] + boff, 0u, lds_req_b);
        }
    };
    auto boff_of = [&](int kstep) {
        uint32_t boff = (uint32_t)kstep * b_step;
        asm volatile("" : "+s"(boff));
        return boff;
    };
    // A scale request as the matrix slot before it prepared it: descriptor (empty when no group is due:
    // the request is issued all the same, so that the number of requests in flight never depends on
    // the step), lane offset, LDS destination.
    struct ScaleReq {
        Rsrc rs;
        uint32_t voff, dst;
    };
    // Scale group `grp` of tile c (steps grp*SPG .. grp*SPG+SPG-1) into the next scale buffer: waves
    // 0-3 fetch 16 bytes of each A row, one row per lane; waves 4-7 the same for the B rows
    // (TB = 1) or 1 KiB each of the group's eight [column][2] rows (TB = 0).
    auto prep_scales = [&](int due, const TileCtx &c, int grp) {
        ScaleReq rq;
        due = uniform(due);
        rq.rs = c.rs_sc;
        rq.rs[2] = due ? rq.rs[2] : 0;
        rq.voff = c.off_sc + ((TB || wave < 4) ? (uint32_t)grp * 16u : (uint32_t)grp * 16u * (uint32_t)p.N);   // TB = 0: 8 rows of 2N bytes
        rq.dst = lds_base + (due ? (uint32_t)(SCALE_OFF + (gi & 1) * SCALE_BUF) + (uint32_t)(wave >= 4) * 4096u + (uint32_t)(wave & 3) * 1024u
                                 : (uint32_t)SINK_OFF);
        gi += due;
        return rq;
    };
    auto issue_scales = [&](const ScaleReq &rq) {
#ifdef CCH_V_NOLOAD
        return;
#endif
        if constexpr (MX) load16_to_lds(rq.rs, rq.voff, 0u, rq.dst);
    };
    // Epilogue parameters of a tile (per-token / per-channel scales, or the destination rows).
    auto issue_params = [&](const TileCtx &c, int parity) {
        const uint32_t lim = c.valid ? 0x7FFFFFFFu : 0u;
        const int idx = (wave & 3) * 64 + lane;
        // destination of lane 0 of this wave; lane l lands 4*l bytes further
        const uint32_t dst = lds_base + (uint32_t)(PARAM_OFF + parity * PARAM_SET) + (uint32_t)(wave & 3) * 256u;
        if (DEQ) {
            load4_to_lds(make_rsrc(p.per_tok + c.m0, min((uint32_t)(p.T - c.m0) * 4u, lim)), (uint32_t)min(tile_row_of(idx), c.rows - 1) * 4u, 0u, dst);
            int col;
            if (SWIGLU) col = ((idx >> 5) & 1) * p.n_out + min(c.j0 + (idx >> 6) * 32 + (idx & 31), p.n_out - 1);
            else col = min(c.j0 + idx, p.N - 1);
            load4_to_lds(make_rsrc(p.per_ch + (size_t)c.e * p.N, min((uint32_t)p.N * 4u, lim)), (uint32_t)col * 4u, 0u, dst + 1024u);
        } else {
            // destination rows of the tile's 256 rows, where the per-token scales of the other
            // epilogues go; without a map the descriptor is empty and nothing is fetched
            load4_to_lds(make_rsrc(p.out_row_map + c.m0, has_map ? min((uint32_t)(p.T - c.m0) * 4u, lim) : 0u),
                         (uint32_t)min(tile_row_of(idx), c.rows - 1) * 4u, 0u, dst);
        }
    };

    // LDS addresses of this lane's scale reads of the coming step (prepared in the matrix slot before
    // its first memory slot): low dword for the A rows and the B columns, and - when rows can start 2
    // bytes past a 4-byte boundary - the dword after the step's last one, which for the last dword of
    // a group's 16 bytes is the first of the next group's.
    uint32_t va_sa = 0, va_sb = 0, va_sa_hi = 0, va_sb_hi = 0;
    // for the first step of a tile whose group 0 is in the buffer of parity gb & 1
    auto prep_scale_reads = [&](int gb) {
        if constexpr (MX) {
            const uint32_t bufc = (uint32_t)(SCALE_OFF + (gb & 1) * SCALE_BUF), bufn = (uint32_t)(SCALE_OFF + ((gb + 1) & 1) * SCALE_BUF);
            va_sa = rd_sa + bufc;
            va_sb = rd_sb + bufc;
            if constexpr (UA) {
                va_sa_hi = rd_sa + (SPG == 1 ? bufn : bufc + (uint32_t)SCALE_DW * 4u);
                va_sb_hi = rd_sb + (SPG == 1 ? bufn : bufc + (uint32_t)SCALE_DW * 4u);
            }
            asm volatile("" : "+v"(va_sa), "+v"(va_sb));
            if constexpr (UA) asm volatile("" : "+v"(va_sa_hi), "+v"(va_sb_hi));
        }
    };
    // from step kt to step kt + 1 of the same tile: a few bytes on, or to the start of the other
    // buffer when the next step opens a group (the addresses move by wave-uniform amounts)
    auto advance_scale_reads = [&](int gb, int kt) {
        if constexpr (MX) {
            const int grp = kt / SPG, ws = kt - grp * SPG;                          // this step's group and place in it
            const int to_other = ((gb + grp) & 1) ? -SCALE_BUF : SCALE_BUF;          // from this group's buffer to the next group's
            const bool opens = ws == SPG - 1;                                       // the next step opens a group
            const int step_a = SCALE_DW * 4, step_b = TB ? SCALE_DW * 4 : 2 * SCALE_DW * 512;
            int da = opens ? to_other - ws * step_a : step_a;
            int db = opens ? to_other - ws * step_b : step_b;
            asm volatile("" : "+s"(da), "+s"(db));
            va_sa += (uint32_t)da;
            va_sb += (uint32_t)db;
            if constexpr (UA) {
                // the dword after the next step's last one: the first of the buffer after its own when
                // that step closes its group
                const int ws1 = opens ? 0 : ws + 1;
                int dh = ws1 == SPG - 1 ? (opens ? -to_other : to_other) - ws1 * step_a : step_a;
                asm volatile("" : "+s"(dh));
                va_sa_hi = va_sa + (uint32_t)dh;
                va_sb_hi = va_sb + (uint32_t)dh;
            }
            asm volatile("" : "+v"(va_sa), "+v"(va_sb));
            if constexpr (UA) asm volatile("" : "+v"(va_sa_hi), "+v"(va_sb_hi));
        }
    };

    TileCtx cur, nxt;
    int t = (int)blockIdx.x, parity = 0;
#ifdef CCH_PROF
    const uint64_t pf_setup = __builtin_readcyclecounter();
#endif
    decode(t, cur);
#ifdef CCH_PROF
    const uint64_t pf_decoded = __builtin_readcyclecounter();
    uint64_t pf_issued = 0;
#endif
    nxt = cur;
    nxt.valid = 0;
    const bool any = cur.valid;
    if (any) {
        // Everything the first tile's step 0 and step 1 need, except the last A rows of step 1 (slot
        // L0 of step 0 requests them); all of it has landed before the first step starts.
        {
            const Tail t0 = tail_of(0), t1 = tail_of(1);
            static_for<NJ>([&](auto j_c) { issue_b(cur, t0, boff_of(0), IC<0>{}, j_c); });
            static_for<NJ>([&](auto q_c) { issue_a(cur, t0, IC<0>{}, q_c); });
            issue_scales(prep_scales(1, cur, 0));
            issue_params(cur, 0);
            if constexpr (KSPLIT) {
                // (slot L0 of step 0 requests the rest of step 1's B panel)
                if constexpr (!TB) {
                    issue_b(cur, t1, boff_of(1), IC<1>{}, IC<0>{});
                    issue_b(cur, t1, boff_of(1), IC<1>{}, IC<1>{});
                }
                static_for<NJ>([&](auto q_c) { issue_a(cur, t1, IC<1>{}, q_c); });
            } else {
                static_for<NJ>([&](auto j_c) { issue_b(cur, t1, boff_of(1), IC<1>{}, j_c); });
                issue_a(cur, t1, IC<1>{}, IC<0>{});
                issue_a(cur, t1, IC<1>{}, IC<1>{});
            }
            issue_scales(prep_scales(SPG == 2 && nk_tile > 2, cur, 1));
        }
        prep_scale_reads(0);
#ifdef CCH_PROF
        pf_issued = __builtin_readcyclecounter();
#endif
        CCH_WAIT_VM_LGKM0(0);
        CCH_BARRIER();
#ifdef CCH_PROF
        if (threadIdx.x == 0 && blockIdx.x < 256) {
            uint64_t *o = cch_prof_entry + (size_t)blockIdx.x * 8;
            o[0] = pf_entry; o[1] = pf_table; o[2] = pf_setup; o[3] = pf_decoded; o[4] = pf_issued; o[5] = __builtin_readcyclecounter();
        }
#endif
        // the second group starts one slot behind the first
        if (wm == 1) CCH_BARRIER();
    }
    while (cur.valid) {
        Acc acc[MT][NT];
        int nbase = 0;  // gi when the next tile's scale group 0 is requested
        // Fragment registers of a slot pair: all B fragments of the step and the A fragments of two
        // row blocks, both 64-byte halves each.
        v8i fa[2][2], fb[NT][2];
        constexpr int NSC = SCALE_DW > 0 ? SCALE_DW : 1;
        uint32_t sc[NSC][MT + NT];  // scale dwords of the current step, this lane's two bytes in bytes 0 and 2

        auto frag_a = [&](auto stg_c, int ks, int i) {
            constexpr int STG = decltype(stg_c)::value;
            const v4i lo = lds_read16_abs(fr_a[ks * 2] + (uint32_t)(STG * PANEL_BYTES + i * 32 * BKB));
            const v4i hi = lds_read16_abs(fr_a[ks * 2 + 1] + (uint32_t)(STG * PANEL_BYTES + i * 32 * BKB));
            return (v8i){lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
        };
        auto frag_b = [&](auto stg_c, int ks, int j) {
            constexpr int STG = decltype(stg_c)::value;
            if constexpr (TB) {
                const v4i lo = lds_read16_abs(fr_b[ks * 2] + (uint32_t)(STG * PANEL_BYTES + j * 32 * BKB));
                const v4i hi = lds_read16_abs(fr_b[ks * 2 + 1] + (uint32_t)(STG * PANEL_BYTES + j * 32 * BKB));
                return (v8i){lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
            } else {
                typedef __attribute__((address_space(3))) v2i *LdsV2;
                // FP4: four nibble transposes, K elements 32g+0..15, 32g+16..31, 64+32g+0..15, 64+32g+16..31 of
                // the substep (K-rows of 128 B); else four byte transposes, K bytes 16g+0..7, 16g+8..15,
                // 32+16g+0..7, 32+16g+8..15 (K-rows of 256 B): the same byte displacements either way
                const uint32_t base = fr_bt[j] + (uint32_t)(STG * PANEL_BYTES) + (uint32_t)ks * 16384u;
                v2i t0, t1, t2, t3;
                if constexpr (FP4K) {
                    t0 = __builtin_amdgcn_ds_read_tr4_b64_v2i32((LdsV2)(uintptr_t)(base));
                    t1 = __builtin_amdgcn_ds_read_tr4_b64_v2i32((LdsV2)(uintptr_t)(base + 2048u));
                    t2 = __builtin_amdgcn_ds_read_tr4_b64_v2i32((LdsV2)(uintptr_t)(base + 8192u));
                    t3 = __builtin_amdgcn_ds_read_tr4_b64_v2i32((LdsV2)(uintptr_t)(base + 10240u));
                } else {
                    t0 = __builtin_amdgcn_ds_read_tr8_b64_v2i32((LdsV2)(uintptr_t)(base));
                    t1 = __builtin_amdgcn_ds_read_tr8_b64_v2i32((LdsV2)(uintptr_t)(base + 2048u));
                    t2 = __builtin_amdgcn_ds_read_tr8_b64_v2i32((LdsV2)(uintptr_t)(base + 8192u));
                    t3 = __builtin_amdgcn_ds_read_tr8_b64_v2i32((LdsV2)(uintptr_t)(base + 10240u));
                }
                return (v8i){t0[0], t0[1], t1[0], t1[1], t2[0], t2[1], t3[0], t3[1]};
            }
        };
        // Scale dwords of the step whose read addresses were prepared (prep_scale_reads), in two parts
        // so that the LDS reads are issued ahead of the fragment reads and the arithmetic runs while
        // those are under way.  In the last two steps of a tile the bytes of the 32-element blocks
        // that lie past K (fetched from the next row, or not at all) are cleared: their payload is
        // zero, and a zero byte (2^-127) keeps the product zero where a stray 0xFF (NaN) would not.
        // Lane group g uses byte g and byte 2 + g of a step's dword: one byte permute brings them to
        // bytes 0 and 2, where the matrix instruction's byte selector finds them.
        uint32_t raw_lo[NSC][MT + NT], raw_hi[NSC][MT + NT];
        // (d0_c .. d1_c: the dwords of the step to handle, all of them or, where the step's two halves fetch their
        // scales apart, one each)
        auto read_scales_raw = [&](auto d0_c, auto d1_c) {
            if constexpr (MX) {
#pragma unroll
                for (int d = decltype(d0_c)::value; d < decltype(d1_c)::value; d++) {
#pragma unroll
                    for (int s = 0; s < MT; s++) {
                        raw_lo[d][s] = lds_read4_abs(va_sa + d * 4 + s * 512);
                        if constexpr (UA) raw_hi[d][s] = d == SCALE_DW - 1 ? lds_read4_abs(va_sa_hi + s * 512) : lds_read4_abs(va_sa + d * 4 + 4 + s * 512);
                    }
#pragma unroll
                    for (int s = 0; s < NT; s++) {
                        if constexpr (TB) {
                            raw_lo[d][MT + s] = lds_read4_abs(va_sb + d * 4 + s * 512);
                            if constexpr (UA)
                                raw_hi[d][MT + s] = d == SCALE_DW - 1 ? lds_read4_abs(va_sb_hi + s * 512) : lds_read4_abs(va_sb + d * 4 + 4 + s * 512);
                        } else {
                            // the two K32 scales of K64 row 2x and of row 2x+1; each row holds two columns per dword
                            raw_lo[d][MT + s] = lds_read4_abs(va_sb + d * 1024 + s * 64);
                            raw_hi[d][MT + s] = lds_read4_abs(va_sb + d * 1024 + 512 + s * 64);
                        }
                    }
                }
            }
        };
        auto finish_scales = [&](auto last_c, int kt, auto d0_c, auto d1_c) {
            if constexpr (MX) {
                constexpr bool LAST = decltype(last_c)::value != 0;
                const int nblk = (p.K + 31) >> 5;
#pragma unroll
                for (int d = decltype(d0_c)::value; d < decltype(d1_c)::value; d++) {
                    uint32_t keep = 0xFFFFFFFFu;
                    if constexpr (LAST) {
                        // blocks of this dword that lie inside K; this lane's two are g and 2 + g
                        const int nb = nblk - (kt * SCALE_DW + d) * 4;
                        keep = (g < nb ? 0xFFu : 0u) | (2 + g < nb ? 0xFF0000u : 0u);
                    }
#pragma unroll
                    for (int s = 0; s < MT + NT; s++) {
                        // rows that all start on 4-byte boundaries need the low dword only
                        const bool two = UA || (!TB && s >= MT);
                        const uint32_t v = __builtin_amdgcn_perm(two ? raw_hi[d][s] : raw_lo[d][s], raw_lo[d][s], s < MT ? cur.sel_a : cur.sel_b);
                        sc[d][s] = LAST ? v & keep : v;
                    }
                }
            }
        };
        // The MFMAs of row block ai on the 64-byte substep ks: all column blocks on the low 32
        // bytes, then (int8 and FP4, which take two MFMAs per 64 bytes) all on the high 32 bytes.
        // With ZERO the accumulators start from zero instead of being read.
        // (int8 and FP4: `only_c` 0 or 1 issues the MFMAs of that 32-byte half alone, -1 both)
        auto mfma_block = [&](auto zero_c, auto ks_c, auto ai_c, const v8i &a, auto only_c) {
            constexpr int ks = decltype(ks_c)::value, ai = decltype(ai_c)::value, ONLY = decltype(only_c)::value;
#ifdef CCH_V_NOMFMA
            if (!decltype(zero_c)::value) { asm volatile("" :: "v"(a)); return; }
#endif
            constexpr bool ZERO = decltype(zero_c)::value != 0;
            constexpr int fbi = KSPLIT ? 0 : ks;   // K-half split: the B fragments of the current half sit in fb[j][0]
            if constexpr (KIND == KIND_F8) {
#pragma unroll
                for (int j = 0; j < NT; j++) {
                    Acc c;
                    if (ZERO) c = (Acc)(0.0f);
                    else c = acc[ai][j];
                    acc[ai][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a, fb[j][fbi], c, CBSZ, CBSZ, 2 * ks, (int)sc[0][ai], 2 * ks,
                                                                                 (int)sc[0][MT + j]);
                }
            } else {
#pragma unroll
                for (int half = 0; half < 2; half++)
#pragma unroll
                    for (int j = 0; j < NT; j++) {
                        if (ONLY >= 0 && half != ONLY) continue;
                        Acc c;
                        if (ZERO && half == 0) c = (Acc)(0);
                        else c = acc[ai][j];
                        if constexpr (KIND == KIND_F4) {
                            // substep = 128 elements = scale dword ks; the low MFMA uses byte g, the high one byte 2+g
                            const v8i ah = (v8i){a[4 * half], a[4 * half + 1], a[4 * half + 2], a[4 * half + 3], 0, 0, 0, 0};
                            const v8i bh = (v8i){fb[j][fbi][4 * half], fb[j][fbi][4 * half + 1], fb[j][fbi][4 * half + 2], fb[j][fbi][4 * half + 3], 0, 0, 0, 0};
                            if (half == 0)
                                acc[ai][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(ah, bh, c, 4, 4, 0, (int)sc[ks][ai], 0, (int)sc[ks][MT + j]);
                            else
                                acc[ai][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(ah, bh, c, 4, 4, 2, (int)sc[ks][ai], 2, (int)sc[ks][MT + j]);
                        } else {
                            const v4i ah = (v4i){a[4 * half], a[4 * half + 1], a[4 * half + 2], a[4 * half + 3]};
                            const v4i bh = (v4i){fb[j][fbi][4 * half], fb[j][fbi][4 * half + 1], fb[j][fbi][4 * half + 2], fb[j][fbi][4 * half + 3]};
                            acc[ai][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(ah, bh, c, 0, 0, 0);
                        }
                    }
            }
        };

        // One K-step of the current tile.  MODE 0: steady state; 1: second to last step (its requests
        // are the next tile's step 0, scales and epilogue parameters); 2: last step (requests the next
        // tile's step 0 / step 1 shares, no barrier at its end: the caller places it around the
        // epilogue).  FIRST: first step of a tile (accumulators start from zero; the previous tile's
        // output stores are among the younger requests that the waits count).  NBLK: row blocks of this
        // wave (1..4) that hold rows of the tile; the others get no fragment reads and no matrix
        // instructions.  STG: ring stage of the step (tiles have an even number of steps, so a step's
        // stage is its parity).
        // The memory slots hold nothing but LDS reads, requests and the waits: every wave-uniform
        // quantity they use is worked out in the matrix slot before them, where the wave has issue
        // cycles to spare between MFMAs.
        auto step = [&](auto mode_c, auto first_c, auto nblk_c, auto stg_c, int kt) {
            constexpr int MODE = decltype(mode_c)::value, NBLK = decltype(nblk_c)::value, STG = decltype(stg_c)::value;
            constexpr int FIRST = decltype(first_c)::value;
            // Requests that may still be in flight when a wait of this step is reached, oldest first:
            //   [L0 C0 L1 C1 of the step before] [output stores] [this L0] [this C0] [this L1]
            constexpr int STORES = FIRST ? NSTORES : 0;
            // tile and step that the requests of C0, L1 and C1 are for (two steps ahead, into this stage)
            const TileCtx &rq = MODE == 0 ? cur : nxt;
            const int rq_kt = MODE == 0 ? kt + 2 : MODE - 1;
            // The read bases are made opaque per step: base + displacement would otherwise be worked out
            // once for every displacement and held in a register each through the whole loop.
#pragma unroll
            for (int x = 0; x < 4; x++) {
                asm volatile("" : "+v"(fr_a[x]));
                if constexpr (TB) asm volatile("" : "+v"(fr_b[x]));
            }
            if constexpr (!TB) {
#pragma unroll
                for (int j = 0; j < NT; j++) asm volatile("" : "+v"(fr_bt[j]));
            }
            // Scale group n of a tile is requested three steps before its first step (a reader of the
            // group before it needs its first bytes one step early); group 0 comes with the tile's
            // first step, and MXFP4's group 1 (steps 2-3) with its second.  Prepared in C0 for L1.
            // SPLIT_SC: two steps before its first step instead, i.e. in the first step of the group before it (the
            // request lands in the buffer of the group before that one, whose second dwords the other wave group
            // still reads in the L1 of its last step, one slot after this group's; nothing is read a step early here,
            // as all scale rows start on 4-byte boundaries).  A request issued in a step's L1 has landed when the
            // next step's L1 ends, one step before the group's first L0.
            auto next_scale_request = [&]() {
                ScaleReq sreq{};
                if constexpr (MX) {
                    if constexpr (MODE == 0 && SPLIT_SC) {
                        sreq = prep_scales(((kt + 2) & (SPG - 1)) == 0 && kt >= SPG && kt + 2 < nk_tile, cur, (kt + 2) / SPG);
                    } else if constexpr (MODE == 0) {
                        sreq = prep_scales(((kt + 3) & (SPG - 1)) == 0 && kt + 3 < nk_tile, cur, (kt + 3) / SPG);
                    } else if constexpr (MODE == 1) {
                        nbase = gi;
                        sreq = prep_scales(1, nxt, 0);
                    } else {
                        sreq = prep_scales(SPG == 2 && nk_tile > 2, nxt, 1);
                    }
                    asm volatile("" : "+s"(sreq.rs), "+v"(sreq.voff), "+s"(sreq.dst));
                }
                return sreq;
            };
            if constexpr (KSPLIT) {
                // [K, N] operands: the step is split by halves of K.  L0 reads the first 64-byte half of the step (B
                // fragments and the A fragments of the wave's row blocks), C0 multiplies it, L1 reads the second half
                // into the same registers, C1 multiplies that: the two memory slots read the same amount and both fit
                // under a matrix slot.  A stage is free once both halves are read, so the requests are: L0 the
                // second-half K-rows of the next step's B panel, L1 the first-half K-rows of B two steps ahead (the
                // other group read them one slot ago) and the scales, C1 the A rows two steps ahead (a group's A rows
                // are read by that group alone).
                constexpr int NB_L0 = NJ / 2, NB_L1 = NJ / 2;
                constexpr int KL1 = NB_L1 + (MX ? 1 : 0), KC1 = NJ;
                constexpr int K_PREV_L1 = KL1 + (MODE == 2 ? NPARAM : 0), K_THIS_L1 = KL1 + (MODE == 1 ? NPARAM : 0);
                // MXFP4 has a scale dword for either half of the step: the second one is read and prepared in L1, with the
                // half it scales, so that the two memory slots stay alike (SPLIT_SC).  That read comes two slots later
                // than one in L0, which the scale requests allow for (next_scale_request); a tile's last step reads both
                // in L0, because the requests for the next tile's scales follow in its L1.
                constexpr int SC_L0 = SPLIT_SC && MODE != 2 ? 1 : SCALE_DW;
                // ------------------------------------------------------------------ L0
                read_scales_raw(IC<0>{}, IC<SC_L0>{});
#pragma unroll
                for (int j = 0; j < NT; j++) fb[j][0] = frag_b(stg_c, 0, j);
                __builtin_amdgcn_sched_barrier(0);
                finish_scales(IC<MODE != 0>{}, kt, IC<0>{}, IC<SC_L0>{});
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int i = 0; i < NBLK; i++) fa[i & 1][i >> 1] = frag_a(stg_c, 0, i);
                __builtin_amdgcn_sched_barrier(0);
                {
                    const TileCtx &nc = MODE == 2 ? nxt : cur;
                    const int nk1 = MODE == 2 ? 0 : kt + 1;
                    const Tail tl = tail_of(nk1);
                    const uint32_t nb = boff_of(nk1);
                    issue_b(nc, tl, nb, IC<STG ^ 1>{}, IC<2>{});
                    issue_b(nc, tl, nb, IC<STG ^ 1>{}, IC<3>{});
                }
                __builtin_amdgcn_sched_barrier(0);
                { PROF_BEGIN(t_); CCH_WAIT_LGKM0(); PROF_END(t_, pf_l0); }
                // the second-half K-rows of this step's B panel (requested in the previous step's L0) must have
                // landed: younger are the previous step's L1 and C1, the stores and this L0
                { PROF_BEGIN(t_); CCH_WAIT_VM(K_PREV_L1 + KC1 + STORES + NB_L0); PROF_END(t_, pf_wa); }
                { PROF_BEGIN(t_); CCH_BARRIER(); PROF_END(t_, pf_b0); }
                // ------------------------------------------------------------------ C0
                // (int8 and FP4 take two MFMAs per accumulator and half of K: all row blocks on the first 32 bytes, then
                // all on the second, so that an accumulator's two MFMAs are not neighbours in the pipe)
                // (what the coming slots need is worked out between the matrix instructions, in the issue cycles that
                // the wave has to spare while the pipe is busy: behind the last one it would hold up the barrier, and
                // with it the other group's first matrix instruction, past the moment the pipe falls free)
                Tail rq_tl{};
                uint32_t rq_boff = 0;
                ScaleReq sreq{};
                static_for<(KIND == KIND_F8 ? 1 : 2)>([&](auto h_c) {
                    static_for<NBLK>([&](auto i_c) {
                        constexpr int i = decltype(i_c)::value, h = decltype(h_c)::value;
                        mfma_block(IC<FIRST>{}, IC<0>{}, i_c, fa[i & 1][i >> 1], IC<(KIND == KIND_F8 ? -1 : h)>{});
                        if constexpr (h == 0 && i == 0) {
                            __builtin_amdgcn_sched_barrier(0);
                            rq_tl = tail_of(rq_kt);
                            rq_boff = boff_of(rq_kt);
                            __builtin_amdgcn_sched_barrier(0);
                        }
                        if constexpr (h == 0 && i == (NBLK > 1 ? 1 : 0)) {
                            __builtin_amdgcn_sched_barrier(0);
                            sreq = next_scale_request();
                            __builtin_amdgcn_sched_barrier(0);
                        }
                    });
                });
                __builtin_amdgcn_sched_barrier(0);
                { PROF_BEGIN(t_); CCH_BARRIER(); PROF_END(t_, pf_b1); }
                // ------------------------------------------------------------------ L1
                read_scales_raw(IC<SC_L0>{}, IC<SCALE_DW>{});
#pragma unroll
                for (int j = 0; j < NT; j++) fb[j][0] = frag_b(stg_c, 1, j);
                __builtin_amdgcn_sched_barrier(0);
                finish_scales(IC<MODE != 0>{}, kt, IC<SC_L0>{}, IC<SCALE_DW>{});
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int i = 0; i < NBLK; i++) fa[i & 1][i >> 1] = frag_a(stg_c, 1, i);
                __builtin_amdgcn_sched_barrier(0);
                issue_b(rq, rq_tl, rq_boff, stg_c, IC<0>{});
                issue_b(rq, rq_tl, rq_boff, stg_c, IC<1>{});
                issue_scales(sreq);
                if constexpr (MODE == 1) issue_params(nxt, parity ^ 1);
                __builtin_amdgcn_sched_barrier(0);
                // what the next step's L0 reads of B must have landed: its first-half K-rows and scales, requested in
                // the previous step's L1; younger are that step's C1, the stores and this step's L0 and L1
                { PROF_BEGIN(t_); CCH_WAIT_VM_LGKM0(KC1 + STORES + NB_L0 + K_THIS_L1); PROF_END(t_, pf_wb); }
                { PROF_BEGIN(t_); CCH_BARRIER(); PROF_END(t_, pf_b2); }
                // ------------------------------------------------------------------ C1
                // (the scale read addresses of the next step move on behind the first matrix instructions, not behind the last)
                static_for<NJ>([&](auto q_c) {
                    constexpr int q = decltype(q_c)::value;
                    if constexpr (q < NBLK) {
                        mfma_block(IC<0>{}, IC<1>{}, q_c, fa[q & 1][q >> 1], IC<(KIND == KIND_F8 ? -1 : 0)>{});
                        __builtin_amdgcn_sched_barrier(0);
                    }
                    if constexpr (q == 0) {
                        if constexpr (MODE == 2) prep_scale_reads(nbase);
                        else advance_scale_reads(gbase, kt);
                        __builtin_amdgcn_sched_barrier(0);
                    }
                    issue_a(rq, rq_tl, stg_c, q_c);
                    __builtin_amdgcn_sched_barrier(0);
                });
                if constexpr (KIND != KIND_F8) {
                    static_for<NBLK>([&](auto q_c) {
                        constexpr int q = decltype(q_c)::value;
                        mfma_block(IC<0>{}, IC<1>{}, q_c, fa[q & 1][q >> 1], IC<1>{});
                    });
                }
                __builtin_amdgcn_sched_barrier(0);
                // this group's A rows of the next step (requested in the previous step's C1) must have landed:
                // younger are the stores and this step's L0, L1 and C1
                { PROF_BEGIN(t_); CCH_WAIT_VM(STORES + NB_L0 + K_THIS_L1 + KC1); PROF_END(t_, pf_wa); }
                if constexpr (MODE != 2) { PROF_BEGIN(t_); CCH_BARRIER(); PROF_END(t_, pf_b3); }
            } else {
                // [N, K] operands: the step is split by row blocks (0-1 in the first slot pair, 2-3 in the second).
                constexpr int PREV_L1 = MODE == 2 ? NL1 + NPARAM : NL1;   // what the step before this one issued in its L1
                constexpr int THIS_L1 = MODE == 1 ? NL1 + NPARAM : NL1;
                constexpr int NB0 = NBLK < 2 ? NBLK : 2, NB1 = NBLK - NB0;   // row blocks of either slot pair
                // ------------------------------------------------------------------ L0
                read_scales_raw(IC<0>{}, IC<SCALE_DW>{});
#pragma unroll
                for (int ks = 0; ks < 2; ks++)
#pragma unroll
                    for (int j = 0; j < NT; j++) fb[j][ks] = frag_b(stg_c, ks, j);
                __builtin_amdgcn_sched_barrier(0);
                finish_scales(IC<MODE != 0>{}, kt, IC<0>{}, IC<SCALE_DW>{});   // while the B fragments arrive; its inputs die before the A fragments need registers
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int ks = 0; ks < 2; ks++)
#pragma unroll
                    for (int i = 0; i < NB0; i++) fa[i][ks] = frag_a(stg_c, ks, i);
                __builtin_amdgcn_sched_barrier(0);
                // the last A rows of the next step, into the other stage
                {
                    const Tail tl = tail_of(MODE == 2 ? 0 : kt + 1);
                    issue_a(MODE == 2 ? nxt : cur, tl, IC<STG ^ 1>{}, IC<2>{});
                    issue_a(MODE == 2 ? nxt : cur, tl, IC<STG ^ 1>{}, IC<3>{});
                }
                __builtin_amdgcn_sched_barrier(0);
                { PROF_BEGIN(t_); CCH_WAIT_LGKM0(); PROF_END(t_, pf_l0); }
                { PROF_BEGIN(t_); CCH_BARRIER(); PROF_END(t_, pf_b0); }
                // ------------------------------------------------------------------ C0
                // (the first A rows of the step after the next are requested between the MFMA blocks: their
                // place, the first rows of this stage's half, was read for the last time in L0)
                mfma_block(IC<FIRST>{}, IC<0>{}, IC<0>{}, fa[0][0], IC<-1>{});
                __builtin_amdgcn_sched_barrier(0);
                const Tail rq_tl = tail_of(rq_kt);
                issue_a(rq, rq_tl, stg_c, IC<0>{});
                __builtin_amdgcn_sched_barrier(0);
                if constexpr (NB0 > 1) mfma_block(IC<FIRST>{}, IC<0>{}, IC<1>{}, fa[1][0], IC<-1>{});
                __builtin_amdgcn_sched_barrier(0);
                issue_a(rq, rq_tl, stg_c, IC<1>{});
                __builtin_amdgcn_sched_barrier(0);
                mfma_block(IC<0>{}, IC<1>{}, IC<0>{}, fa[0][1], IC<-1>{});
                if constexpr (NB0 > 1) mfma_block(IC<0>{}, IC<1>{}, IC<1>{}, fa[1][1], IC<-1>{});
                __builtin_amdgcn_sched_barrier(0);
                const ScaleReq sreq = next_scale_request();
                __builtin_amdgcn_sched_barrier(0);
                // the last A rows of this step (requested in the previous step's L0) must have landed:
                // younger than them are the previous step's C0, L1 and C1, the stores, and this step's L0 and C0
                { PROF_BEGIN(t_); CCH_WAIT_VM(NC0 + PREV_L1 + NC1 + STORES + NL0 + NC0); PROF_END(t_, pf_wa); }
                { PROF_BEGIN(t_); CCH_BARRIER(); PROF_END(t_, pf_b1); }
                // ------------------------------------------------------------------ L1
#pragma unroll
                for (int ks = 0; ks < 2; ks++)
#pragma unroll
                    for (int i = 0; i < NB1; i++) fa[i][ks] = frag_a(stg_c, ks, 2 + i);
                __builtin_amdgcn_sched_barrier(0);
                issue_b(rq, rq_tl, 0u, stg_c, IC<0>{});
                issue_b(rq, rq_tl, 0u, stg_c, IC<1>{});
                issue_scales(sreq);
                if constexpr (MODE == 1) issue_params(nxt, parity ^ 1);
                __builtin_amdgcn_sched_barrier(0);
                // B and the first A rows of the next step (requested in the previous step's C0, L1 and C1)
                // must have landed: younger than them are the stores and this step's L0, C0 and L1
                { PROF_BEGIN(t_); CCH_WAIT_VM_LGKM0(STORES + NL0 + NC0 + THIS_L1); PROF_END(t_, pf_wb); }
                { PROF_BEGIN(t_); CCH_BARRIER(); PROF_END(t_, pf_b2); }
                // ------------------------------------------------------------------ C1
                if constexpr (NB1 > 0) mfma_block(IC<FIRST>{}, IC<0>{}, IC<2>{}, fa[0][0], IC<-1>{});
                __builtin_amdgcn_sched_barrier(0);
                issue_b(rq, rq_tl, 0u, stg_c, IC<2>{});
                __builtin_amdgcn_sched_barrier(0);
                if constexpr (NB1 > 1) mfma_block(IC<FIRST>{}, IC<0>{}, IC<3>{}, fa[1][0], IC<-1>{});
                __builtin_amdgcn_sched_barrier(0);
                issue_b(rq, rq_tl, 0u, stg_c, IC<3>{});
                __builtin_amdgcn_sched_barrier(0);
                if constexpr (NB1 > 0) mfma_block(IC<0>{}, IC<1>{}, IC<2>{}, fa[0][1], IC<-1>{});
                if constexpr (NB1 > 1) mfma_block(IC<0>{}, IC<1>{}, IC<3>{}, fa[1][1], IC<-1>{});
                __builtin_amdgcn_sched_barrier(0);
                // where the next step (of this tile, or the next tile's first) reads its scales
                if constexpr (MODE == 2) prep_scale_reads(nbase);
                else advance_scale_reads(gbase, kt);
                __builtin_amdgcn_sched_barrier(0);
                if constexpr (MODE != 2) { PROF_BEGIN(t_); CCH_BARRIER(); PROF_END(t_, pf_b3); }
            }
            if constexpr (FIRST && NBLK < MT) {
                // row blocks that hold no row of the tile are never stored; give them a value all the same
#pragma unroll
                for (int i = NBLK; i < MT; i++)
#pragma unroll
                    for (int j = 0; j < NT; j++)
#pragma unroll
                        for (int x = 0; x < 16; x++) acc[i][j][x] = 0;
            }
            if constexpr (MODE != 0) {
                // Pin the accumulators here: otherwise the compiler sinks the MFMAs of the
                // peeled steps into the epilogue and spills their fragments to get them there.
#pragma unroll
                for (int i = 0; i < MT; i++)
#pragma unroll
                    for (int j = 0; j < NT; j++) asm volatile("" : "+v"(acc[i][j]));
            }
        };
        // Row blocks of this wave that hold rows of the tile: the K loop is instantiated for each count.
        // Block i of wave group wm starts at tile row 64*i + 32*wm, so of the tile's ceil(rows/32) blocks
        // the first group owns every other one from the first on and the second group the ones between
        // (a tile of at most 32 rows leaves the second group one block of zeros).
        auto k_loop = [&](auto nblk_c) {
            // The step count is made opaque per tile: addresses that depend on it (the scale
            // reads of the peeled steps) would otherwise be hoisted out of the tile loop and
            // held in registers through the K loop.
            int nk = nk_tile;
            asm volatile("" : "+s"(nk));
            if (nk > 2) {
                step(IC<0>{}, IC<1>{}, nblk_c, IC<0>{}, 0);
                step(IC<0>{}, IC<0>{}, nblk_c, IC<1>{}, 1);
                for (int kt = 2; kt + 2 < nk; kt += 2) {
                    step(IC<0>{}, IC<0>{}, nblk_c, IC<0>{}, kt);
                    step(IC<0>{}, IC<0>{}, nblk_c, IC<1>{}, kt + 1);
                }
                { PROF_BEGIN(t_); decode(t + nwg, nxt); PROF_END(t_, pf_dec); }
                step(IC<1>{}, IC<0>{}, nblk_c, IC<0>{}, nk - 2);
            } else {
                decode(t + nwg, nxt);
                step(IC<1>{}, IC<1>{}, nblk_c, IC<0>{}, 0);
            }
            step(IC<2>{}, IC<0>{}, nblk_c, IC<1>{}, nk - 1);
        };
#ifdef CCH_PROF
        const uint64_t pf_k0 = __builtin_readcyclecounter();
#endif
        const int nblk = uniform(min(max((((cur.rows + 31) >> 5) + 1 - wm) >> 1, 1), MT));
        if (nblk == 4) k_loop(IC<4>{});
        else if (nblk == 3) k_loop(IC<3>{});
        else if (nblk == 2) k_loop(IC<2>{});
        else k_loop(IC<1>{});
#ifdef CCH_PROF
        const uint64_t pf_k1 = __builtin_readcyclecounter();
#endif

        // Both groups run the epilogue in the same slot: the first group after the barrier that
        // ends its last matrix slot, the second (one slot behind) before it.
        if (wm == 0) CCH_BARRIER();

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
            const __amdgpu_buffer_rsrc_t rs_out = __builtin_amdgcn_make_buffer_rsrc(
                reinterpret_cast<uint8_t *>(p.out) + (has_map ? (size_t)0 : (size_t)cur.m0 * out_row_bytes), 0, 0x7FFFFFFF, 0x00020000);
            float chs[NT];
            if (DEQ) {
#pragma unroll
                for (int j = 0; j < NT; j++) chs[j] = __uint_as_float(lds_read4(prm + 1024u + (uint32_t)(wn * WN + j * 32 + r) * 4u));
            }
            // One pass = PASS_ROWS rows of a 32-row block: `produce` converts and writes them into the staging
            // buffer, `readback` fetches this lane's 16 bytes (and the row's destination), `emit` stores them.
            // The passes are software-pipelined: the values of pass n+1 are converted and written while the read
            // of pass n is under way (one wave's LDS operations execute in order, so the later writes cannot
            // overtake the earlier read), and only then is pass n stored.
            auto produce = [&](auto i_c, auto ps_c, auto fp16_c, auto half_step_c) {
                constexpr int i = decltype(i_c)::value, ps = decltype(ps_c)::value;
                // int8 epilogues: the per-channel product passes through IEEE half first (GemmProblem::i8_fp16_step)
                constexpr bool HALF_STEP = decltype(half_step_c)::value != 0;
#pragma unroll
                for (int qq = 0; qq < PASS_ROWS / 8; qq++) {
                    const int q = ps * (PASS_ROWS / 8) + qq;
                    float tok[4];
                    if (DEQ) {
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
                                if (EPI == EPI_SWIGLU) {
                                    // the up projection's result is a bf16 tile before the activation sees it
                                    const float gate = (float)(__bf16)(float)acc[i][0][x + d];
                                    const float up = (float)(__bf16)(float)acc[i][1][x + d];
                                    v[d] = gate * __builtin_amdgcn_rcpf(1.0f + __expf(-gate)) * up;
                                } else if (SWIGLU) {
                                    float gate = (float)acc[i][0][x + d] * chs[0], up = (float)acc[i][1][x + d] * chs[1];
                                    if constexpr (HALF_STEP) {
                                        // (the fp32 product is rounded before the half conversion sees it, as the golden's
                                        // two casts do: the compiler would otherwise fuse product and conversion into one
                                        // mixed-precision instruction with a single rounding)
                                        asm volatile("" : "+v"(gate), "+v"(up));
                                        gate = (float)(_Float16)gate;
                                        up = (float)(_Float16)up;
                                    }
                                    gate *= tok[xr + d];
                                    up *= tok[xr + d];
                                    // hardware exp2 and reciprocal: relative error ~1e-6, far inside the bf16 result
                                    v[d] = gate * __builtin_amdgcn_rcpf(1.0f + __expf(-gate)) * up;
                                } else if (EPI == EPI_DEQUANT) {
                                    if constexpr (HALF_STEP) {
                                        float prod = (float)acc[i][j][x + d] * chs[j];
                                        asm volatile("" : "+v"(prod));   // (see the SwiGLU branch)
                                        v[d] = (float)(_Float16)prod * tok[xr + d];
                                    } else {
                                        v[d] = (float)acc[i][j][x + d] * tok[xr + d] * chs[j];
                                    }
                                } else {
                                    v[d] = (float)acc[i][j][x + d];
                                }
                            }
                            // hardware RNE to bf16, both rows in one dword; then the neighbour's dword
                            // and one byte permute: even lanes keep the low halves (row x), odd lanes
                            // the high halves (row x+1), own column in its place
                            uint32_t pk;
                            if constexpr (decltype(fp16_c)::value) pk = __builtin_bit_cast(uint32_t, __builtin_convertvector((f32x2){v[0], v[1]}, f16x2));
                            else pk = __builtin_bit_cast(uint32_t, __builtin_convertvector((f32x2){v[0], v[1]}, bf16x2));
                            const uint32_t nb = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)pk, 0xB1, 0xF, 0xF, true);
                            const uint32_t packed = __builtin_amdgcn_perm(nb, pk, odd ? 0x03020706u : 0x05040100u);
                            const int lrow = qq * 8 + g * 4 + xr + (odd ? 1 : 0);
                            const int lcol = j * 32 + (r & ~1);
                            *reinterpret_cast<uint32_t *>(smem + epi + (uint32_t)(lrow * ROWB + lcol * 2)) = packed;
                        }
                }
            };
            struct PassData {
                v4i val;
                int mapped;
            };
            auto readback = [&](auto i_c, auto ps_c) {
                constexpr int i = decltype(i_c)::value, ps = decltype(ps_c)::value;
                PassData d;
                const int lrow = lane_e / CPR, chunk = lane_e % CPR;
                d.val = lds_read16(epi + (uint32_t)(lrow * ROWB + chunk * 16));
                d.mapped = 0;
                if constexpr (EPI == EPI_PLAIN) d.mapped = (int)lds_read4(prm + (uint32_t)(wm * WM + i * 32 + ps * PASS_ROWS + lrow) * 4u);
                return d;
            };
            auto emit = [&](auto i_c, auto ps_c, const PassData &d) {
                constexpr int i = decltype(i_c)::value, ps = decltype(ps_c)::value;
                const v4i val = d.val;
                const int lrow = lane_e / CPR, chunk = lane_e % CPR;
                const int row = i * 64 + wm * 32 + ps * PASS_ROWS + lrow;  // relative to m0 (row block i of this wave group)
                const int col = cur.j0 + wn * WN_OUT + chunk * 8;
                bool ok = (row < cur.rows) & (col + 8 <= p.n_out);
                uint32_t out_row = (uint32_t)row;
                if constexpr (EPI == EPI_PLAIN) {
                    // dropped or out of range: not written (without a map the destination is the row itself)
                    ok = ok & (!has_map | ((d.mapped >= 0) & (d.mapped < (int)p.out_rows)));
                    out_row = has_map ? (uint32_t)d.mapped : out_row;
                }
                if constexpr (SWIGLU) {
                    if (mx_out) {
                        // The four lanes of a quad hold the 32 columns of one row that this wave owns:
                        // one MX block.  Its maximum, shared exponent and codes as the row quantiser
                        // makes them from the bf16 values.
                        const uint32_t w[4] = {(uint32_t)val[0], (uint32_t)val[1], (uint32_t)val[2], (uint32_t)val[3]};
                        const uint32_t amax = block_amax_bits(w);
                        uint32_t code[2], sbyte;
                        int e;
                        bool is_nan;
                        if (p.mx_out_fmt == CCH_FMT_E2M1) {
                            sbyte = shared_exp_byte<CCH_FMT_E2M1>(amax, e, is_nan);
                            quant8_hw<CCH_FMT_E2M1>(w, e, is_nan, code);
                        } else if (p.mx_out_fmt == CCH_FMT_E5M2) {
                            sbyte = shared_exp_byte<CCH_FMT_E5M2>(amax, e, is_nan);
                            quant8_hw<CCH_FMT_E5M2>(w, e, is_nan, code);
                        } else {
                            sbyte = shared_exp_byte<CCH_FMT_E4M3>(amax, e, is_nan);
                            quant8_hw<CCH_FMT_E4M3>(w, e, is_nan, code);
                        }
                        const uint32_t elem = out_row * (uint32_t)p.n_out + (uint32_t)col;
                        if (p.mx_out_fmt == CCH_FMT_E2M1)
                            __builtin_amdgcn_raw_buffer_store_b32(code[0], rs_out, (int)(ok ? elem >> 1 : NO_FETCH), 0, 0);
                        else
                            __builtin_amdgcn_raw_buffer_store_b64((v2u){code[0], code[1]}, rs_out, (int)(ok ? elem : NO_FETCH), 0, 0);
                        // the quad's first lane writes the block's scale, and behind the last block of a row
                        // with an odd count of blocks the padding byte
                        const __amdgpu_buffer_rsrc_t rs_sc_out = __builtin_amdgcn_make_buffer_rsrc(
                            p.out_scales + (size_t)cur.m0 * p.mx_out_sld, 0, 0x7FFFFFFF, 0x00020000);
                        const uint32_t blk = (uint32_t)col >> 5, soff = out_row * (uint32_t)p.mx_out_sld + blk;
                        const bool first = ok && chunk == 0;
                        __builtin_amdgcn_raw_buffer_store_b8((uint8_t)sbyte, rs_sc_out, (int)(first ? soff : NO_FETCH), 0, 0);
                        if ((p.n_out & 32) != 0 && (int)blk == (p.n_out >> 5) - 1)
                            __builtin_amdgcn_raw_buffer_store_b8((uint8_t)127, rs_sc_out, (int)(first ? soff + 1 : NO_FETCH), 0, 0);
                        return;
                    }
                }
                const uint32_t off = ok ? (out_row * (uint32_t)p.n_out + (uint32_t)col) * 2u : NO_FETCH;
                const v4u sv = (v4u){(uint32_t)val[0], (uint32_t)val[1], (uint32_t)val[2], (uint32_t)val[3]};
                if (p.nt_out) __builtin_amdgcn_raw_buffer_store_b128(sv, rs_out, (int)off, 0, 2);   // non-temporal
                else __builtin_amdgcn_raw_buffer_store_b128(sv, rs_out, (int)off, 0, 0);
            };
            constexpr int NP = MT * NPASS;
            auto all_passes = [&](auto fp16_c, auto half_step_c) {
                produce(IC<0>{}, IC<0>{}, fp16_c, half_step_c);
                PassData pending = readback(IC<0>{}, IC<0>{});
                static_for<NP - 1>([&](auto n_c) {
                    constexpr int n = decltype(n_c)::value + 1;
                    produce(IC<n / NPASS>{}, IC<n % NPASS>{}, fp16_c, half_step_c);
                    __builtin_amdgcn_sched_barrier(0);   // the store's address arithmetic waits for the read: keep it behind the conversions
                    emit(IC<(n - 1) / NPASS>{}, IC<(n - 1) % NPASS>{}, pending);
                    pending = readback(IC<n / NPASS>{}, IC<n % NPASS>{});
                });
                emit(IC<(NP - 1) / NPASS>{}, IC<(NP - 1) % NPASS>{}, pending);
            };
            // the output type is a wave-uniform choice: one copy of the passes for each (the MX-quantised activation is
            // made from bf16 values)
            if constexpr (DEQ) {
                if (p.i8_fp16_step) {
                    if (p.out_fp16) all_passes(IC<1>{}, IC<1>{});
                    else all_passes(IC<0>{}, IC<1>{});
                } else {
                    if (p.out_fp16) all_passes(IC<1>{}, IC<0>{});
                    else all_passes(IC<0>{}, IC<0>{});
                }
            } else {
                if (p.out_fp16) all_passes(IC<1>{}, IC<0>{});
                else all_passes(IC<0>{}, IC<0>{});
            }
        }
#ifdef CCH_PROF
        if (lane == 0 && (wave & 3) == 0 && blockIdx.x < 256 && pf_nt < PROF_TILES) {
            uint64_t *o = cch_prof_tiles + (((size_t)blockIdx.x * 2 + wm) * PROF_TILES + pf_nt) * 6;
            o[0] = (uint64_t)(uint32_t)t | ((uint64_t)(uint32_t)cur.rows << 32) | ((uint64_t)(uint32_t)cur.e << 48);
            o[1] = pf_k0; o[2] = pf_k1; o[3] = __builtin_readcyclecounter(); o[4] = pf_dec; o[5] = pf_entry;
        }
        pf_nt++;
#endif
        if (wm == 1) CCH_BARRIER();
        cur = nxt;
        gbase = nbase;
        t += nwg;
        parity ^= 1;
    }
    if (any) {
        // the first group executed one barrier fewer than the second (which started one slot behind);
        // requests against empty descriptors may still be on their way to this workgroup's LDS
        if (wm == 0) CCH_BARRIER();
        CCH_WAIT_VM_LGKM0(0);
    }
#ifdef CCH_PROF
    if (lane == 0 && blockIdx.x < 256) {
        uint64_t *o = cch_prof + ((size_t)blockIdx.x * 8 + wave) * 8;
        o[0] = __builtin_readcyclecounter() - pf_start; o[1] = pf_l0; o[2] = pf_b0; o[3] = pf_wa; o[4] = pf_b1; o[5] = pf_wb; o[6] = pf_b2; o[7] = pf_b3;
    }
#endif
}

template <int KIND, int EPI, int FMT, int TB, int UA>
static int launch_tile_ua(const GemmProblem &p, hipStream_t stream)
{
    // the LDS size attribute is set once per device and kernel; setting it twice from two threads is harmless
    static std::atomic<uint64_t> attr_set{0};
    auto kern = gemm_tile_kernel<KIND, EPI, FMT, TB, UA>;
    int dev = 0, cus = 0;
    CCH_HIP(hipGetDevice(&dev));
    const uint64_t dev_bit = (uint64_t)1 << (dev & 63);
    if (dev >= 64 || !(attr_set.load(std::memory_order_acquire) & dev_bit)) {
        CCH_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, LDS_BYTES));
        attr_set.fetch_or(dev_bit, std::memory_order_release);
    }
    CCH_HIP(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev));
    constexpr int bn_out = (EPI == EPI_DEQUANT_SWIGLU || EPI == EPI_SWIGLU) ? BN / 2 : BN;
    const int64_t row_tiles = (p.T + BM - 1) / BM + (p.group_sizes ? p.num_groups : 0);  // upper bound
    const int64_t tiles = row_tiles * ((p.n_out + bn_out - 1) / bn_out);
    const unsigned grid = (unsigned)std::max<int64_t>(1, std::min<int64_t>(tiles, cus));
    hipLaunchKernelGGL(kern, dim3(grid), dim3(TILE_THREADS), LDS_BYTES, stream, p);
#ifdef CCH_PROF
    g_prof_copy = &prof_copy;
#endif
    return launch_status("gemm_tile_kernel");
}

// One kernel family (operand kind, epilogue, payload format, B layout): the instantiation for scale rows
// that all start on 4-byte boundaries and, for the MX kinds, the one for rows that do not.  Each family is
// compiled in a translation unit of its own (gemm_tile_*.hip) so that the library builds in parallel.
template <int KIND, int EPI, int FMT, int TB>
int launch_tile_t(const GemmProblem &p, hipStream_t stream)
{
    if constexpr (KIND != KIND_I8) {
        if ((p.sld & 3) != 0 || (p.sa_pitch & 3) != 0) return launch_tile_ua<KIND, EPI, FMT, TB, 1>(p, stream);
    }
    return launch_tile_ua<KIND, EPI, FMT, TB, 0>(p, stream);
}

}  // namespace cch
