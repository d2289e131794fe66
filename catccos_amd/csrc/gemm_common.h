// Shared definitions of the GEMM family: problem description, grouped-tile bookkeeping.
#pragma once
#include <hip/hip_runtime.h>

#include <cstdint>

#include "catccos_hip.h"

namespace cch {

enum GemmKind { KIND_I8 = 0, KIND_F8 = 1, KIND_F4 = 2 };
// EPI_SWIGLU (MX kinds): the accumulators are rounded to bf16, then out = silu(gate) * up on those values,
// as the reference's up projection hands its bf16 tile to the SwiGLU stage
// (include/catccos/epilogue/block/block_epilogue_regbase_swiglu.hpp:38-80)
enum GemmEpilogue { EPI_PLAIN = 0, EPI_DEQUANT = 1, EPI_DEQUANT_SWIGLU = 2, EPI_SWIGLU = 3 };

constexpr int MAX_GROUPS = 256;

// One (dense or grouped) problem: out[T, n_out] = epilogue(A[T,K] x B_e[K,N]).
struct GemmProblem {
    const uint8_t *a;        // [T, K] payload (FP4: K/2 bytes per row)
    const uint8_t *b;        // per expert: trans_b ? [N, K] : [K, N]   (FP4: last axis halved)
    const uint8_t *sa;       // MX: [T, sld] E8M0
    int64_t a_pitch;         // bytes between rows of a (0: rows are back to back)
    int64_t sa_pitch;        // bytes between rows of sa (0: sld); packed rows [payload | scales] have a_pitch == sa_pitch
    const uint8_t *sb;       // MX: per expert trans_b ? [N, sld] : [sld/2, N, 2]
    const float *per_tok;    // int8: [T]
    const float *per_ch;     // int8: [E, N]
    uint16_t *out;           // bf16 [T, n_out] (with out_row_map: [out_rows, n_out])
    const int32_t *out_row_map;  // device int32[T] or nullptr: row of `out` that receives row i (negative: dropped)
    int64_t out_rows;        // rows of `out` when out_row_map is given
    int out_fp16;            // output elements are IEEE half instead of bf16 (both rounded to nearest even)
    int i8_fp16_step;        // int8 epilogues: acc * per_channel is rounded to IEEE half (nearest even) before the per-token
                             // factor, as the reference's device does - its matrix unit's output stage writes the per-channel
                             // product as fp16 and the vector epilogue widens it again
                             // (include/catccos/epilogue/block/block_epilogue_per_token_dequant_swiglu.hpp:348-361; the golden
                             // generator's option, examples/utils/gen_data_dispatch_gmm_dequant_swiglu.py:309-310).  0 keeps
                             // fp32 throughout, the golden generator's default path.
    int mx_out;              // SwiGLU epilogue only: 1 = the activation leaves MX-quantised along its rows (what the
                             // row quantiser would make of the bf16 output): payload [T, n_out] codes of format
                             // mx_out_fmt at `out` (FP4: two per byte), E8M0 scales [T, mx_out_sld] at `out_scales`
    int mx_out_fmt;          // CCH_FMT_E4M3, CCH_FMT_E5M2 or CCH_FMT_E2M1
    int mx_out_sld;          // scale bytes per output row: 2*ceil(n_out/64), padding bytes are 127
    uint8_t *out_scales;
    const int32_t *group_sizes;  // device int32[E] or nullptr (dense, E = 1)
    int num_groups;
    int T, N, K;             // K in elements
    int n_out;               // N, or N/2 with SwiGLU
    int fmt;                 // CCH_FMT_* for MX kinds
    int trans_b;
    int sld;                 // scale bytes per row: 2*ceil(K/64)
    int64_t b_stride;        // bytes between experts in b
    int64_t sb_stride;       // bytes between experts in sb
    int nt_out;              // tiled kernels: output stores carry the non-temporal hint
    int tile_order;          // tiled kernels: 0 = row-major over (row tile, column tile); 1 = runs of consecutive tiles per XCD;
                             // 2 = a block of 4 row tiles x 8 column tiles per XCD where the shape allows (else 1 for groups, 0 without)
};

// Row ranges and tile counts of the groups, kept in LDS by every workgroup.
//   row_start[g] .. row_start[g+1]   rows of group g (g == num_groups: rows past the last group,
//                                    which are written as zeros)
//   tile_start[g]                    index of the group's first row-tile in the global tile-row list
struct GroupTable {
    int row_start[MAX_GROUPS + 2];
    int tile_start[MAX_GROUPS + 2];
};

// Fills the table (one thread), with rows clipped to T like the reference's golden does
// (examples/utils/gen_data_fp4_mx_alltoallv_gmm.py:788-790 zero-pads the remainder).
__device__ inline void build_group_table(GroupTable &tab, const int32_t *group_sizes, int num_groups, int T, int bm)
{
    int row = 0, tile = 0;
    for (int g = 0; g < num_groups; g++) {
        int sz = group_sizes ? group_sizes[g] : T;
        sz = max(0, min(sz, T - row));
        tab.row_start[g] = row;
        tab.tile_start[g] = tile;
        row += sz;
        tile += (sz + bm - 1) / bm;
    }
    tab.row_start[num_groups] = row;  // pseudo group: rows that belong to no expert
    tab.tile_start[num_groups] = tile;
    tile += (T - row + bm - 1) / bm;
    tab.row_start[num_groups + 1] = T;
    tab.tile_start[num_groups + 1] = tile;
}

// Group that owns global tile-row `tr` (largest g with tile_start[g] <= tr and a non-empty range).
__device__ inline int find_group(const GroupTable &tab, int num_groups, int tr)
{
    int lo = 0, hi = num_groups + 1;  // tile_start[lo] <= tr < tile_start[hi]
    while (hi - lo > 1) {
        const int mid = (lo + hi) >> 1;
        if (tab.tile_start[mid] <= tr) lo = mid; else hi = mid;
    }
    return lo;
}

}  // namespace cch
