// MX block quantiser: bf16 -> FP8 (E4M3/E5M2) or FP4 (E2M1/E1M2) payload + one E8M0 scale per
// 32 elements.  Streaming, HBM-bound kernel: every lane owns 8 consecutive elements (one
// 16-byte load), four neighbouring lanes own one MX block and reduce its maximum with two
// DPP quad permutes; payload leaves as one 8-byte (FP8) or 4-byte (FP4) store per lane.
//
// Follows CommBlockMxQuant::ComputeMxQuant (include/catccos/comm/block/comm_block_mx_quant.hpp:414-663)
// in intent and the generator examples/utils/gen_mx_quant_allgather_data.py:255-313, :385-449
// bit for bit.
#include <atomic>
#include <cstring>

#include "common.h"
#include "mx_formats.h"
#include "mx_quant_block.h"

namespace cch {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

constexpr int QUANT_THREADS = 512;        // large workgroups: the dispatcher places 512 blocks of 256 threads noticeably slower
constexpr int QUANT_UNROLL = 2;           // wave-steps (64 lanes x 8 elements) per batch
constexpr int QUANT_BLOCKS_PER_CU = 8;    // resident workgroups per CU the grid is sized for

// x [rows,K] bf16.  One wave-step = 64 lanes x 8 elements of one row; a row has `wpr` wave-steps.
// The grid is sized to the machine, not to the problem: every wave walks the list of wave-steps
// with a grid stride, QUANT_UNROLL at a time, and requests the next batch before it converts the
// current one, so that each wave always has loads in flight.
// VEC: K % 8 == 0 and all pointers suitably aligned, so whole-vector accesses are legal.
// PAIR (needs VEC, K % 16 == 0 and 16-byte aligned payload rows): neighbouring lanes swap halves
// of two wave-steps so that each lane stores one 16-byte (FP8) or 8-byte (FP4) piece instead of
// two of half that size; the store path's cost is per instruction, not per byte.
// SCATTER (without PAIR): row r of x is written to rows dst_idx[r*topk + 0 .. topk-1] of the output
// instead of row r; negative entries are skipped.  The row's destinations are read with the row
// itself, one batch ahead of their use.  `sstride` is the distance between scale rows (equal to
// `sld` unless payload and scales share one packed row).
constexpr int QUANT_MAX_TOPK = 8;
template <int FMT, int RND, bool HWCVT, bool VEC, bool PAIR, bool SCATTER = false>
__global__ __launch_bounds__(QUANT_THREADS) void mx_quant_rows_kernel(
    const uint16_t *__restrict__ x, uint8_t *__restrict__ payload, uint8_t *__restrict__ scales, int rows, int K,
    int nblk, int sld, int pld, int wpr, int total_ws, const int32_t *__restrict__ dst_idx = nullptr, int topk = 1,
    int sstride = 0, int out_rows = 0x7FFFFFFF)
{
    static_assert(!(SCATTER && PAIR), "the scatter variant stores one wave-step at a time");
    if (!SCATTER) sstride = sld;
    constexpr bool FP4 = is_fp4_v<FMT>;
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane((int)(blockIdx.x * (QUANT_THREADS / 64) + (threadIdx.x >> 6)));
    const int stride = (int)gridDim.x * (QUANT_THREADS / 64) * QUANT_UNROLL;

    struct Batch {
        uint32_t w[QUANT_UNROLL][4];
        int row[QUANT_UNROLL], k0[QUANT_UNROLL];
        int dst[QUANT_UNROLL][SCATTER ? QUANT_MAX_TOPK : 1];
    };
    auto fetch = [&](int ws0, Batch &bt) {
#pragma unroll
        for (int u = 0; u < QUANT_UNROLL; u++) {
            const int ws = ws0 + u;
            const int r = ws / wpr;
            bt.row[u] = ws < total_ws ? r : -1;
            bt.k0[u] = ((ws - r * wpr) * 64 + lane) * 8;
            bt.w[u][0] = bt.w[u][1] = bt.w[u][2] = bt.w[u][3] = 0;
            if constexpr (SCATTER) {
#pragma unroll
                for (int t = 0; t < QUANT_MAX_TOPK; t++) {
                    bt.dst[u][t] = (bt.row[u] >= 0 && t < topk) ? dst_idx[(size_t)bt.row[u] * topk + t] : -1;
                    if (bt.dst[u][t] >= out_rows) bt.dst[u][t] = -1;   // a row past the output is skipped like a negative one
                }
            }
            if (bt.row[u] >= 0 && bt.k0[u] < K) {
                const uint16_t *src = x + (size_t)bt.row[u] * K + bt.k0[u];
                if (VEC) {
                    const u32x4 v = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(src));
                    bt.w[u][0] = v[0]; bt.w[u][1] = v[1]; bt.w[u][2] = v[2]; bt.w[u][3] = v[3];
                } else {
#pragma unroll
                    for (int i = 0; i < 8; i++)
                        if (bt.k0[u] + i < K) bt.w[u][i >> 1] |= (uint32_t)src[i] << ((i & 1) * 16);
                }
            }
        }
    };
    auto convert = [&](const Batch &bt) {
        uint32_t held[2] = {0, 0};  // PAIR: payload of the even wave-step, waiting for its partner
#pragma unroll
        for (int u = 0; u < QUANT_UNROLL; u++) {
            if (bt.row[u] < 0) continue;  // wave-uniform
            const uint32_t amax_bits = block_amax_bits(bt.w[u]);
            int e;
            bool is_nan;
            const uint32_t sbyte = shared_exp_byte<FMT>(amax_bits, e, is_nan);
            uint32_t q[2];
            quant8<FMT, RND, HWCVT>(bt.w[u], e, is_nan, q);
            const int k0 = bt.k0[u], blk = k0 >> 5;
            if (PAIR) {
                // Wave-steps come in pairs (u even, u odd); a pair is complete unless the list
                // ends on the even one.  Even lanes end up with the even step's 16 (8) bytes of
                // lanes l and l+1, odd lanes with the odd step's bytes of lanes l-1 and l.
                const bool odd_lane = lane & 1;
                const bool partner = (u & 1) || (u + 1 < QUANT_UNROLL && bt.row[u + 1] >= 0);  // wave-uniform
                if (!(u & 1) && partner) {
                    held[0] = q[0];
                    held[1] = q[1];
                } else if (u & 1) {
                    const int ke = bt.k0[u - 1], ko = k0;  // same lane offset in both steps unless the row changed
                    uint32_t send0 = odd_lane ? held[0] : q[0], send1 = odd_lane ? held[1] : q[1];
                    const uint32_t recv0 = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)send0, 0xB1, 0xF, 0xF, true);
                    const uint32_t recv1 = FP4 ? 0u : (uint32_t)__builtin_amdgcn_update_dpp(0, (int)send1, 0xB1, 0xF, 0xF, true);
                    const int rw = odd_lane ? bt.row[u] : bt.row[u - 1];
                    const int kk = odd_lane ? ko - 8 : ke;
                    if (kk < K) {
                        uint8_t *dst = payload + (size_t)rw * pld + (FP4 ? (kk >> 1) : kk);
                        if (FP4) {
                            u32x2 o = odd_lane ? (u32x2){recv0, q[0]} : (u32x2){held[0], recv0};
                            __builtin_nontemporal_store(o, reinterpret_cast<u32x2 *>(dst));
                        } else {
                            u32x4 o = odd_lane ? (u32x4){recv0, recv1, q[0], q[1]} : (u32x4){held[0], held[1], recv0, recv1};
                            __builtin_nontemporal_store(o, reinterpret_cast<u32x4 *>(dst));
                        }
                    }
                } else if (k0 < K) {  // unpaired last step
                    uint8_t *dst = payload + (size_t)bt.row[u] * pld + (FP4 ? (k0 >> 1) : k0);
                    if (FP4) {
                        __builtin_nontemporal_store(q[0], reinterpret_cast<uint32_t *>(dst));
                    } else {
                        u32x2 o = {q[0], q[1]};
                        __builtin_nontemporal_store(o, reinterpret_cast<u32x2 *>(dst));
                    }
                }
            } else if (SCATTER) {
#pragma unroll
                for (int t = 0; t < QUANT_MAX_TOPK; t++) {
                    const int drow = bt.dst[u][t];
                    if (drow < 0) continue;  // wave-uniform
                    if (k0 < K) {
                        uint8_t *dst = payload + (size_t)drow * pld + (FP4 ? (k0 >> 1) : k0);
                        if (VEC) {
                            if (FP4) {
                                __builtin_nontemporal_store(q[0], reinterpret_cast<uint32_t *>(dst));
                            } else {
                                u32x2 o = {q[0], q[1]};
                                __builtin_nontemporal_store(o, reinterpret_cast<u32x2 *>(dst));
                            }
                        } else if (FP4) {
                            for (int i = 0; i < 4; i++)
                                if (k0 + 2 * i < K) dst[i] = (uint8_t)(q[0] >> (8 * i)) & (k0 + 2 * i + 1 < K ? 0xFF : 0x0F);
                        } else {
                            for (int i = 0; i < 8; i++)
                                if (k0 + i < K) dst[i] = (uint8_t)(q[i >> 2] >> (8 * (i & 3)));
                        }
                    }
                    if (blk < nblk) {
                        uint8_t *srow = scales + (size_t)drow * sstride;
                        if ((lane & 3) == 0) srow[blk] = (uint8_t)sbyte;
                        if ((lane & 3) == 1 && blk == nblk - 1 && sld != nblk) srow[nblk] = 127;  // even padding, 1.0
                    }
                }
                continue;
            } else if (k0 < K) {
                uint8_t *dst = payload + (size_t)bt.row[u] * pld + (FP4 ? (k0 >> 1) : k0);
                if (VEC) {
                    if (FP4) {
                        __builtin_nontemporal_store(q[0], reinterpret_cast<uint32_t *>(dst));
                    } else {
                        u32x2 o = {q[0], q[1]};
                        __builtin_nontemporal_store(o, reinterpret_cast<u32x2 *>(dst));
                    }
                } else if (FP4) {
                    for (int i = 0; i < 4; i++)
                        if (k0 + 2 * i < K) dst[i] = (uint8_t)(q[0] >> (8 * i)) & (k0 + 2 * i + 1 < K ? 0xFF : 0x0F);
                } else {
                    for (int i = 0; i < 8; i++)
                        if (k0 + i < K) dst[i] = (uint8_t)(q[i >> 2] >> (8 * (i & 3)));
                }
            }
            if (blk < nblk) {
                uint8_t *srow = scales + (size_t)bt.row[u] * sld;
                if ((lane & 3) == 0) srow[blk] = (uint8_t)sbyte;
                if ((lane & 3) == 1 && blk == nblk - 1 && sld != nblk) srow[nblk] = 127;  // even padding, 1.0
            }
        }
    };

    // Two batches in ping-pong: while one is converted and stored, the other's loads are in flight.
    Batch b0, b1;
    int ws0 = wave * QUANT_UNROLL;
    if (ws0 >= total_ws) return;
    fetch(ws0, b0);
    for (;;) {
        const int ws1 = ws0 + stride, ws2 = ws1 + stride;  // all wave-uniform
        if (ws1 < total_ws) fetch(ws1, b1);
        convert(b0);
        if (ws1 >= total_ws) break;
        if (ws2 < total_ws) fetch(ws2, b0);
        convert(b1);
        if (ws2 >= total_ws) break;
        ws0 = ws2;
    }
}

// Fast path of the row quantiser: round to nearest even with the hardware conversions, K a
// multiple of 1024 (so that wave-steps pair up inside a row and none is partial) and 16-byte
// aligned buffers.  No per-lane bounds checks; a wave owns pairs of adjacent wave-steps
// (1024 elements of one row), keeps the next pair's loads in flight while it converts the
// current one, stores 16 (FP8) or 8 (FP4) payload bytes per lane and writes the 32 scale bytes
// of the pair as dwords gathered with row shifts.
// SCATTER: as in mx_quant_rows_kernel, the row goes to rows dst_idx[r*topk + 0 .. topk-1]; `sld`
// is then the distance between scale rows of the packed output.
// HALF: the input is IEEE half instead of bf16 (same layout, same stores; the shared exponent comes
// from the block maximum widened to fp32 and the codes from the packed-half conversions).
template <int FMT, bool SCATTER = false, bool HALF = false>
__global__ __launch_bounds__(QUANT_THREADS) void mx_quant_rows_fast_kernel(
    const uint16_t *__restrict__ x, uint8_t *__restrict__ payload, uint8_t *__restrict__ scales, int K, int sld, int pld,
    int ppr, int npairs, const int32_t *__restrict__ dst_idx = nullptr, int topk = 1, int out_rows = 0x7FFFFFFF)
{
    constexpr bool FP4 = is_fp4_v<FMT>;
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane((int)(blockIdx.x * (QUANT_THREADS / 64) + (threadIdx.x >> 6)));
    const int stride = (int)gridDim.x * (QUANT_THREADS / 64);
    const bool odd_lane = lane & 1;

    struct Dest {
        int row[SCATTER ? QUANT_MAX_TOPK : 1];
    };
    auto fetch = [&](int p, u32x4 (&v)[2], Dest &d) {
        const int r = p / ppr, c = p - r * ppr;  // row, pair within the row (wave-uniform)
        const uint16_t *src = x + (size_t)r * K + (size_t)c * 1024 + lane * 8;
        v[0] = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(src));
        v[1] = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(src + 512));
        if constexpr (SCATTER) {
#pragma unroll
            for (int t = 0; t < QUANT_MAX_TOPK; t++) {
                d.row[t] = t < topk ? dst_idx[(size_t)r * topk + t] : -1;
                if (d.row[t] >= out_rows) d.row[t] = -1;   // a row past the output is skipped like a negative one
            }
        }
    };
    auto convert = [&](int p, const u32x4 (&v)[2], const Dest &d) {
        const int r0 = p / ppr, c = p - r0 * ppr;
        uint32_t q[2][2], sdw[2];
#pragma unroll
        for (int h = 0; h < 2; h++) {
            const uint32_t w[4] = {v[h][0], v[h][1], v[h][2], v[h][3]};
            const uint32_t amax_bits = block_amax_bits(w);   // |half| patterns order like |bf16| patterns
            int e;
            bool is_nan;
            uint32_t sbyte;
            if constexpr (HALF) {
                is_nan = amax_bits >= 0x7C00u;   // Inf or NaN in the block
                sbyte = shared_exp_byte_f32<FMT>(half_bits_to_f32(amax_bits), is_nan, e);
                quant8_f16_hw<FMT>(w, e, q[h]);
                if (is_nan) q[h][0] = q[h][1] = FP4 ? 0x77777777u : 0x7F7F7F7Fu;
            } else {
                sbyte = shared_exp_byte<FMT>(amax_bits, e, is_nan);
                quant8_hw<FMT>(w, e, is_nan, q[h]);
            }
            // lanes 4j hold block j's scale byte: gather 4 of them into lanes 0, 16, 32, 48
            const uint32_t b1 = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)sbyte, 0x104, 0xF, 0xF, true);  // row_shl:4
            const uint32_t b2 = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)sbyte, 0x108, 0xF, 0xF, true);  // row_shl:8
            const uint32_t b3 = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)sbyte, 0x10C, 0xF, 0xF, true);  // row_shl:12
            sdw[h] = sbyte | (b1 << 8) | (b2 << 16) | (b3 << 24);
        }
        // Neighbouring lanes swap: even lanes take both halves of step 0, odd lanes of step 1.
        const uint32_t send0 = odd_lane ? q[0][0] : q[1][0], send1 = odd_lane ? q[0][1] : q[1][1];
        const uint32_t recv0 = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)send0, 0xB1, 0xF, 0xF, true);
        const uint32_t recv1 = FP4 ? 0u : (uint32_t)__builtin_amdgcn_update_dpp(0, (int)send1, 0xB1, 0xF, 0xF, true);
        // element offset inside the row of the first value this lane stores
        const int k = c * 1024 + (odd_lane ? 512 + (lane - 1) * 8 : lane * 8);
#pragma unroll
        for (int t = 0; t < (SCATTER ? QUANT_MAX_TOPK : 1); t++) {
            const int r = SCATTER ? d.row[t] : r0;
            if (r < 0) continue;  // wave-uniform
            uint8_t *dst = payload + (size_t)r * pld + (FP4 ? (k >> 1) : k);
            if (FP4) {
                const u32x2 o = odd_lane ? (u32x2){recv0, q[1][0]} : (u32x2){q[0][0], recv0};
                __builtin_nontemporal_store(o, reinterpret_cast<u32x2 *>(dst));
            } else {
                const u32x4 o = odd_lane ? (u32x4){recv0, recv1, q[1][0], q[1][1]} : (u32x4){q[0][0], q[0][1], recv0, recv1};
                __builtin_nontemporal_store(o, reinterpret_cast<u32x4 *>(dst));
            }
            if ((lane & 15) == 0) {
                uint32_t *sp = reinterpret_cast<uint32_t *>(scales + (size_t)r * sld + c * 32 + (lane >> 4) * 4);
                sp[0] = sdw[0];
                sp[4] = sdw[1];
            }
        }
    };

    u32x4 v0[2], v1[2];
    Dest d0, d1;
    int p0 = wave;
    if (p0 >= npairs) return;
    fetch(p0, v0, d0);
    for (;;) {
        const int p1 = p0 + stride, p2 = p1 + stride;  // wave-uniform
        if (p1 < npairs) fetch(p1, v1, d1);
        convert(p0, v0, d0);
        if (p1 >= npairs) break;
        if (p2 < npairs) fetch(p2, v0, d0);
        convert(p1, v1, d1);
        if (p2 >= npairs) break;
        p0 = p2;
    }
}

// Fast form for IEEE half input (round to nearest even): returns 1 when the shape or the alignment
// is not the fast kernel's, so that the caller takes its general kernel.
template <int FMT>
static int launch_rows_fast_half(const void *x, void *payload, void *scales, int64_t m, int64_t k, hipStream_t stream)
{
    if (!(k % 1024 == 0 && aligned(x, 16) && aligned(payload, 16) && aligned(scales, 4) && m * (k / 1024) < ((int64_t)1 << 30))) return 1;
    const int64_t nblk = k / 32, sld = 2 * ((nblk + 1) / 2), pld = is_fp4_v<FMT> ? k / 2 : k;
    int dev = 0, cus = 0;
    CCH_HIP(hipGetDevice(&dev));
    CCH_HIP(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev));
    const int64_t npairs = m * (k / 1024);
    const unsigned grid = (unsigned)std::min<int64_t>((npairs + QUANT_THREADS / 64 - 1) / (QUANT_THREADS / 64), (int64_t)cus * QUANT_BLOCKS_PER_CU);
    hipLaunchKernelGGL((mx_quant_rows_fast_kernel<FMT, false, true>), dim3(grid), dim3(QUANT_THREADS), 0, stream,
                       static_cast<const uint16_t *>(x), static_cast<uint8_t *>(payload), static_cast<uint8_t *>(scales), (int)k, (int)sld,
                       (int)pld, (int)(k / 1024), (int)npairs);
    return launch_status("mx_quant_rows_fast_kernel (half input)");
}

int mx_quant_rows_fast_half(const void *x, void *payload, void *scales, int64_t m, int64_t k, int fmt, hipStream_t stream)
{
    if (fmt == CCH_FMT_E4M3) return launch_rows_fast_half<CCH_FMT_E4M3>(x, payload, scales, m, k, stream);
    if (fmt == CCH_FMT_E5M2) return launch_rows_fast_half<CCH_FMT_E5M2>(x, payload, scales, m, k, stream);
    if (fmt == CCH_FMT_E2M1) return launch_rows_fast_half<CCH_FMT_E2M1>(x, payload, scales, m, k, stream);
    return 1;
}

template <int FMT, int RND, bool HWCVT>
static int launch_rows(const void *x, void *payload, void *scales, int64_t m, int64_t k, hipStream_t stream)
{
    const bool fp4 = is_fp4_v<FMT>;
    const int64_t nblk = (k + 31) / 32, sld = 2 * ((nblk + 1) / 2), pld = fp4 ? (k + 1) / 2 : k;
    const int64_t wpr = (nblk * 4 + 63) / 64;
    const bool vec = (k % 8 == 0) && aligned(x, 16) && aligned(payload, 8);
    const bool pair = vec && (k % 16 == 0) && aligned(payload, 16) && QUANT_UNROLL % 2 == 0;
    int dev = 0, cus = 0;
    CCH_HIP(hipGetDevice(&dev));
    CCH_HIP(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev));
    const int64_t max_blocks = (int64_t)cus * QUANT_BLOCKS_PER_CU;
    if constexpr (HWCVT)
    if (k % 1024 == 0 && aligned(x, 16) && aligned(payload, 16) && aligned(scales, 4) && m * (k / 1024) < ((int64_t)1 << 30)) {
        const int64_t npairs = m * (k / 1024);
        const unsigned grid = (unsigned)std::min<int64_t>((npairs + QUANT_THREADS / 64 - 1) / (QUANT_THREADS / 64), max_blocks);
        hipLaunchKernelGGL((mx_quant_rows_fast_kernel<FMT>), dim3(grid), dim3(QUANT_THREADS), 0, stream,
                           static_cast<const uint16_t *>(x), static_cast<uint8_t *>(payload), static_cast<uint8_t *>(scales),
                           (int)k, (int)sld, (int)pld, (int)(k / 1024), (int)npairs);
        return launch_status("mx_quant_rows_fast_kernel");
    }
    const int64_t rows_per_launch = std::max<int64_t>(1, (int64_t)(1 << 30) / wpr);
    for (int64_t r0 = 0; r0 < m; r0 += rows_per_launch) {
        const int64_t rows = std::min(rows_per_launch, m - r0);
        const int64_t total_ws = rows * wpr;
        const int64_t waves = (total_ws + QUANT_UNROLL - 1) / QUANT_UNROLL;
        const unsigned grid = (unsigned)std::min<int64_t>((waves + QUANT_THREADS / 64 - 1) / (QUANT_THREADS / 64), max_blocks);
        const uint16_t *xs = static_cast<const uint16_t *>(x) + r0 * k;
        uint8_t *ps = static_cast<uint8_t *>(payload) + r0 * pld;
        uint8_t *ss = static_cast<uint8_t *>(scales) + r0 * sld;
        if (vec && pair)
            hipLaunchKernelGGL((mx_quant_rows_kernel<FMT, RND, HWCVT, true, true>), dim3(grid), dim3(QUANT_THREADS), 0, stream,
                               xs, ps, ss, (int)rows, (int)k, (int)nblk, (int)sld, (int)pld, (int)wpr, (int)total_ws);
        else if (vec)
            hipLaunchKernelGGL((mx_quant_rows_kernel<FMT, RND, HWCVT, true, false>), dim3(grid), dim3(QUANT_THREADS), 0, stream,
                               xs, ps, ss, (int)rows, (int)k, (int)nblk, (int)sld, (int)pld, (int)wpr, (int)total_ws);
        else
            hipLaunchKernelGGL((mx_quant_rows_kernel<FMT, RND, HWCVT, false, false>), dim3(grid), dim3(QUANT_THREADS), 0,
                               stream, xs, ps, ss, (int)rows, (int)k, (int)nblk, (int)sld, (int)pld, (int)wpr,
                               (int)total_ws);
        int rc = launch_status("mx_quant_rows_kernel");
        if (rc) return rc;
    }
    return CCH_OK;
}


// Quantiser for a right-hand operand b [K,N] with MX blocks running down K.  One thread owns
// two adjacent columns of one 32-row block: 32 coalesced 4-byte loads, results written in
// either boundary layout.  Input preparation, not a hot path.
template <int FMT, int RND>
__global__ __launch_bounds__(256) void mx_quant_b_kernel(const uint32_t *__restrict__ b, uint8_t *__restrict__ payload,
                                                         uint8_t *__restrict__ scales, int K, int N, int trans_b)
{
    using T = FmtTraits<FMT>;
    constexpr bool FP4 = is_fp4_v<FMT>;
    const int np = blockIdx.x * 256 + threadIdx.x;  // column pair
    const int kb = blockIdx.y;
    if (np * 2 >= N) return;
    const int sld = K / 32;
    uint32_t w[32];
    uint32_t m0 = 0, m1 = 0;
#pragma unroll
    for (int i = 0; i < 32; i++) {
        w[i] = b[((size_t)(kb * 32 + i) * N) / 2 + np];
        m0 = max(m0, w[i] & 0x7FFFu);
        m1 = max(m1, (w[i] >> 16) & 0x7FFFu);
    }
    int e0, e1;
    bool n0, n1;
    const uint32_t s0 = shared_exp_byte<FMT>(m0, e0, n0), s1 = shared_exp_byte<FMT>(m1, e1, n1);
    // 2^-e in two exact factors (2^-127 is no normal float)
    const float i0 = pow2i(-min(e0, 126)), i1 = pow2i(-min(e1, 126));
    const float j0 = e0 > 126 ? 0.5f : 1.0f, j1 = e1 > 126 ? 0.5f : 1.0f;
    uint32_t q0[32], q1[32];
#pragma unroll
    for (int i = 0; i < 32; i++) {
        q0[i] = n0 ? T::NANCODE : encode_small<FMT, RND>(__uint_as_float(w[i] << 16) * i0 * j0);
        q1[i] = n1 ? T::NANCODE : encode_small<FMT, RND>(__uint_as_float(w[i] & 0xFFFF0000u) * i1 * j1);
    }
    const int n = np * 2;
    if (!trans_b) {
#pragma unroll
        for (int i = 0; i < 32; i++) {
            const size_t k = (size_t)kb * 32 + i;
            if (FP4) payload[k * (N / 2) + np] = (uint8_t)(q0[i] | (q1[i] << 4));
            else *reinterpret_cast<uint16_t *>(payload + k * N + n) = (uint16_t)(q0[i] | (q1[i] << 8));
        }
        uint8_t *sp = scales + ((size_t)(kb >> 1) * N + n) * 2 + (kb & 1);
        sp[0] = (uint8_t)s0;
        sp[2] = (uint8_t)s1;
    } else {
        if (FP4) {
            uint8_t *d0 = payload + (size_t)n * (K / 2) + kb * 16, *d1 = d0 + K / 2;
#pragma unroll
            for (int i = 0; i < 16; i++) {
                d0[i] = (uint8_t)(q0[2 * i] | (q0[2 * i + 1] << 4));
                d1[i] = (uint8_t)(q1[2 * i] | (q1[2 * i + 1] << 4));
            }
        } else {
            uint8_t *d0 = payload + (size_t)n * K + kb * 32, *d1 = d0 + K;
#pragma unroll
            for (int i = 0; i < 32; i++) {
                d0[i] = (uint8_t)q0[i];
                d1[i] = (uint8_t)q1[i];
            }
        }
        scales[(size_t)n * sld + kb] = (uint8_t)s0;
        scales[(size_t)(n + 1) * sld + kb] = (uint8_t)s1;
    }
}

template <int FMT, int RND>
static int launch_b(const void *b, void *payload, void *scales, int64_t k, int64_t n, int trans_b, hipStream_t stream)
{
    dim3 grid((unsigned)((n / 2 + 255) / 256), (unsigned)(k / 32));
    hipLaunchKernelGGL((mx_quant_b_kernel<FMT, RND>), grid, dim3(256), 0, stream, static_cast<const uint32_t *>(b),
                       static_cast<uint8_t *>(payload), static_cast<uint8_t *>(scales), (int)k, (int)n, trans_b);
    return launch_status("mx_quant_b_kernel");
}

// Quantise-once, scatter-to-top-K launch: packed output rows of `row_bytes` = payload bytes +
// padded scale bytes.
template <int FMT, int RND, bool HWCVT>
static int launch_scatter(const void *x, const int32_t *dst_idx, void *packed, int64_t tokens, int64_t k, int topk,
                          int out_rows, hipStream_t stream)
{
    const bool fp4 = is_fp4_v<FMT>;
    const int64_t nblk = (k + 31) / 32, sld = 2 * ((nblk + 1) / 2), pbytes = fp4 ? (k + 1) / 2 : k;
    const int64_t row_bytes = pbytes + sld;
    const int64_t wpr = (nblk * 4 + 63) / 64;
    const bool vec = (k % 8 == 0) && aligned(x, 16) && aligned(packed, 8) && row_bytes % 8 == 0;
    int dev = 0, cus = 0;
    CCH_HIP(hipGetDevice(&dev));
    CCH_HIP(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev));
    const int64_t max_blocks = (int64_t)cus * QUANT_BLOCKS_PER_CU;
    uint8_t *out = static_cast<uint8_t *>(packed);
    if constexpr (HWCVT)
    if (k % 1024 == 0 && aligned(x, 16) && aligned(packed, 16) && row_bytes % 16 == 0 &&
        tokens * (k / 1024) < ((int64_t)1 << 30)) {
        const int64_t npairs = tokens * (k / 1024);
        const unsigned grid = (unsigned)std::min<int64_t>((npairs + QUANT_THREADS / 64 - 1) / (QUANT_THREADS / 64), max_blocks);
        hipLaunchKernelGGL((mx_quant_rows_fast_kernel<FMT, true>), dim3(grid), dim3(QUANT_THREADS), 0, stream,
                           static_cast<const uint16_t *>(x), out, out + pbytes, (int)k, (int)row_bytes, (int)row_bytes,
                           (int)(k / 1024), (int)npairs, dst_idx, topk, out_rows);
        return launch_status("mx_quant_rows_fast_kernel (scatter)");
    }
    const int64_t rows_per_launch = std::max<int64_t>(1, (int64_t)(1 << 30) / wpr);
    for (int64_t r0 = 0; r0 < tokens; r0 += rows_per_launch) {
        const int64_t rows = std::min(rows_per_launch, tokens - r0);
        const int64_t total_ws = rows * wpr;
        const int64_t waves = (total_ws + QUANT_UNROLL - 1) / QUANT_UNROLL;
        const unsigned grid = (unsigned)std::min<int64_t>((waves + QUANT_THREADS / 64 - 1) / (QUANT_THREADS / 64), max_blocks);
        const uint16_t *xs = static_cast<const uint16_t *>(x) + r0 * k;
        const int32_t *ds = dst_idx + r0 * topk;
        if (vec)
            hipLaunchKernelGGL((mx_quant_rows_kernel<FMT, RND, HWCVT, true, false, true>), dim3(grid), dim3(QUANT_THREADS), 0,
                               stream, xs, out, out + pbytes, (int)rows, (int)k, (int)nblk, (int)sld, (int)row_bytes, (int)wpr,
                               (int)total_ws, ds, topk, (int)row_bytes, out_rows);
        else
            hipLaunchKernelGGL((mx_quant_rows_kernel<FMT, RND, HWCVT, false, false, true>), dim3(grid), dim3(QUANT_THREADS), 0,
                               stream, xs, out, out + pbytes, (int)rows, (int)k, (int)nblk, (int)sld, (int)row_bytes, (int)wpr,
                               (int)total_ws, ds, topk, (int)row_bytes, out_rows);
        int rc = launch_status("mx_quant_rows_kernel (scatter)");
        if (rc) return rc;
    }
    return CCH_OK;
}

// Library switch "quant_integer_encoder": the E4M3 round-to-nearest-even quantiser runs through the
// integer encoder instead of the hardware conversion, so that the two can be compared bit for bit
// on the device.
static std::atomic<int> g_quant_integer_encoder{0};
bool quant_set_option(const char *name, int value)
{
    if (strcmp(name, "quant_integer_encoder") != 0) return false;
    g_quant_integer_encoder.store(value);
    return true;
}

}  // namespace cch

extern "C" int cch_mx_quant_scatter_packed(const void *x, const int32_t *expanded_row_idx, void *packed_out, int64_t tokens,
                                           int64_t k, int top_k, int fmt, int rounding, void *stream)
{
    return cch_mx_quant_scatter_packed_rows(x, expanded_row_idx, packed_out, 0x7FFFFFFF, tokens, k, top_k, fmt, rounding, stream);
}

extern "C" int cch_mx_quant_scatter_packed_rows(const void *x, const int32_t *expanded_row_idx, void *packed_out, int64_t out_rows,
                                                int64_t tokens, int64_t k, int top_k, int fmt, int rounding, void *stream)
{
    using namespace cch;
    CCH_REQUIRE(out_rows >= 0, "cch_mx_quant_scatter_packed: out_rows=%lld", (long long)out_rows);
    const int orows = (int)std::min<int64_t>(out_rows, 0x7FFFFFFF);
    CCH_REQUIRE(tokens >= 0 && k >= 0, "cch_mx_quant_scatter_packed: negative shape tokens=%lld k=%lld", (long long)tokens,
                (long long)k);
    CCH_REQUIRE(k < (int64_t)1 << 30, "cch_mx_quant_scatter_packed: k=%lld too large", (long long)k);
    CCH_REQUIRE(top_k >= 0 && top_k <= QUANT_MAX_TOPK, "cch_mx_quant_scatter_packed: top_k=%d outside 0..%d", top_k,
                QUANT_MAX_TOPK);
    CCH_REQUIRE(rounding == CCH_ROUND_RNE || rounding == CCH_ROUND_LUT, "cch_mx_quant_scatter_packed: rounding %d", rounding);
    if (tokens == 0 || k == 0 || top_k == 0) return CCH_OK;  // as the reference: nothing to do
    CCH_REQUIRE(x && expanded_row_idx && packed_out, "cch_mx_quant_scatter_packed: null pointer");
    hipStream_t s = static_cast<hipStream_t>(stream);
    const bool lut = rounding == CCH_ROUND_LUT;
    switch (fmt) {
        case CCH_FMT_E4M3:
            return lut ? launch_scatter<CCH_FMT_E4M3, CCH_ROUND_LUT, false>(x, expanded_row_idx, packed_out, tokens, k, top_k, orows, s)
                       : launch_scatter<CCH_FMT_E4M3, CCH_ROUND_RNE, true>(x, expanded_row_idx, packed_out, tokens, k, top_k, orows, s);
        case CCH_FMT_E5M2:
            return lut ? launch_scatter<CCH_FMT_E5M2, CCH_ROUND_LUT, false>(x, expanded_row_idx, packed_out, tokens, k, top_k, orows, s)
                       : launch_scatter<CCH_FMT_E5M2, CCH_ROUND_RNE, true>(x, expanded_row_idx, packed_out, tokens, k, top_k, orows, s);
        case CCH_FMT_E2M1:
            return lut ? launch_scatter<CCH_FMT_E2M1, CCH_ROUND_LUT, false>(x, expanded_row_idx, packed_out, tokens, k, top_k, orows, s)
                       : launch_scatter<CCH_FMT_E2M1, CCH_ROUND_RNE, true>(x, expanded_row_idx, packed_out, tokens, k, top_k, orows, s);
        case CCH_FMT_E1M2:  // no hardware conversion for this format: integer encoder for both rules
            return lut ? launch_scatter<CCH_FMT_E1M2, CCH_ROUND_LUT, false>(x, expanded_row_idx, packed_out, tokens, k, top_k, orows, s)
                       : launch_scatter<CCH_FMT_E1M2, CCH_ROUND_RNE, false>(x, expanded_row_idx, packed_out, tokens, k, top_k, orows, s);
        default:
            return fail(CCH_EINVAL, "cch_mx_quant_scatter_packed: unknown format %d", fmt);
    }
}

extern "C" int cch_mx_quant_rows(const void *x, void *payload, void *scales, int64_t m, int64_t k, int fmt,
                                 int rounding, void *stream)
{
    using namespace cch;
    CCH_REQUIRE(m >= 0 && k >= 0, "cch_mx_quant_rows: negative shape m=%lld k=%lld", (long long)m, (long long)k);
    CCH_REQUIRE(k < (int64_t)1 << 30, "cch_mx_quant_rows: k=%lld too large", (long long)k);
    CCH_REQUIRE(rounding == CCH_ROUND_RNE || rounding == CCH_ROUND_LUT, "cch_mx_quant_rows: rounding %d", rounding);
    if (m == 0 || k == 0) return CCH_OK;
    CCH_REQUIRE(x && payload && scales, "cch_mx_quant_rows: null pointer");
    hipStream_t s = static_cast<hipStream_t>(stream);
    const bool lut = rounding == CCH_ROUND_LUT;
    switch (fmt) {
        case CCH_FMT_E4M3:
            if (!lut && g_quant_integer_encoder.load())   // cross-check of the hardware conversion on the device
                return launch_rows<CCH_FMT_E4M3, CCH_ROUND_RNE, false>(x, payload, scales, m, k, s);
            return lut ? launch_rows<CCH_FMT_E4M3, CCH_ROUND_LUT, false>(x, payload, scales, m, k, s)
                       : launch_rows<CCH_FMT_E4M3, CCH_ROUND_RNE, true>(x, payload, scales, m, k, s);
        case CCH_FMT_E5M2:
            return lut ? launch_rows<CCH_FMT_E5M2, CCH_ROUND_LUT, false>(x, payload, scales, m, k, s)
                       : launch_rows<CCH_FMT_E5M2, CCH_ROUND_RNE, true>(x, payload, scales, m, k, s);
        case CCH_FMT_E2M1:
            return lut ? launch_rows<CCH_FMT_E2M1, CCH_ROUND_LUT, false>(x, payload, scales, m, k, s)
                       : launch_rows<CCH_FMT_E2M1, CCH_ROUND_RNE, true>(x, payload, scales, m, k, s);
        case CCH_FMT_E1M2:  // no hardware conversion for this format: integer encoder for both rules
            return lut ? launch_rows<CCH_FMT_E1M2, CCH_ROUND_LUT, false>(x, payload, scales, m, k, s)
                       : launch_rows<CCH_FMT_E1M2, CCH_ROUND_RNE, false>(x, payload, scales, m, k, s);
        default:
            return fail(CCH_EINVAL, "cch_mx_quant_rows: unknown format %d", fmt);
    }
}

extern "C" int cch_mx_quant_b(const void *b, void *payload, void *scales, int64_t k, int64_t n, int fmt, int rounding,
                              int trans_b, void *stream)
{
    using namespace cch;
    CCH_REQUIRE(k >= 0 && n >= 0, "cch_mx_quant_b: negative shape");
    CCH_REQUIRE(k % 64 == 0 && n % 2 == 0, "cch_mx_quant_b: needs k %% 64 == 0 and n %% 2 == 0 (k=%lld n=%lld)",
                (long long)k, (long long)n);
    CCH_REQUIRE(k / 32 <= 65535 && k * n < ((int64_t)1 << 40), "cch_mx_quant_b: shape too large");
    CCH_REQUIRE(rounding == CCH_ROUND_RNE || rounding == CCH_ROUND_LUT, "cch_mx_quant_b: rounding %d", rounding);
    CCH_REQUIRE(trans_b == 0 || trans_b == 1, "cch_mx_quant_b: trans_b %d", trans_b);
    if (k == 0 || n == 0) return CCH_OK;
    CCH_REQUIRE(b && payload && scales, "cch_mx_quant_b: null pointer");
    CCH_REQUIRE(aligned(b, 4) && aligned(payload, 2), "cch_mx_quant_b: misaligned pointer");
    hipStream_t s = static_cast<hipStream_t>(stream);
    const bool lut = rounding == CCH_ROUND_LUT;
    switch (fmt) {
        case CCH_FMT_E4M3:
            return lut ? launch_b<CCH_FMT_E4M3, CCH_ROUND_LUT>(b, payload, scales, k, n, trans_b, s)
                       : launch_b<CCH_FMT_E4M3, CCH_ROUND_RNE>(b, payload, scales, k, n, trans_b, s);
        case CCH_FMT_E5M2:
            return lut ? launch_b<CCH_FMT_E5M2, CCH_ROUND_LUT>(b, payload, scales, k, n, trans_b, s)
                       : launch_b<CCH_FMT_E5M2, CCH_ROUND_RNE>(b, payload, scales, k, n, trans_b, s);
        case CCH_FMT_E2M1:
            return lut ? launch_b<CCH_FMT_E2M1, CCH_ROUND_LUT>(b, payload, scales, k, n, trans_b, s)
                       : launch_b<CCH_FMT_E2M1, CCH_ROUND_RNE>(b, payload, scales, k, n, trans_b, s);
        case CCH_FMT_E1M2:
            return lut ? launch_b<CCH_FMT_E1M2, CCH_ROUND_LUT>(b, payload, scales, k, n, trans_b, s)
                       : launch_b<CCH_FMT_E1M2, CCH_ROUND_RNE>(b, payload, scales, k, n, trans_b, s);
        default:
            return fail(CCH_EINVAL, "cch_mx_quant_b: unknown format %d", fmt);
    }
}
