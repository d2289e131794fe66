/*
 * catccos_hip.h -- C ABI of the MI355X (gfx950) compute library.
 *
 * One shared library (libcatccos_hip.so) exports the per-rank compute half of
 * five CATCCOS fused operators.  All arguments are plain pointers and sizes;
 * device pointers are HIP device addresses, `stream` is a hipStream_t passed as
 * void* (NULL = the default stream).  Every call returns 0 on success or a
 * negative CCH_E* code; cch_last_error() then gives a message for the calling
 * thread.  Kernel entry points only enqueue work; they never synchronise.
 *
 * Reference interfaces these entry points stand in for (paths relative to the
 * reference tree) are cited on each declaration.
 */
#ifndef CATCCOS_HIP_H
#define CATCCOS_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* status codes */
#define CCH_OK 0
#define CCH_EINVAL (-1)   /* bad argument (shape, alignment, enum)          */
#define CCH_EHIP (-2)     /* a HIP runtime call failed                      */
#define CCH_ENODEV (-3)   /* no gfx950 device visible                       */
#define CCH_ENOSUP (-4)   /* valid request this build does not implement    */

/* payload formats (MX_QUANT_DTYPE of examples/ascend950_mx_quant_allgather/CMakeLists.txt:11-36) */
#define CCH_FMT_E4M3 0
#define CCH_FMT_E5M2 1
#define CCH_FMT_E2M1 2
#define CCH_FMT_E1M2 3 /* FP4 with one exponent and two mantissa bits (0, .25 ... 1.75): quantiser only */

/* payload rounding: 0 = round to nearest even, sign of zero kept (the device
 * cast, include/catccos/comm/block/comm_block_mx_quant.hpp:596-642);
 * 1 = the golden generator's table rule: ties to the smaller magnitude, zero
 * always +0 (examples/utils/gen_mx_quant_allgather_data.py:198-247). */
#define CCH_ROUND_RNE 0
#define CCH_ROUND_LUT 1

/* Output element types of the GEMM entry points that take an out_dtype. */
#define CCH_OUT_BF16 0
#define CCH_OUT_FP16 1

/* ---- runtime shims: what the host operator layer needs in place of acl.h ----
 * Replace aclInit/aclrtSetDevice, aclrtMalloc/aclrtFree, aclrtMallocHost/
 * aclrtFreeHost, aclrtMemcpy, aclrtMemset, aclrtCreateStream/
 * aclrtSynchronizeStream/aclrtDestroyStream as used by utils/info.h:135-193 and
 * examples/<op>/<op>_host.h. */
int cch_init(int device);
const char *cch_last_error(void);
int cch_device_info(char *name, size_t name_len, int *compute_units, int *clock_mhz, uint64_t *hbm_bytes);
int cch_malloc(void **ptr, size_t bytes);
int cch_free(void *ptr);
int cch_malloc_host(void **ptr, size_t bytes);
int cch_free_host(void *ptr);
int cch_memcpy_h2d(void *dst, const void *src, size_t bytes);
int cch_memcpy_d2h(void *dst, const void *src, size_t bytes);
int cch_memset(void *dst, int value, size_t bytes);
int cch_stream_create(void **stream);
int cch_stream_sync(void *stream);
int cch_stream_destroy(void *stream);

/* ---- MX block quantisation (config 1) --------------------------------------
 * Replaces the quantising half of Comm::Kernel::MxQuantAllGather
 * (include/catccos/comm/kernel/mx_quant_allgather.hpp:165-212) and
 * CommBlockMxQuant::ComputeMxQuant (include/catccos/comm/block/
 * comm_block_mx_quant.hpp:414-663), launched in the reference by
 * LaunchAscend950BF16QuantAllGatherFP8E4M3FN
 * (tests/dynamic_tiling/impl/kernel_mxfp_ascend950.cpp:19).
 *   x        bf16 [m,k] row-major
 *   payload  FP8: [m,k] bytes; FP4: [m,ceil(k/2)], element 2j in the low nibble
 *   scales   E8M0 [m, 2*ceil(k/64)]; entries past ceil(k/32) are 127 (=1.0)
 * One scale per 32 consecutive elements of a row; a ragged last block is
 * treated as zero padded.  fmt: any CCH_FMT_* — the four output types of the
 * reference's example (examples/ascend950_mx_quant_allgather/main.cpp:24-37,
 * MX_QUANT_DTYPE 0..3 = fp8_e4m3, fp8_e5m2, fp4_e2m1, fp4_e1m2). */
int cch_mx_quant_rows(const void *x, void *payload, void *scales, int64_t m, int64_t k, int fmt, int rounding,
                      void *stream);

/* The same quantiser for IEEE half input, the `half` instantiation of the reference's quantiser
 * (MxQuantTraits<half>, include/catccos/epilogue/block/block_epilogue_dynamic_mx_quant.hpp:57-71:
 * the input is widened to fp32 and the shared exponent is taken from the fp32 exponent field of the
 * block maximum).  x: half [m,k]; outputs, formats and rounding rules as cch_mx_quant_rows. */
int cch_mx_quant_rows_f16(const void *x, void *payload, void *scales, int64_t m, int64_t k, int fmt, int rounding,
                          void *stream);

/* Same quantiser for a right-hand GEMM operand b [k,n] (row-major bf16) with
 * blocks running down the k axis, i.e. what the reference's generators do for B
 * (examples/ascend950_mxfp8_matmul_reduce_scatter/scripts/gen_data_mxfp8_mmrs.py:202-217).
 *   trans_b = 0: payload [k,n] (FP4 [k,n/2]), scales physical [ceil(k/64), n, 2]
 *   trans_b = 1: payload [n,k] (FP4 [n,k/2]), scales [n, 2*ceil(k/64)]
 * Requires k % 64 == 0 and n % 2 == 0. */
int cch_mx_quant_b(const void *b, void *payload, void *scales, int64_t k, int64_t n, int fmt, int rounding,
                   int trans_b, void *stream);

/* ---- int8 W8A8 matmul + per-token x per-channel dequant (config 2) ----------
 * Replaces LaunchAllGatherMatmulDequantINT8 (tests/dynamic_tiling/impl/kernel_int8.cpp:113-130)
 * minus its allgather, i.e. FixpipeBlockMmad::operator()
 * (include/catccos/dgemm/block/block_mmad_preload_fixpipe.hpp:151-379) followed by the
 * per-token epilogue (include/catccos/epilogue/block/block_epilogue_per_token_dequant.hpp:247-266):
 *   out[m,n] = bf16( float(sum_k a[m,k]*b[k,n]) * per_tok[m] * per_ch[n] )
 *   a int8 [m,k]; b int8 [k,n] (trans_b=0) or [n,k] (trans_b=1); per_tok fp32 [m];
 *   per_ch fp32 [n]; out bf16 [m,n]. */
int cch_gemm_i8_dequant(const void *a, const void *b, const float *per_tok, const float *per_ch, void *out, int64_t m,
                        int64_t n, int64_t k, int trans_b, void *stream);
/* The same with a choice of output type: out_dtype CCH_OUT_BF16 or CCH_OUT_FP16 (IEEE half, the
 * type the reference's int8 launchers write: `using ElementC = half`,
 * tests/dynamic_tiling/impl/kernel_int8.cpp:16); both are the fp32 result rounded to nearest even. */
int cch_gemm_i8_dequant_out(const void *a, const void *b, const float *per_tok, const float *per_ch, void *out, int64_t m,
                            int64_t n, int64_t k, int trans_b, int out_dtype, void *stream);

/* ---- MoE grouped W8A8 matmul + dequant, without the activation ----------------
 * The grouped GEMM and per-token dequantisation of AlltoallvGmmDequantKernel
 * (include/catccos/dgemm/kernel/alltoallv_gmm_dequant_v2.hpp:164-244 with
 * include/catccos/epilogue/block/block_epilogue_per_token_dequant.hpp:247-266) on their own, i.e.
 * cch_gmm_i8_dequant_swiglu before its SwiGLU:
 *   out[r,j] = bf16( float(acc) * per_ch[e,j] * per_tok[r] ), out bf16 [t,n];
 * operands and grouping as below.  Rows past sum(group_sizes) are written as zeros. */
int cch_gmm_i8_dequant(const void *x, const void *w, const int32_t *group_sizes, const float *per_tok, const float *per_ch,
                       void *out, int64_t num_experts, int64_t t, int64_t n, int64_t k, int trans_b, void *stream);
/* The same with a choice of output type (CCH_OUT_BF16 / CCH_OUT_FP16). */
int cch_gmm_i8_dequant_out(const void *x, const void *w, const int32_t *group_sizes, const float *per_tok, const float *per_ch,
                           void *out, int64_t num_experts, int64_t t, int64_t n, int64_t k, int trans_b, int out_dtype,
                           void *stream);

/* ---- MoE grouped W8A8 matmul + dequant + SwiGLU (config 4) -------------------
 * Replaces the grouped GEMM of AlltoallvGmmDequantKernel::operator()<AIC>
 * (include/catccos/dgemm/kernel/alltoallv_gmm_dequant_v2.hpp:164-244) and DequantSwigluKernel
 * (examples/aux_ops/group_dequant_swiglu.h:91-168), fused:
 *   rows of x are grouped by expert in expert order, group_sizes[e] rows each (device int32);
 *   c = float(acc) * per_ch[e,n] * per_tok[r];  out[r,j] = silu(c[j]) * c[j+n/2], j < n/2
 *   x int8 [t,k]; w int8 [E,k,n] (trans_b=0) or [E,n,k] (trans_b=1); per_ch fp32 [E,n];
 *   out bf16 [t,n/2].  Rows past sum(group_sizes) are written as zeros.
 * Every grouped entry point of this library takes 1 <= num_experts <= 256 (the kernels keep the
 * group table in LDS); more is CCH_EINVAL. */
int cch_gmm_i8_dequant_swiglu(const void *x, const void *w, const int32_t *group_sizes, const float *per_tok,
                              const float *per_ch, void *out, int64_t num_experts, int64_t t, int64_t n, int64_t k,
                              int trans_b, void *stream);
/* The same with a choice of output type (CCH_OUT_BF16 / CCH_OUT_FP16). */
int cch_gmm_i8_dequant_swiglu_out(const void *x, const void *w, const int32_t *group_sizes, const float *per_tok,
                                  const float *per_ch, void *out, int64_t num_experts, int64_t t, int64_t n, int64_t k,
                                  int trans_b, int out_dtype, void *stream);
/* The same with the activation leaving MX-quantised along its rows instead of as bf16: what
 * cch_mx_quant_rows (round to nearest even) makes of the bf16 output above, bit for bit, without the
 * bf16 tensor in between - the reference's SwiGLU-from-UB stage followed by its MX quantiser
 * (examples/aux_ops/ascend950_swiglu_from_ub.h:216-389,
 * include/catccos/comm/block/comm_block_mx_quant.hpp:213-266), as the input of the down-projection
 * MX grouped matmul.
 *   payload: codes of `fmt` (CCH_FMT_E4M3, CCH_FMT_E5M2; CCH_FMT_E2M1 two per byte), [t, n/2] elements;
 *   scales:  E8M0 [t, 2*ceil(n/2/64)], one per 32 columns, padding bytes 127.
 * Rows past sum(group_sizes) hold zero codes and scale bytes 127.  The tiled kernels take it when n/2 is
 * a multiple of 32 (besides their other conditions); other shapes run on the generic kernels. */
int cch_gmm_i8_dequant_swiglu_mx(const void *x, const void *w, const int32_t *group_sizes, const float *per_tok,
                                 const float *per_ch, void *payload, void *scales, int64_t num_experts, int64_t t, int64_t n,
                                 int64_t k, int trans_b, int fmt, void *stream);

/* ---- MX (FP8 / FP4 payload, E8M0 scales) dense GEMM (config 3) ---------------
 * Replaces the compute half of MatmulReduceScatterMxTla::operator()<AIC>
 * (include/catccos/dgemm/kernel/matmul_reduce_scatter_mx_tla.hpp:277-322), whose block MMAD
 * lives in the absent catlass submodule:
 *   out[m,n] = bf16( sum_k deq(a)[m,k] * deq(b)[k,n] ),  fp32 accumulation
 *   a payload [m,k] (FP4 [m,k/2]); sa [m, 2*ceil(k/64)];
 *   trans_b=0: b [k,n] (FP4 [k,n/2]), sb [ceil(k/64), n, 2]
 *   trans_b=1: b [n,k] (FP4 [n,k/2]), sb [n, 2*ceil(k/64)] */
int cch_mx_gemm(const void *a, const void *sa, const void *b, const void *sb, void *out, int64_t m, int64_t n, int64_t k,
                int fmt, int trans_b, void *stream);
/* The same with a choice of output type (CCH_OUT_BF16 / CCH_OUT_FP16; the reference's Ascend950 MX
 * matmul launchers are registered for fp16, e.g. LaunchAscend950Fp4MxMatmulReduceScatterFP16,
 * tests/dynamic_tiling/impl/kernel_fp16_ascend950.cpp:211). */
int cch_mx_gemm_out(const void *a, const void *sa, const void *b, const void *sb, void *out, int64_t m, int64_t n, int64_t k,
                    int fmt, int trans_b, int out_dtype, void *stream);

/* ---- MX grouped matmul over variable-size expert groups (config 5) -----------
 * Replaces the compute half of MxAllToAllVGroupedMatmulTla::operator()<AIC>
 * (include/catccos/dgemm/kernel/mx_alltoallv_group_matmul.hpp:265-316) and its tile scheduler
 * (include/catccos/dgemm/block/block_scheduler_alltoallv_allgather.hpp:27-233) with the
 * source-rank dimension collapsed: rows of a are grouped by expert, group_sizes[e] rows each
 * (device int32), b / sb hold num_experts operands back to back in the cch_mx_gemm layouts.
 * Rows past sum(group_sizes) are written as zeros. */
int cch_mx_gmm(const void *a, const void *sa, const void *b, const void *sb, const int32_t *group_sizes, void *out,
               int64_t num_experts, int64_t t, int64_t n, int64_t k, int fmt, int trans_b, void *stream);

/* ---- MX grouped matmul + SwiGLU: the up projection of the MX FFN chain ------
 * Replaces GMM1 and the SwiGLU stage of the Ascend950 dispatch-FFN-combine kernel
 * (examples/ascend950_dispatch_ffn_combine/ascend950_dispatch_ffn_combine_device.h:124-176: the up
 * projection writes a bf16 tile, Ascend950SwigluFromUbKernel turns its gate and up planes into the
 * activation, examples/aux_ops/ascend950_swiglu_from_ub.h:92-213; arithmetic of
 * include/catccos/epilogue/block/block_epilogue_regbase_swiglu.hpp:38-80):
 *   c = bf16(A_e x B_e) [t, n] per expert as cch_mx_gmm (columns [0, n/2) gate, [n/2, n) up);
 *   out[r, j] = bf16( g / (1 + exp(-g)) * u ) with g = c[r, j], u = c[r, j + n/2], in fp32
 * out [t, n/2] of out_dtype (CCH_OUT_BF16 / CCH_OUT_FP16); rows past sum(group_sizes) are zeros. */
int cch_mx_gmm_swiglu(const void *a, const void *sa, const void *b, const void *sb, const int32_t *group_sizes, void *out,
                      int64_t num_experts, int64_t t, int64_t n, int64_t k, int fmt, int trans_b, int out_dtype, void *stream);
/* The same with the activation leaving MX-quantised along its rows (Ascend950SwigluMxQuantFromUbKernel,
 * examples/aux_ops/ascend950_swiglu_from_ub.h:216-389): the bytes cch_mx_quant_rows (round to nearest
 * even) makes of the bf16 output above, as the input of the down projection (cch_mx_gmm_mapped).
 * payload / scales / out_fmt as cch_gmm_i8_dequant_swiglu_mx. */
int cch_mx_gmm_swiglu_mx(const void *a, const void *sa, const void *b, const void *sb, const int32_t *group_sizes, void *payload,
                         void *scales, int64_t num_experts, int64_t t, int64_t n, int64_t k, int fmt, int trans_b, int out_fmt,
                         void *stream);
/* The same reading its left-hand operand as the packed rows that cch_mx_quant_scatter_packed writes
 * ([payload | scales] per row, t rows of k (FP8) or ceil(k/2) (FP4) + 2*ceil(k/64) bytes): the dispatch
 * stage's buffer goes into the up projection as it is, as the reference's GMM1 reads its packed
 * operand (PackedMxTileCopyTlaToUB, examples/ascend950_dispatch_ffn_combine/
 * ascend950_dispatch_ffn_combine_device.h:118-122).  The tiled kernels take rows of a multiple of 4
 * bytes (every K that is a multiple of 64). */
int cch_mx_gmm_swiglu_mx_packed(const void *packed_a, const void *b, const void *sb, const int32_t *group_sizes, void *payload,
                                void *scales, int64_t num_experts, int64_t t, int64_t n, int64_t k, int fmt, int trans_b, int out_fmt,
                                void *stream);

/* ---- MXFP8 / MXFP4 grouped matmul with mapped output rows (down projection, config-5 twin) ----
 * Replaces the matmul half of GroupedMatmulAllToAllV for MX operands
 * (include/catccos/dgemm/kernel/grouped_matmul_alltoallv_mx.hpp:250 with the scheduler's RemapperC,
 * include/catccos/dgemm/block/block_scheduler_reducescatter_alltoallv.hpp:237-256; launched by
 * LaunchAscend950Fp8MxGroupedMatmulAllToAllVFP16, tests/dynamic_tiling/impl/kernel_fp16_ascend950.cpp:446):
 * the result rows leave in the order of the send buffer (by destination rank, then expert) instead of
 * the order of the tokens (by expert, then source rank).  Operands as cch_mx_gmm, plus
 *   out_row_map  int32 [t]: row of `out` that receives the result of row i of a; negative or
 *                >= out_rows = dropped.
 *                Entries of rows past sum(group_sizes) are ignored (those rows produce nothing).
 *                NULL: no mapping, out_rows == t, and the call is cch_mx_gmm with a choice of output
 *                type (rows past sum(group_sizes) zero-filled) - the fp16 launchers of the
 *                AllToAllVGroupedMatmul operators (tests/dynamic_tiling/include/launch_map.h:100-101).
 *   out          [out_rows, n] of out_dtype; rows that the map does not name are not written
 *   out_dtype    CCH_OUT_BF16, or CCH_OUT_FP16 (IEEE half, the type the reference registers these
 *                operators for); fp32 accumulators are rounded to nearest even either way
 * Destination rows must be distinct. */
int cch_mx_gmm_mapped(const void *a, const void *sa, const void *b, const void *sb, const int32_t *group_sizes,
                      const int32_t *out_row_map, void *out, int64_t out_rows, int out_dtype, int64_t num_experts, int64_t t,
                      int64_t n, int64_t k, int fmt, int trans_b, void *stream);

/* ---- MX quantisation scattered to the routed rows, packed (dispatch side of the MoE path) ----
 * Replaces CommBlockMxQuant::QuantScatterPacked (include/catccos/comm/block/
 * comm_block_mx_quant.hpp:319-369), called by the dispatch stage of
 * examples/ascend950_dispatch_ffn_combine/ascend950_dispatch_ffn_combine_device.h: every token
 * row is quantised once and the same packed row is written to each of its top_k destinations.
 *   x                 bf16 [tokens, k] row-major
 *   expanded_row_idx  int32 [tokens * top_k]: destination row of (token, route); negative = skip
 *   packed_out        bytes [rows, payload_bytes + scale_bytes]: payload_bytes = k (FP8) or
 *                     ceil(k/2) (FP4), scale_bytes = 2*ceil(k/64) E8M0 bytes (a padding entry is
 *                     127); rows that no route names are not touched
 *   top_k             0..8; fmt / rounding as cch_mx_quant_rows
 * Destination rows must be distinct (two routes writing one row race, as in the reference). */
int cch_mx_quant_scatter_packed(const void *x, const int32_t *expanded_row_idx, void *packed_out, int64_t tokens,
                                int64_t k, int top_k, int fmt, int rounding, void *stream);
/* The same with the number of rows of packed_out stated: an entry of expanded_row_idx at or past
 * out_rows is skipped like a negative one instead of being written outside the buffer (a caller that
 * cannot vouch for its routing table needs no pass over it on the host). */
int cch_mx_quant_scatter_packed_rows(const void *x, const int32_t *expanded_row_idx, void *packed_out, int64_t out_rows,
                                     int64_t tokens, int64_t k, int top_k, int fmt, int rounding, void *stream);

/* ---- MoE token un-permute (combine side of the MoE path) ----
 * Replaces KernelMoeTokenUnpermute (examples/aux_ops/moe_token_unpermute/
 * moe_token_unpermute.h:235-355), the last stage of DispatchFFNCombine
 * (examples/dispatch_ffn_combine/dispatch_ffn_combine_device.h:886-898).
 *   permuted_tokens  bf16 [rows, hidden]: expert outputs in the expert-sorted row order
 *   sorted_indices   int32 [tokens * top_k]: row of permuted_tokens that holds route j of token t;
 *                    an entry outside [0, rows) contributes nothing
 *   probs            fp32 [tokens * top_k] routing weights, or NULL for an unweighted sum
 *   out              bf16 [tokens, hidden] = sum_j permuted[sorted_indices[t,j]] * probs[t,j]: fp32,
 *                    each product rounded before it is added, routes in order, route 0 assigns;
 *                    rounded to nearest even
 *   top_k            1..8 */
int cch_moe_token_unpermute(const void *permuted_tokens, const int32_t *sorted_indices, const float *probs, void *out,
                            int64_t rows, int64_t tokens, int64_t hidden, int top_k, void *stream);

/* ---- MoE routing: stable sort of the (token, route) list by expert ----
 * Replaces the sort stage of moe_init_routing_quant_v2 (examples/aux_ops/moe_init_routing_quant_v2/
 * moe_init_routing_quant_v2.h:70-110 with moe_v2_src_to_dst_op.h and moe_v2_expert_token_out.h;
 * CPU stand-in examples/utils/gen_data_moe.py:48-57).
 *   expert_idx     int32 [rows]: expert of flat entry token * top_k + route; an entry outside
 *                  [0, num_experts) is dropped
 *   dst_to_src     int32 [rows]: flat entry at sorted position i (experts ascending, ties in flat
 *                  order), -1 past the routed entries; this is the src_rows of cch_dyn_quant_i8_rows
 *   src_to_dst     int32 [rows]: sorted position of flat entry i, -1 if dropped; this is the
 *                  sorted_indices of cch_moe_token_unpermute and the expanded_row_idx the reference's
 *                  operator returns
 *   expert_tokens  int32 [num_experts]: entries per expert, or their running sum with cumsum != 0
 *   workspace      device memory of at least cch_moe_init_routing_workspace_bytes(rows, num_experts)
 * num_experts <= 1024.  Up to 8192 rows and 256 experts the sort is one launch of one workgroup (the
 * workspace is then not touched), three launches otherwise; the results are the same integers. */
int64_t cch_moe_init_routing_workspace_bytes(int64_t rows, int num_experts);
int cch_moe_init_routing(const int32_t *expert_idx, int64_t rows, int num_experts, int32_t *dst_to_src, int32_t *src_to_dst,
                         int32_t *expert_tokens, int cumsum, void *workspace, int64_t workspace_bytes, void *stream);

/* cch_moe_init_routing for callers that cannot allocate device memory (code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc).  No counterpart in the
 * reference.  Same arguments and results minus the workspace: the histogram area is a 1 MiB array
 * inside the library's device image (one copy per GPU, held until the process ends), whose
 * address is looked up once per device by cch_init or by the first call on that device.  The call
 * itself allocates and frees nothing.
 *   limit   ceil(rows / 1024) * num_experts <= CCH_ROUTING_NOALLOC_MAX_ENTRIES (e.g. 262144 rows
 *           over 1024 experts, or 8 Mi rows over 32); larger requests return CCH_EINVAL.
 *   sharing every call on a GPU uses that GPU's one array: calls that overlap on one GPU (two
 *           streams, two threads) race; calls in stream order do not.  Nothing in the array has to
 *           be cleared between calls (each call writes every entry it later reads).  Inputs that
 *           one workgroup sorts (up to 8192 rows and 256 experts) do not touch the array at all. */
#define CCH_ROUTING_NOALLOC_MAX_ENTRIES 262144
int cch_moe_init_routing_noalloc(const int32_t *expert_idx, int64_t rows, int num_experts, int32_t *dst_to_src,
                                 int32_t *src_to_dst, int32_t *expert_tokens, int cumsum, void *stream);

/* ---- Per-token dynamic int8 quantisation with row gather (feeds config 4) ----
 * Replaces MoeV2GatherDynamicQuant (examples/aux_ops/moe_init_routing_quant_v2/
 * moe_v2_gather_dynamic_quant.h:117-150 Compute, :213-250 the gather loop).
 *   x         bf16 [rows_in, k] row-major
 *   src_rows  int32 [t] or NULL: output row i quantises input row src_rows[i] / topk
 *             (the reference's sorted expanded-row index divided by top-K); a negative
 *             entry or one past the input gives a zero row with scale 0.  NULL: row i.
 *   q         int8 [t, k];  scale  fp32 [t] = amax(row) / 127 (0 for an all-zero row)
 *   mode      CCH_DQ_DEVICE: y = x / scale in fp32, truncated to half, rounded to the nearest
 *             integer with halves away from zero (the reference kernel's casts);
 *             CCH_DQ_GOLDEN: rint(x * 127 / amax), ties to even (the reference's Python
 *             golden, examples/utils/gen_data_dispatch_gmm_dequant_swiglu.py:275-280). */
#define CCH_DQ_DEVICE 0
#define CCH_DQ_GOLDEN 1
int cch_dyn_quant_i8_rows(const void *x, const int32_t *src_rows, void *q, float *scale, int64_t rows_in, int64_t t,
                          int64_t k, int topk, int mode, void *stream);
/* The same with the reference's smoothing (quantSmooth, moe_v2_gather_dynamic_quant.h:127-130): every
 * element is multiplied in fp32 by its column's entry of a smoothing vector before the maximum is taken.
 *   smooth       fp32 [num_smooth, k]
 *   smooth_rows  int32 [t] or NULL: output row i uses vector smooth_rows[i] (the row's expert, the
 *                reference's smoothType 2, :241); an index outside [0, num_smooth) gives a zero row
 *                with scale 0.  NULL: vector 0 for every row (smoothType 1, :170-174). */
int cch_dyn_quant_i8_rows_smooth(const void *x, const int32_t *src_rows, const float *smooth, const int32_t *smooth_rows,
                                 int64_t num_smooth, void *q, float *scale, int64_t rows_in, int64_t t, int64_t k, int topk,
                                 int mode, void *stream);

/* Library switches for tests and benchmarks.  They are process-wide (one atomic each, read at
 * every call): two callers that want different settings at the same time race; set them once, or
 * from one thread between calls.  "force_generic_gemm" = 1 routes every GEMM entry
 * point through the shape-agnostic one-thread-per-element kernels instead of the tiled MFMA
 * kernels; "require_tiled_gemm" = 1 makes a GEMM entry point return CCH_ENOSUP instead of
 * falling back to them when the tiled kernels do not take the problem; "gemm_tile_order" picks the
 * order in which the persistent workgroups of the tiled kernels walk the output tiles: 0 = row-major
 * over (row tile, column tile), 1 = each XCD takes a run of consecutive tiles of every round (whole
 * row tiles next to each other: fewer token and weight panels per L2), 2 = each XCD takes a block of
 * 4 row tiles x 8 column tiles of every round (where 8, 16, 32 or 64 column tiles and 256 workgroups
 * allow it; else 1 for grouped problems and 0 for dense ones), -1 (default) = 2;
 * "i8_epilogue_fp16_step" = 1 makes the int8 epilogues (cch_gemm_i8_dequant*, cch_gmm_i8_dequant*, both kernel paths)
 * round acc * per_channel to IEEE half before the per-token factor, as the reference's device kernel does
 * (include/catccos/epilogue/block/block_epilogue_per_token_dequant_swiglu.hpp:348-361: the matrix unit's output stage
 * writes fp16, the vector epilogue widens it; the golden generator's option,
 * examples/utils/gen_data_dispatch_gmm_dequant_swiglu.py:309-310); 0 (default) keeps fp32 throughout, the golden
 * generator's default path - this one switch does change results, by at most 2^-11 relative;
 * "gemm_nt_output" = 1 / 0 gives or denies the output stores the non-temporal hint, -1 (default) gives it to the MXFP4 kernels, where it measured
 * 3-4 % faster (no difference for the others); "quant_integer_encoder" = 1 runs the E4M3
 * round-to-nearest-even quantiser through the integer encoder instead of the hardware conversion (an
 * on-device cross-check; same bytes).  Results depend on none of them but "i8_epilogue_fp16_step".
 * The tiled MFMA kernels take every problem whose rows of K are a multiple of 16 bytes, with
 * n % 8 == 0 (and, for [K,N] operands, rows of B a multiple of 4 bytes), 16-byte aligned operands
 * below 2 GiB each and MX scale arrays back to back.  The generic kernels take everything else.
 * When a GEMM entry point falls back from the tiled MFMA kernels to the one-thread-per-element
 * kernels (orders of magnitude slower), the call still returns CCH_OK, cch_last_error() names the
 * precondition that failed, and the first such call of the process prints one line to stderr.  Every
 * GEMM entry point empties the calling thread's message when it starts, so after CCH_OK the message is
 * either that note of this very call or empty. */
int cch_set_option(const char *name, int value);

#ifdef __cplusplus
}
#endif
#endif /* CATCCOS_HIP_H */
