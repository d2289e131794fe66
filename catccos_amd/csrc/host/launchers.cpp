// Launch<Op><DType> functions with the reference's KernelFuncPtr signature
// (tests/dynamic_tiling/include/launch_map.h:15-16; bodies there: impl/kernel_int8.cpp:113-130,
// impl/kernel_mxfp_ascend950.cpp:19, impl/kernel_fp16_ascend950.cpp:592-612).  Each one maps the
// KernelParams pointer roles of its operator onto the kernel's Arguments and runs it through the
// device-operator facade like the reference's bodies do (Arguments -> Initialize -> Run, which
// synchronises the stream, include/catccos/dgemm/device/device_dgemm.hpp:89-120); the launchers of
// the dispatch / combine additions call the C ABI directly and synchronise the same way.
#include "device_dgemm.h"
#include "launch_map.h"

using namespace Catccos;
using Catccos::DGemm::Device::DeviceDGemm;
namespace K = Catccos::DGemm::Kernel;

namespace {
void Finish(int rc, void *stream, const char *what)
{
    if (rc != CCH_OK) fprintf(stderr, "%s: cchError:%d %s\n", what, rc, cch_last_error());
    CCH_CHECK(cch_stream_sync(stream));
}
inline GM_ADDR Gm(void *p) { return static_cast<GM_ADDR>(p); }
template <class Kernel> void RunOp(const typename Kernel::Arguments &args, void *stream, uint32_t blockNum, uint64_t fftsAddr,
                                   uint8_t *workSpace)
{
    DeviceDGemm<Kernel> op;
    op.Initialize(args, workSpace);
    op.Run(stream, blockNum, fftsAddr);
}
struct AutoRegister {
    AutoRegister(CocCommType type, CocDataType dtype, KernelFuncPtr fn) { KernelDispatcher::RegisterKernelFunc(type, dtype, fn); }
};
}  // namespace

void LaunchAscend950BF16QuantAllGatherFP8E4M3FN(void *stream, uint32_t blockNum, uint64_t fftsAddr, KernelParams &p,
                                                uint8_t *workSpace, uint8_t *symmetricPtr, CocTilingParams &t, uint32_t, uint32_t)
{
    K::MxQuantAllGather::Arguments args{};
    args.problemShape = MatrixCoord{t.m, t.n};
    args.rankIdx = 0;
    args.rankSize = t.rankSize;
    args.ptrInput = Gm(p.ptrA);
    args.ptrOutput = Gm(p.ptrC);
    args.ptrMxScale = Gm(p.ptrB);
    args.ptrSymmetric = symmetricPtr;
    RunOp<K::MxQuantAllGather>(args, stream, blockNum, fftsAddr, workSpace);
}

void LaunchAllGatherMatmulDequantINT8(void *stream, uint32_t blockNum, uint64_t fftsAddr, KernelParams &p, uint8_t *workSpace,
                                      uint8_t *symmetricPtr, CocTilingParams &t, uint32_t, uint32_t transB)
{
    K::AllGatherMatmulDequant::Arguments args{};
    args.problemShape = GemmCoord{t.m, t.n, t.k};
    args.rankSize = t.rankSize;
    args.commInterval = t.commInterval;
    args.ptrA = Gm(p.ptrA);
    args.ptrB = Gm(p.ptrB);
    args.ptrD = Gm(p.ptrC);
    args.ptrScale = Gm(p.customPtrs[0]);
    args.ptrPerToken = Gm(p.customPtrs[1]);
    args.ptrWB = workSpace;
    args.ptrSymmetric = symmetricPtr;
    args.transB = transB;
    RunOp<K::AllGatherMatmulDequant>(args, stream, blockNum, fftsAddr, workSpace);
}

void LaunchAscend950MxFp8MatmulReduceScatterFP8E4M3FN(void *stream, uint32_t blockNum, uint64_t fftsAddr, KernelParams &p,
                                                      uint8_t *workSpace, uint8_t *symmetricPtr, CocTilingParams &t, uint32_t,
                                                      uint32_t transB)
{
    K::MatmulReduceScatterMx::Arguments args{};
    args.problemShape = GemmCoord{t.m, t.n, t.k};
    args.rankSize = t.rankSize;
    args.commInterval = t.commInterval;
    args.ptrA = Gm(p.ptrA);
    args.ptrB = Gm(p.ptrB);
    args.ptrMxScaleA = Gm(p.customPtrs[0]);
    args.ptrMxScaleB = Gm(p.customPtrs[1]);
    args.ptrD = Gm(p.ptrC);
    args.ptrSymmetric = symmetricPtr;
    args.format = CCH_FMT_E4M3;
    args.transB = transB;
    RunOp<K::MatmulReduceScatterMx>(args, stream, blockNum, fftsAddr, workSpace);
}

void LaunchDispatchGmmDequantSwigluINT8(void *stream, uint32_t, uint64_t, KernelParams &p, uint8_t *, uint8_t *,
                                        CocTilingParams &t, uint32_t, uint32_t transB)
{
    if (p.customCount >= 6) {
        // from bf16 tokens: routing sort, dynamic int8 quantisation with the expert-sorted gather, grouped matmul
        const int64_t topK = t.topK ? t.topK : 1, rows = (int64_t)t.m * topK;
        int rc = cch_moe_init_routing(reinterpret_cast<const int32_t *>(p.customPtrs[1]), rows, (int)t.expertNum,
                                      reinterpret_cast<int32_t *>(p.customPtrs[4]), reinterpret_cast<int32_t *>(p.customPtrs[6]),
                                      reinterpret_cast<int32_t *>(p.customPtrs[3]), 0, p.customPtrs[7],
                                      cch_moe_init_routing_workspace_bytes(rows, (int)t.expertNum), stream);
        if (rc == CCH_OK)
            rc = cch_dyn_quant_i8_rows(p.ptrA, reinterpret_cast<const int32_t *>(p.customPtrs[4]), p.customPtrs[5],
                                       reinterpret_cast<float *>(p.customPtrs[2]), t.m, rows, t.k, (int)topK, CCH_DQ_DEVICE, stream);
        if (rc == CCH_OK)
            rc = cch_gmm_i8_dequant_swiglu(p.customPtrs[5], p.ptrB, reinterpret_cast<const int32_t *>(p.customPtrs[3]),
                                           reinterpret_cast<const float *>(p.customPtrs[2]),
                                           reinterpret_cast<const float *>(p.customPtrs[0]), p.ptrC, t.expertNum, rows, t.n, t.k,
                                           (int)transB, stream);
        Finish(rc, stream, "DispatchGmmDequantSwiglu");
        return;
    }
    K::AlltoallvGmmDequantSwiglu::Arguments args{};
    args.problemShape = GemmCoord{t.m, t.n, t.k};
    args.EP = 1;
    args.expertPerRank = (int32_t)t.expertNum;
    args.rankSize = t.rankSize;
    args.ptrA = Gm(p.ptrA);
    args.ptrB = Gm(p.ptrB);
    args.ptrC = Gm(p.ptrC);
    args.ptrScale = Gm(p.customPtrs[0]);
    args.ptrTokenPerExpert = Gm(p.customPtrs[1]);
    args.ptrPerTokenScale = Gm(p.customPtrs[2]);
    args.transB = transB;
    RunOp<K::AlltoallvGmmDequantSwiglu>(args, stream, 0, 0, nullptr);
}

// Up projection (Arguments as in tests/dynamic_tiling/impl/kernel_fp16_ascend950.cpp:592-612).  The
// reference registers these operators for fp16 output (launch_map.h:100-101); this build has that
// launcher and a bf16 twin.
static void MxAllToAllVGroupedMatmul(void *stream, uint32_t blockNum, uint64_t fftsAddr, KernelParams &p, uint8_t *workSpace,
                                     uint8_t *symmetricPtr, CocTilingParams &t, uint32_t transB, int fmt, bool fp16)
{
    K::MxAllToAllVGroupMatmul::Arguments args{};
    args.gemmShape = GemmCoord{t.m, t.n, t.k};
    args.rankSize = t.rankSize;
    args.commInterval = t.commInterval;
    args.epSize = 1;                 // the experts of this call are this rank's
    args.expertNum = t.expertNum;
    args.ptrA = Gm(p.ptrA);
    args.ptrB = Gm(p.ptrB);
    args.ptrC = Gm(p.ptrC);
    args.ptrMxScaleA = Gm(p.customPtrs[0]);
    args.ptrMxScaleB = Gm(p.customPtrs[1]);
    args.ptrLocalTokensPerExpert = Gm(p.customPtrs[2]);
    args.ptrGlobalTokensPerLocalExpert = Gm(p.customPtrs[3]);
    args.ptrSymmetric = symmetricPtr;
    args.format = fmt;
    args.transB = transB;
    args.outFp16 = fp16;
    RunOp<K::MxAllToAllVGroupMatmul>(args, stream, blockNum, fftsAddr, workSpace);
}

void LaunchAscend950Fp4MxAllToAllVGroupedMatmulBF16(void *stream, uint32_t blockNum, uint64_t fftsAddr, KernelParams &p,
                                                    uint8_t *workSpace, uint8_t *symmetricPtr, CocTilingParams &t, uint32_t,
                                                    uint32_t transB)
{
    MxAllToAllVGroupedMatmul(stream, blockNum, fftsAddr, p, workSpace, symmetricPtr, t, transB, CCH_FMT_E2M1, false);
}

void LaunchAscend950Fp8MxAllToAllVGroupedMatmulBF16(void *stream, uint32_t blockNum, uint64_t fftsAddr, KernelParams &p,
                                                    uint8_t *workSpace, uint8_t *symmetricPtr, CocTilingParams &t, uint32_t,
                                                    uint32_t transB)
{
    MxAllToAllVGroupedMatmul(stream, blockNum, fftsAddr, p, workSpace, symmetricPtr, t, transB, CCH_FMT_E4M3, false);
}

void LaunchAscend950Fp4MxAllToAllVGroupedMatmulFP16(void *stream, uint32_t blockNum, uint64_t fftsAddr, KernelParams &p,
                                                    uint8_t *workSpace, uint8_t *symmetricPtr, CocTilingParams &t, uint32_t,
                                                    uint32_t transB)
{
    MxAllToAllVGroupedMatmul(stream, blockNum, fftsAddr, p, workSpace, symmetricPtr, t, transB, CCH_FMT_E2M1, true);
}

void LaunchAscend950Fp8MxAllToAllVGroupedMatmulFP16(void *stream, uint32_t blockNum, uint64_t fftsAddr, KernelParams &p,
                                                    uint8_t *workSpace, uint8_t *symmetricPtr, CocTilingParams &t, uint32_t,
                                                    uint32_t transB)
{
    MxAllToAllVGroupedMatmul(stream, blockNum, fftsAddr, p, workSpace, symmetricPtr, t, transB, CCH_FMT_E4M3, true);
}

// Down projection.  The reference registers these two operators for fp16 output only
// (tests/dynamic_tiling/impl/kernel_fp16_ascend950.cpp:446-485, launch_map.h:98-99); this build has
// that launcher and a bf16 twin, which the driver uses by default like for every other operator.
static void MxGroupedMatmulAllToAllV(void *stream, KernelParams &p, CocTilingParams &t, uint32_t transB, int fmt, int outDtype,
                                     const char *what)
{
    const int64_t ranks = t.rankSize ? t.rankSize : 1, experts = t.expertNum / (t.epSize ? t.epSize : 1);
    Finish(cch_mx_gmm_mapped(p.ptrA, p.customPtrs[0], p.ptrB, p.customPtrs[1], reinterpret_cast<const int32_t *>(p.customPtrs[4]),
                             reinterpret_cast<const int32_t *>(p.customPtrs[5]), p.ptrC, ranks * t.m, outDtype, experts, t.m, t.n,
                             t.k, fmt, (int)transB, stream),
           stream, what);
}

void LaunchAscend950Fp8MxGroupedMatmulAllToAllVBF16(void *stream, uint32_t, uint64_t, KernelParams &p, uint8_t *, uint8_t *,
                                                    CocTilingParams &t, uint32_t, uint32_t transB)
{
    MxGroupedMatmulAllToAllV(stream, p, t, transB, CCH_FMT_E4M3, CCH_OUT_BF16, "Ascend950Fp8MxGroupedMatmulAllToAllV");
}

void LaunchAscend950Fp4MxGroupedMatmulAllToAllVBF16(void *stream, uint32_t, uint64_t, KernelParams &p, uint8_t *, uint8_t *,
                                                    CocTilingParams &t, uint32_t, uint32_t transB)
{
    MxGroupedMatmulAllToAllV(stream, p, t, transB, CCH_FMT_E2M1, CCH_OUT_BF16, "Ascend950Fp4MxGroupedMatmulAllToAllV");
}

void LaunchAscend950Fp8MxGroupedMatmulAllToAllVFP16(void *stream, uint32_t, uint64_t, KernelParams &p, uint8_t *, uint8_t *,
                                                    CocTilingParams &t, uint32_t, uint32_t transB)
{
    MxGroupedMatmulAllToAllV(stream, p, t, transB, CCH_FMT_E4M3, CCH_OUT_FP16, "Ascend950Fp8MxGroupedMatmulAllToAllV");
}

void LaunchAscend950Fp4MxGroupedMatmulAllToAllVFP16(void *stream, uint32_t, uint64_t, KernelParams &p, uint8_t *, uint8_t *,
                                                    CocTilingParams &t, uint32_t, uint32_t transB)
{
    MxGroupedMatmulAllToAllV(stream, p, t, transB, CCH_FMT_E2M1, CCH_OUT_FP16, "Ascend950Fp4MxGroupedMatmulAllToAllV");
}

// The MXFP8 FFN of one rank, the stages of the reference's single kernel
// (examples/ascend950_dispatch_ffn_combine/ascend950_dispatch_ffn_combine_device.h:124-176: routing sort, MX quantisation
// into the dispatch rows, GMM1, SwiGLU + MX quantisation, GMM2, weighted un-permute) as five launches on one
// stream with no host round trip: the packed rows feed GMM1 in place, GMM1 hands over MXFP8 payload and scales.
// Pointer roles: see Ascend950DispatchFFNCombineOperator.  The weight files hold W transposed ([E,n,k]) whatever
// the transB argument says (the reference passes weightNz = 1, transB = 0 for them, scripts/run.sh:92).
void LaunchAscend950DispatchFFNCombineBF16(void *stream, uint32_t, uint64_t, KernelParams &p, uint8_t *, uint8_t *, CocTilingParams &t,
                                           uint32_t, uint32_t)
{
    const int64_t topK = t.topK ? t.topK : 1, rows = (int64_t)t.m * topK, e = t.expertNum, k = t.k, n = t.n;
    if (p.customCount < 13) {
        Finish(CCH_EINVAL, stream, "Ascend950DispatchFFNCombine (buffers not allocated by its operator)");
        return;
    }
    auto i32 = [&](int i) { return reinterpret_cast<int32_t *>(p.customPtrs[i]); };
    int rc = cch_moe_init_routing(i32(1), rows, (int)e, i32(6), i32(5), i32(7), 0, p.customPtrs[12],
                                  cch_moe_init_routing_workspace_bytes(rows, (int)e), stream);
    if (rc == CCH_OK)
        rc = cch_mx_quant_scatter_packed_rows(p.ptrA, i32(5), p.customPtrs[8], rows, t.m, k, (int)topK, CCH_FMT_E4M3, CCH_ROUND_RNE, stream);
    if (rc == CCH_OK)
        rc = cch_mx_gmm_swiglu_mx_packed(p.customPtrs[8], p.ptrB, p.customPtrs[3], i32(7), p.customPtrs[9], p.customPtrs[10], e, rows, n, k,
                                         CCH_FMT_E4M3, 1, CCH_FMT_E4M3, stream);
    if (rc == CCH_OK)
        rc = cch_mx_gmm(p.customPtrs[9], p.customPtrs[10], p.customPtrs[0], p.customPtrs[4], i32(7), p.customPtrs[11], e, rows, k, n / 2,
                        CCH_FMT_E4M3, 1, stream);
    if (rc == CCH_OK)
        rc = cch_moe_token_unpermute(p.customPtrs[11], i32(5), reinterpret_cast<const float *>(p.customPtrs[2]), p.ptrC, rows, t.m, k,
                                     (int)topK, stream);
    Finish(rc, stream, "Ascend950DispatchFFNCombine");
}

static AutoRegister s_reg0(MX_QUANT_ALLGATHER, FP8E4M3FN, &LaunchAscend950BF16QuantAllGatherFP8E4M3FN);
static AutoRegister s_reg1(ALLGATHER_MATMUL_DEQUANT, INT8, &LaunchAllGatherMatmulDequantINT8);
static AutoRegister s_reg2(ASCEND950_MXFP8_MATMUL_REDUCE_SCATTER, FP8E4M3FN, &LaunchAscend950MxFp8MatmulReduceScatterFP8E4M3FN);
static AutoRegister s_reg3(DISPATCH_GMM_DEQUANT_SWIGLU, INT8, &LaunchDispatchGmmDequantSwigluINT8);
static AutoRegister s_reg4(ASCEND950_FP4_MX_ALLTOALLV_GROUPED_MATMUL, BF16, &LaunchAscend950Fp4MxAllToAllVGroupedMatmulBF16);
static AutoRegister s_reg5(ASCEND950_FP8_MX_ALLTOALLV_GROUPED_MATMUL, BF16, &LaunchAscend950Fp8MxAllToAllVGroupedMatmulBF16);
static AutoRegister s_reg6(ASCEND950_FP8_MX_GROUPED_MATMUL_ALLTOALLV, BF16, &LaunchAscend950Fp8MxGroupedMatmulAllToAllVBF16);
static AutoRegister s_reg7(ASCEND950_FP4_MX_GROUPED_MATMUL_ALLTOALLV, BF16, &LaunchAscend950Fp4MxGroupedMatmulAllToAllVBF16);
static AutoRegister s_reg8(ASCEND950_FP8_MX_GROUPED_MATMUL_ALLTOALLV, FP16, &LaunchAscend950Fp8MxGroupedMatmulAllToAllVFP16);
static AutoRegister s_reg9(ASCEND950_FP4_MX_GROUPED_MATMUL_ALLTOALLV, FP16, &LaunchAscend950Fp4MxGroupedMatmulAllToAllVFP16);
static AutoRegister s_reg10(ASCEND950_FP4_MX_ALLTOALLV_GROUPED_MATMUL, FP16, &LaunchAscend950Fp4MxAllToAllVGroupedMatmulFP16);
static AutoRegister s_reg11(ASCEND950_FP8_MX_ALLTOALLV_GROUPED_MATMUL, FP16, &LaunchAscend950Fp8MxAllToAllVGroupedMatmulFP16);
static AutoRegister s_reg12(ASCEND950_DISPATCH_FFN_COMBINE, BF16, &LaunchAscend950DispatchFFNCombineBF16);
