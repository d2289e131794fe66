// Device-operator facade: DeviceDGemm<Kernel> with GetWorkspaceSize / Initialize / Run, the
// interface the reference's launchers drive (include/catccos/dgemm/device/device_dgemm.hpp:50-126:
// Arguments -> Initialize(args, workspace) stores the kernel's Params, Run(stream, blockDim,
// fftsAddr) launches and synchronises the stream).  A Kernel here is a plain host struct with
// the reference's `Arguments` (pointers + GemmCoord / MatrixCoord, field names as in the cited
// headers), a `Params` it is lowered to, and a `Launch` that makes one C-ABI call.  Fields of
// the dropped communication half (rankIdx, rankSize, commInterval, ptrSymmetric, comm*Shape)
// are carried so that reference launcher bodies compile unchanged; only rankSize is looked at.
#ifndef CATCCOS_HOST_DEVICE_DGEMM_H
#define CATCCOS_HOST_DEVICE_DGEMM_H

#include <cstddef>
#include <cstdint>

#include "catccos_hip.h"
#include "utils.h"

namespace Catccos {

using GM_ADDR = uint8_t *;

// catlass's coordinate helpers, as far as Arguments need them
struct GemmCoord {
    uint32_t coord[3];
    GemmCoord(uint32_t m = 0, uint32_t n = 0, uint32_t k = 0) : coord{m, n, k} {}
    uint32_t m() const { return coord[0]; }
    uint32_t n() const { return coord[1]; }
    uint32_t k() const { return coord[2]; }
};
struct MatrixCoord {
    uint32_t coord[2];
    MatrixCoord(uint32_t row = 0, uint32_t column = 0) : coord{row, column} {}
    uint32_t row() const { return coord[0]; }
    uint32_t column() const { return coord[1]; }
};

enum class Status { kSuccess = 0, kErrorInvalidProblem, kErrorInternal };

namespace DGemm {
namespace Kernel {

// The local quantisation of one rank's [rows, columns] bf16 input.  The reference starts this
// kernel directly, MxQuantAllGather<...><<<blockNum, nullptr, stream>>>(fftsAddr, ptrA, ptrC, ptrB,
// symmetricPtr, cocTiling, 10) (tests/dynamic_tiling/impl/kernel_mxfp_ascend950.cpp:19-30); here it
// takes the same three calls as the matmul kernels.
struct MxQuantAllGather {
    struct Arguments {
        MatrixCoord problemShape;   // rows, columns of the local input
        uint32_t rankIdx, rankSize;
        GM_ADDR ptrInput, ptrOutput, ptrMxScale, ptrSymmetric;
        int format = CCH_FMT_E4M3, rounding = CCH_ROUND_RNE;
    };
    using Params = Arguments;
    static size_t GetWorkspaceSize(const Arguments &) { return 0; }
    static Params ToUnderlyingArguments(const Arguments &args, uint8_t * = nullptr) { return args; }
    static int Launch(const Params &p, void *stream)
    {
        return cch_mx_quant_rows(p.ptrInput, p.ptrOutput, p.ptrMxScale, p.problemShape.row(), p.problemShape.column(), p.format,
                                 p.rounding, stream);
    }
};

// include/catccos/dgemm/kernel/allgather_matmul_dequant.hpp:129-143.  problemShape.m is the local
// row count; ptrPerToken is this build's per-token scale vector (the reference's build adds it).
struct AllGatherMatmulDequant {
    struct Arguments {
        GemmCoord problemShape;
        uint32_t rankIdx, rankSize, commInterval;
        GM_ADDR ptrA, ptrB, ptrD, ptrScale, ptrWB, ptrSymmetric;
        MatrixCoord commCoreSplit, commBlockShape, commTileShape;
        GM_ADDR ptrPerToken = nullptr;
        uint32_t transB = 0;
    };
    using Params = Arguments;
    static size_t GetWorkspaceSize(const Arguments &) { return 0; }   // no padded copy of B on this path
    static Params ToUnderlyingArguments(const Arguments &args, uint8_t * = nullptr) { return args; }
    static int Launch(const Params &p, void *stream)
    {
        return cch_gemm_i8_dequant(p.ptrA, p.ptrB, reinterpret_cast<const float *>(p.ptrPerToken),
                                   reinterpret_cast<const float *>(p.ptrScale), p.ptrD, p.problemShape.m(), p.problemShape.n(),
                                   p.problemShape.k(), (int)p.transB, stream);
    }
};

// include/catccos/dgemm/kernel/matmul_reduce_scatter_mx_tla.hpp:128-142 (problemShape.m is the
// total row count of the local GEMM: on one rank the reduce-scatter keeps all of them).
struct MatmulReduceScatterMx {
    struct Arguments {
        GemmCoord problemShape;
        uint32_t rankIdx, rankSize, commInterval;
        GM_ADDR ptrA, ptrB, ptrMxScaleA, ptrMxScaleB, ptrD, ptrSymmetric;
        MatrixCoord commCoreSplit, commBlockShape, commTileShape;
        int format = CCH_FMT_E4M3;
        uint32_t transB = 0;
    };
    using Params = Arguments;
    static size_t GetWorkspaceSize(const Arguments &) { return 0; }
    static Params ToUnderlyingArguments(const Arguments &args, uint8_t * = nullptr) { return args; }
    static int Launch(const Params &p, void *stream)
    {
        return cch_mx_gemm(p.ptrA, p.ptrMxScaleA, p.ptrB, p.ptrMxScaleB, p.ptrD, p.problemShape.m(), p.problemShape.n(),
                           p.problemShape.k(), p.format, (int)p.transB, stream);
    }
};

// The grouped int8 matmul of AlltoallvGmmDequantKernel (fields named as its Params,
// include/catccos/dgemm/kernel/alltoallv_gmm_dequant_v2.hpp:93-115) fused with the SwiGLU pass of
// examples/aux_ops/group_dequant_swiglu.h: int8 tokens already grouped by expert, tokens per
// local expert and per-token scales on the device (inputs here; the reference's kernel produces
// the scales while it dispatches).  ptrC receives the bf16 [m, n/2] result, not int32 partials.
struct AlltoallvGmmDequantSwiglu {
    struct Arguments {
        GemmCoord problemShape;     // m = rows received, n = gate + up columns, k
        int32_t EP, expertPerRank;
        uint32_t rank, rankSize;
        GM_ADDR ptrA, ptrB, ptrC, ptrScale, ptrPerTokenScale, ptrTokenPerExpert, symmetricPtr;
        uint32_t transB = 0;
    };
    using Params = Arguments;
    static size_t GetWorkspaceSize(const Arguments &) { return 0; }   // no [T, N] intermediate: the epilogue is fused
    static Params ToUnderlyingArguments(const Arguments &args, uint8_t * = nullptr) { return args; }
    static int Launch(const Params &p, void *stream)
    {
        return cch_gmm_i8_dequant_swiglu(p.ptrA, p.ptrB, reinterpret_cast<const int32_t *>(p.ptrTokenPerExpert),
                                         reinterpret_cast<const float *>(p.ptrPerTokenScale),
                                         reinterpret_cast<const float *>(p.ptrScale), p.ptrC, p.expertPerRank, p.problemShape.m(),
                                         p.problemShape.n(), p.problemShape.k(), (int)p.transB, stream);
    }
};

// include/catccos/dgemm/kernel/mx_alltoallv_group_matmul.hpp:135-152.  gemmShape.m is the row
// count of A; expertNum / epSize local experts; ptrGlobalTokensPerLocalExpert holds one count per
// local expert on a single rank.  outFp16 selects IEEE half output (the type the reference
// registers these operators for).
struct MxAllToAllVGroupMatmul {
    struct Arguments {
        GemmCoord gemmShape;
        uint32_t rankIdx, rankSize, commInterval, epSize, expertNum;
        GM_ADDR ptrA, ptrB, ptrC, ptrMxScaleA, ptrMxScaleB, ptrLocalTokensPerExpert, ptrGlobalTokensPerLocalExpert, ptrSymmetric;
        MatrixCoord commBlockShape, commTileShape;
        int format = CCH_FMT_E2M1;
        uint32_t transB = 0;
        bool outFp16 = false;
    };
    struct Params {
        Arguments args;
        int64_t localExperts;
    };
    static size_t GetWorkspaceSize(const Arguments &) { return 0; }
    static Params ToUnderlyingArguments(const Arguments &args, uint8_t * = nullptr)
    {
        return Params{args, (int64_t)(args.expertNum / (args.epSize ? args.epSize : 1))};
    }
    static int Launch(const Params &p, void *stream)
    {
        const Arguments &a = p.args;
        const int32_t *groups = reinterpret_cast<const int32_t *>(a.ptrGlobalTokensPerLocalExpert);
        if (a.outFp16)
            return cch_mx_gmm_mapped(a.ptrA, a.ptrMxScaleA, a.ptrB, a.ptrMxScaleB, groups, nullptr, a.ptrC, a.gemmShape.m(),
                                     CCH_OUT_FP16, p.localExperts, a.gemmShape.m(), a.gemmShape.n(), a.gemmShape.k(), a.format,
                                     (int)a.transB, stream);
        return cch_mx_gmm(a.ptrA, a.ptrMxScaleA, a.ptrB, a.ptrMxScaleB, groups, a.ptrC, p.localExperts, a.gemmShape.m(),
                          a.gemmShape.n(), a.gemmShape.k(), a.format, (int)a.transB, stream);
    }
};

}  // namespace Kernel

namespace Device {

template <class DGemmKernel> class DeviceDGemm {
public:
    using Arguments = typename DGemmKernel::Arguments;
    using Params = typename DGemmKernel::Params;

    const Params &params() const { return params_; }

    static size_t GetWorkspaceSize(const Arguments &args) { return DGemmKernel::GetWorkspaceSize(args); }

    Status Initialize(const Arguments &args, uint8_t *workspace = nullptr)
    {
        params_ = DGemmKernel::ToUnderlyingArguments(args, workspace);
        initialized_ = true;
        return Status::kSuccess;
    }

    // blockDim and fftsAddr belong to the reference's core grid and cross-core flags; the HIP
    // library sizes its own grid.  Like the reference's Run this returns after the stream has
    // drained; a failed launch is reported the way ACL_CHECK reports (stderr, carry on) and as
    // the returned status.
    Status Run(void *stream, uint32_t /*blockDim*/, uint64_t /*fftsAddr*/)
    {
        if (!initialized_) return Status::kErrorInvalidProblem;
        const int rc = DGemmKernel::Launch(params_, stream);
        if (rc != CCH_OK) fprintf(stderr, "DeviceDGemm::Run: cchError:%d %s\n", rc, cch_last_error());
        CCH_CHECK(cch_stream_sync(stream));
        return rc == CCH_OK ? Status::kSuccess : (rc == CCH_EINVAL ? Status::kErrorInvalidProblem : Status::kErrorInternal);
    }
    Status operator()(void *stream, uint32_t blockDim, uint64_t fftsAddr) { return Run(stream, blockDim, fftsAddr); }

private:
    Params params_{};
    bool initialized_ = false;
};

}  // namespace Device
}  // namespace DGemm
}  // namespace Catccos

#endif  // CATCCOS_HOST_DEVICE_DGEMM_H
