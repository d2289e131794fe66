// Tiling / pointer structs and operator-kind tables of the operator surface.
// Enumerator values, short names and registry names are those of the reference's utils/info.h:46-275,
// so that registry keys and (commType << 8 | dataType) dispatch keys stay interchangeable.
#ifndef CATCCOS_HOST_INFO_H
#define CATCCOS_HOST_INFO_H

#include <cstdint>
#include <map>
#include <string>

#include "utils.h"

constexpr uint32_t WARM_UP_TIMES = 10;
constexpr uint32_t PERF_TEST_CYCLE_TIMES = 3;
constexpr uint32_t MX_BLOCK_SIZE = 32;

enum CocCommType {
    MATMUL_ALLREDUCE = 0,
    ALLGATHER_MATMUL,
    ASCEND950_ALLGATHER_MATMUL,
    MATMUL_REDUCE_SCATTER,
    ASCEND950_MATMUL_REDUCE_SCATTER,
    ALLGATHER_MATMUL_WITH_GATHER_RESULT,
    GROUPED_MATMUL_ALLTOALLV,
    GROUPED_MATMUL_ALLTOALLV_TLA,
    ASCEND950_GROUPED_MATMUL_ALLTOALLV,
    ALLTOALLV_GROUPED_MATMUL,
    ALLGATHER_MATMUL_RDMA,
    ALLTOALLV_GMM_V2,
    ALLGATHER_MATMUL_DEQUANT_BIAS,
    ALLGATHER_MATMUL_DEQUANT,
    ALLGATHER_MATMUL_DEQUANT_PADDING,
    QUANT_ALLTOALL,
    QUANT_ALLGATHER,
    MATMUL_DEQUANT_REDUCE_SCATTER_WRITE,
    ASCEND950_MXFP8_MATMUL_REDUCE_SCATTER,
    ASCEND950_MXFP8_MATMUL_ALLTOALL,
    ALLGATHER_MATMUL_REMOTE_READ,
    DISPATCH_GMM_DEQUANT_SWIGLU,
    ASCEND950_FP8_MX_ALLGATHER_MATMUL,
    ASCEND950_FP4_MX_ALLGATHER_MATMUL,
    MX_QUANT_ALLGATHER,
    ASCEND950_FP8_MX_GROUPED_MATMUL_ALLTOALLV,
    ASCEND950_FP4_MX_GROUPED_MATMUL_ALLTOALLV,
    ASCEND950_FP8_MX_ALLTOALLV_GROUPED_MATMUL,
    ASCEND950_FP4_MX_ALLTOALLV_GROUPED_MATMUL,
    ASCEND950_ALLTOALLV_GROUPED_MATMUL,
    ASCEND950_FP4_MX_MATMUL_REDUCE_SCATTER,
    DISPATCH_FFN_COMBINE,
    ASCEND950_DISPATCH_FFN_COMBINE,
    ASCEND950_ALLGATHER_MATMUL_UDMA,
    ASCEND950_MXFP8_ALLTOALL_MATMUL_SPLIT_K_URMA,
    TYPE_NUM,
    UNKNOWN
};

enum CocDataType { FP16 = 1, INT8 = 2, BF16 = 27, FP8E4M3FN = 36 };

struct CocTilingParams {
    uint32_t m = 0;
    uint32_t k = 0;
    uint32_t n = 0;
    uint32_t transA = 0;
    uint32_t transB = 0;
    uint32_t m0 = 0;
    uint32_t k0 = 0;
    uint32_t n0 = 0;
    uint32_t commTileM = 0;
    uint32_t commInterval = 0;
    uint32_t commNpuSplit = 0;
    uint32_t commDataSplit = 0;
    uint32_t commBlockM = 0;
    uint32_t rankSize = 0;
    uint32_t epSize = 0;
    uint32_t expertNum = 0;
    uint32_t topK = 1;
};

// Device pointers handed to a launcher: three fixed roles plus a pinned-host array of extras.
// The struct owns only that array; device buffers are released by FreeDeviceSpace.
struct KernelParams {
    uint8_t *ptrA = nullptr;
    uint8_t *ptrB = nullptr;
    uint8_t *ptrC = nullptr;
    uint8_t **customPtrs = nullptr;
    uint32_t customCount = 0;

    KernelParams() = default;
    KernelParams(const KernelParams &) = delete;
    KernelParams &operator=(const KernelParams &) = delete;

    template <typename... Args> void SetKernelParams(uint8_t *a, uint8_t *b, uint8_t *c, Args... extras)
    {
        ptrA = a;
        ptrB = b;
        ptrC = c;
        ReleaseCustom();
        customCount = sizeof...(extras);
        if (customCount > 0) {
            void *mem = nullptr;
            CCH_CHECK(cch_malloc_host(&mem, customCount * sizeof(uint8_t *)));
            customPtrs = static_cast<uint8_t **>(mem);
            uint8_t *list[] = {extras...};
            for (uint32_t i = 0; customPtrs && i < customCount; ++i) customPtrs[i] = list[i];
        }
    }

    ~KernelParams() { ReleaseCustom(); }

private:
    void ReleaseCustom()
    {
        if (customPtrs != nullptr) CCH_CHECK(cch_free_host(customPtrs));
        customPtrs = nullptr;
    }
};

inline void FreeDeviceSpace(KernelParams &params)
{
    CCH_CHECK(cch_free(params.ptrA));
    CCH_CHECK(cch_free(params.ptrB));
    CCH_CHECK(cch_free(params.ptrC));
    params.ptrA = params.ptrB = params.ptrC = nullptr;
    for (uint32_t i = 0; params.customPtrs && i < params.customCount; i++) {
        CCH_CHECK(cch_free(params.customPtrs[i]));
        params.customPtrs[i] = nullptr;
    }
}

// short kernel names accepted on the command line (reference utils/info.h:196-231)
const std::map<std::string, CocCommType> CommTypeMap = {
    {"mmar", MATMUL_ALLREDUCE},
    {"agmm", ALLGATHER_MATMUL},
    {"a5agmm", ASCEND950_ALLGATHER_MATMUL},
    {"mmrs", MATMUL_REDUCE_SCATTER},
    {"a5mmrs", ASCEND950_MATMUL_REDUCE_SCATTER},
    {"agmmwg", ALLGATHER_MATMUL_WITH_GATHER_RESULT},
    {"gmmata", GROUPED_MATMUL_ALLTOALLV},
    {"gmmatatla", GROUPED_MATMUL_ALLTOALLV_TLA},
    {"a5gmmata", ASCEND950_GROUPED_MATMUL_ALLTOALLV},
    {"atavgmm", ALLTOALLV_GROUPED_MATMUL},
    {"agmmrdma", ALLGATHER_MATMUL_RDMA},
    {"atavgmmv2", ALLTOALLV_GMM_V2},
    {"agmmdq", ALLGATHER_MATMUL_DEQUANT},
    {"agmmdqbs", ALLGATHER_MATMUL_DEQUANT_BIAS},
    {"mmdqrs", MATMUL_DEQUANT_REDUCE_SCATTER_WRITE},
    {"a5mxfp8mmrs", ASCEND950_MXFP8_MATMUL_REDUCE_SCATTER},
    {"a5mxfp8mmata", ASCEND950_MXFP8_MATMUL_ALLTOALL},
    {"agmmrr", ALLGATHER_MATMUL_REMOTE_READ},
    {"dgds", DISPATCH_GMM_DEQUANT_SWIGLU},
    {"a5fp8mxagmm", ASCEND950_FP8_MX_ALLGATHER_MATMUL},
    {"a5fp4mxagmm", ASCEND950_FP4_MX_ALLGATHER_MATMUL},
    {"mxqtag", MX_QUANT_ALLGATHER},
    {"a5fp8gmmata", ASCEND950_FP8_MX_GROUPED_MATMUL_ALLTOALLV},
    {"a5fp4gmmata", ASCEND950_FP4_MX_GROUPED_MATMUL_ALLTOALLV},
    {"a5fp8mxatavgmm", ASCEND950_FP8_MX_ALLTOALLV_GROUPED_MATMUL},
    {"a5fp4mxatavgmm", ASCEND950_FP4_MX_ALLTOALLV_GROUPED_MATMUL},
    {"a5atavgmm", ASCEND950_ALLTOALLV_GROUPED_MATMUL},
    {"a5fp4mmrs", ASCEND950_FP4_MX_MATMUL_REDUCE_SCATTER},
    {"moe", DISPATCH_FFN_COMBINE},
    {"a5moe", ASCEND950_DISPATCH_FFN_COMBINE},
    {"a5agmmudma", ASCEND950_ALLGATHER_MATMUL_UDMA},
    {"a5mxfp8atammsplitkurma", ASCEND950_MXFP8_ALLTOALL_MATMUL_SPLIT_K_URMA},
};

inline CocCommType GetCommType(const std::string &kernelName)
{
    auto it = CommTypeMap.find(kernelName);
    return it != CommTypeMap.end() ? it->second : UNKNOWN;
}

// registry names (reference utils/info.h:242-275)
const std::map<CocCommType, std::string> CommTypeOpNameMap = {
    {MATMUL_ALLREDUCE, "MatmulAllReduce"},
    {ALLGATHER_MATMUL, "AllGatherMatmul"},
    {ASCEND950_ALLGATHER_MATMUL, "Ascend950AllGatherMatmul"},
    {MATMUL_REDUCE_SCATTER, "MatmulReduceScatter"},
    {ASCEND950_MATMUL_REDUCE_SCATTER, "Ascend950MatmulReduceScatter"},
    {ALLGATHER_MATMUL_WITH_GATHER_RESULT, "AllGatherMatmulWithGatherResult"},
    {GROUPED_MATMUL_ALLTOALLV, "GroupedMatmulAllToAllV"},
    {GROUPED_MATMUL_ALLTOALLV_TLA, "GroupedMatmulAllToAllVTla"},
    {ASCEND950_GROUPED_MATMUL_ALLTOALLV, "Ascend950GroupedMatmulAllToAllV"},
    {ALLTOALLV_GROUPED_MATMUL, "AllToAllVGroupedMatmul"},
    {ALLGATHER_MATMUL_RDMA, "AllGatherMatmulRdma"},
    {ALLTOALLV_GMM_V2, "AllToAllVGMMV2"},
    {ALLGATHER_MATMUL_DEQUANT, "AllGatherMatmulDequant"},
    {ALLGATHER_MATMUL_DEQUANT_BIAS, "AllGatherMatmulDequantBias"},
    {ASCEND950_MXFP8_MATMUL_REDUCE_SCATTER, "Ascend950MxFp8MatmulReduceScatter"},
    {ASCEND950_MXFP8_MATMUL_ALLTOALL, "Ascend950MxFp8MatmulAllToAll"},
    {ALLGATHER_MATMUL_REMOTE_READ, "AllGatherMatmulRemoteRead"},
    {DISPATCH_GMM_DEQUANT_SWIGLU, "DispatchGmmDequantSwiglu"},
    {ASCEND950_FP8_MX_ALLGATHER_MATMUL, "Ascend950Fp8MxAllGatherMatmul"},
    {ASCEND950_FP4_MX_ALLGATHER_MATMUL, "Ascend950Fp4MxAllGatherMatmul"},
    {MX_QUANT_ALLGATHER, "MxQuantAllGather"},
    {MATMUL_DEQUANT_REDUCE_SCATTER_WRITE, "MatmulDequantReduceScatterWrite"},
    {ASCEND950_FP8_MX_GROUPED_MATMUL_ALLTOALLV, "Ascend950Fp8MxGroupedMatmulAllToAllV"},
    {ASCEND950_FP4_MX_GROUPED_MATMUL_ALLTOALLV, "Ascend950Fp4MxGroupedMatmulAllToAllV"},
    {ASCEND950_FP8_MX_ALLTOALLV_GROUPED_MATMUL, "Ascend950Fp8MxAllToAllVGroupedMatmul"},
    {ASCEND950_FP4_MX_ALLTOALLV_GROUPED_MATMUL, "Ascend950Fp4MxAllToAllVGroupedMatmul"},
    {ASCEND950_ALLTOALLV_GROUPED_MATMUL, "Ascend950AllToAllVGroupedMatmul"},
    {ASCEND950_FP4_MX_MATMUL_REDUCE_SCATTER, "Ascend950Fp4MxMatmulReduceScatter"},
    {DISPATCH_FFN_COMBINE, "DispatchFFNCombine"},
    {ASCEND950_DISPATCH_FFN_COMBINE, "Ascend950DispatchFFNCombine"},
    {ASCEND950_ALLGATHER_MATMUL_UDMA, "Ascend950AllGatherMatmulUdma"},
    {ASCEND950_MXFP8_ALLTOALL_MATMUL_SPLIT_K_URMA, "Ascend950MxFp8AllToAllMatmulSplitKUrma"},
};

inline int32_t CeilDev(int32_t num, int32_t div) { return div == 0 ? 0 : (num + div - 1) / div; }

#endif  // CATCCOS_HOST_INFO_H
