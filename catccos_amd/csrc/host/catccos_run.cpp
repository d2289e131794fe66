// Command-line driver over the operator surface, the counterpart of the reference's generic
// harness (tests/dynamic_tiling/main.cpp:186-398) for one rank and without tiling search:
//   registry -> CheckCocTilingParams -> AllocateDeviceSpace -> launcher (warm-up + timed loop)
//   -> WriteResultFile -> FreeDeviceSpace.
//
//   catccos_run <kernel> <m> <k> <n> <data_dir|-> [--transB 0|1] [--experts E] [--rank R] [--ranks S] [--topk T] [--fp16 0|1]
//               [--warmup W] [--iters I]
//   catccos_run --list            registry names and dispatch keys, no device needed
// <kernel> is a short name of CommTypeMap (mxqtag, agmmdq, a5mxfp8mmrs, dgds, a5fp4mxatavgmm,
// a5fp8mxatavgmm); "-" as data_dir runs on constant inputs and writes nothing (perf mode).
#include <chrono>
#include <cstdlib>

#include "launch_map.h"
#include "operator_registry.h"

static CocDataType DataTypeOf(CocCommType type)
{
    switch (type) {
        case MX_QUANT_ALLGATHER:
        case ASCEND950_MXFP8_MATMUL_REDUCE_SCATTER: return FP8E4M3FN;
        case ALLGATHER_MATMUL_DEQUANT:
        case DISPATCH_GMM_DEQUANT_SWIGLU: return INT8;
        default: return BF16;
    }
}

int main(int argc, char **argv)
{
    if (argc >= 2 && std::string(argv[1]) == "--list") {
        for (auto &name : OperatorRegistry::Instance().Names()) printf("operator %s\n", name.c_str());
        for (auto &kv : CommTypeMap) {
            for (CocDataType dt : {FP16, INT8, BF16, FP8E4M3FN}) {
                if (KernelDispatcher::GetKernelFunc(kv.second, dt))
                    printf("launcher %s type=%d dtype=%d key=%d name=%s%s\n", kv.first.c_str(), (int)kv.second, (int)dt,
                           ((int)kv.second << 8) | (int)dt, CommTypeOpNameMap.at(kv.second).c_str(),
                           dt == DataTypeOf(kv.second) ? "" : " (--fp16 1)");
            }
        }
        return 0;
    }
    if (argc < 6) {
        ERROR_LOG("usage: %s <kernel> <m> <k> <n> <data_dir|-> [--transB 0|1] [--experts E] [--rank R] [--ranks S] [--topk T] [--fp16 0|1] [--warmup W] [--iters I]", argv[0]);
        return -1;
    }
    const std::string kernelName = argv[1];
    CocTilingParams tiling;
    tiling.m = (uint32_t)atoll(argv[2]);
    tiling.k = (uint32_t)atoll(argv[3]);
    tiling.n = (uint32_t)atoll(argv[4]);
    std::string dataDir = argv[5];
    if (dataDir == "-") dataDir.clear();
    tiling.rankSize = 1;
    tiling.epSize = 1;
    tiling.expertNum = 1;
    uint32_t rank = 0, warmup = WARM_UP_TIMES, iters = PERF_TEST_CYCLE_TIMES, fp16Out = 0;
    for (int i = 6; i + 1 < argc; i += 2) {
        const std::string key = argv[i];
        const uint32_t val = (uint32_t)atoll(argv[i + 1]);
        if (key == "--transB") tiling.transB = val;
        else if (key == "--experts") tiling.expertNum = val;
        else if (key == "--rank") rank = val;
        else if (key == "--ranks") tiling.rankSize = val ? val : 1;
        else if (key == "--topk") tiling.topK = val ? val : 1;
        else if (key == "--fp16") fp16Out = val;
        else if (key == "--warmup") warmup = val;
        else if (key == "--iters") iters = val;
        else { ERROR_LOG("unknown option %s", key.c_str()); return -1; }
    }

    const CocCommType commType = GetCommType(kernelName);
    if (commType == UNKNOWN || CommTypeOpNameMap.find(commType) == CommTypeOpNameMap.end()) {
        ERROR_LOG("unknown kernel %s", kernelName.c_str());
        return -1;
    }
    auto op = OperatorRegistry::Instance().CreateOperator(CommTypeOpNameMap.at(commType));
    if (!op) {
        ERROR_LOG("operator %s is not part of this build", CommTypeOpNameMap.at(commType).c_str());
        return -1;
    }
    if (!op->CheckCocTilingParams(tiling.rankSize, tiling)) {
        ERROR_LOG("invalid shape m=%u k=%u n=%u experts=%u for %s", tiling.m, tiling.k, tiling.n, tiling.expertNum, kernelName.c_str());
        return -1;
    }
    int rc = cch_init(0);
    if (rc != CCH_OK) {
        ERROR_LOG("cch_init failed: %s", cch_last_error());
        return -1;
    }
    void *stream = nullptr;
    CCH_CHECK(cch_stream_create(&stream));

    KernelParams params;
    op->AllocateDeviceSpace(params, tiling, rank, dataDir);
    const CocCommType actual = op->GetActualKernelType(tiling);
    // --fp16 1 asks for the half-precision launcher of an operator that has one
    KernelFuncPtr fn = KernelDispatcher::GetKernelFunc(actual, fp16Out ? FP16 : DataTypeOf(actual));
    if (!fn) {
        ERROR_LOG("no launcher for kernel type %d", (int)actual);
        return -1;
    }
    for (uint32_t i = 0; i < warmup; i++) fn(stream, 0, 0, params, nullptr, nullptr, tiling, tiling.transA, tiling.transB);
    auto t0 = std::chrono::steady_clock::now();
    for (uint32_t i = 0; i < iters; i++) fn(stream, 0, 0, params, nullptr, nullptr, tiling, tiling.transA, tiling.transB);
    auto t1 = std::chrono::steady_clock::now();
    if (iters) printf("[PERF] Avg latency: %.2f us/iter\n", std::chrono::duration<double, std::micro>(t1 - t0).count() / iters);

    if (!dataDir.empty()) op->WriteResultFile(params, tiling, rank, dataDir);
    FreeDeviceSpace(params);
    CCH_CHECK(cch_stream_destroy(stream));
    INFO_LOG("%s finished, error num: 0", kernelName.c_str());
    return 0;
}
