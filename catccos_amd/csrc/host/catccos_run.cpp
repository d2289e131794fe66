// Command-line driver over the operator surface, the counterpart of the reference's generic
// harness (tests/dynamic_tiling/main.cpp:186-398) for one rank and without tiling search:
//   registry -> CheckCocTilingParams -> AllocateDeviceSpace -> launcher (warm-up + timed loop)
//   -> WriteResultFile -> FreeDeviceSpace.
//
//   catccos_run <kernel> <m> <k> <n> <data_dir|-> [--transB 0|1] [--experts E] [--rank R] [--ranks S] [--topk T] [--fp16 0|1]
//               [--warmup W] [--iters I]
//   catccos_run <kernel> --shapes <csv> <data_dir|-> [options]
//                                 one run per line "M,K,N[,TA,TB]" of a test_shapes.csv, the loop of
//                                 the reference's run.sh scripts; with a data directory, shape
//                                 M,K,N reads and writes <data_dir>/<M>_<K>_<N>/
//   catccos_run --list            registry names and dispatch keys, no device needed
// <kernel> is a short name of CommTypeMap (mxqtag, agmmdq, a5mxfp8mmrs, dgds, a5fp4mxatavgmm,
// a5fp8mxatavgmm, a5fp8gmmata, a5fp4gmmata, a5moe); "-" as data_dir runs on constant inputs and writes nothing (perf mode).
#include <chrono>
#include <cstdlib>
#include <fstream>
#include <sstream>
#include <string>
#include <vector>

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

struct RunOptions {
    CocTilingParams tiling;
    uint32_t rank = 0, warmup = WARM_UP_TIMES, iters = PERF_TEST_CYCLE_TIMES, fp16Out = 0;
};

static int RunOne(const std::string &kernelName, const RunOptions &opt, const std::string &dataDir)
{
    CocTilingParams tiling = opt.tiling;
    const uint32_t rank = opt.rank, warmup = opt.warmup, iters = opt.iters, fp16Out = opt.fp16Out;
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
    const bool walk = argc >= 3 && std::string(argv[2]) == "--shapes";
    if (argc < (walk ? 5 : 6)) {
        ERROR_LOG("usage: %s <kernel> <m> <k> <n> <data_dir|-> [--transB 0|1] [--experts E] [--rank R] [--ranks S] [--topk T] [--fp16 0|1] [--warmup W] [--iters I]\n"
                  "       %s <kernel> --shapes <csv> <data_dir|-> [options]", argv[0], argv[0]);
        return -1;
    }
    const std::string kernelName = argv[1];
    RunOptions opt;
    opt.tiling.rankSize = 1;
    opt.tiling.epSize = 1;
    opt.tiling.expertNum = 1;
    std::string dataDir = argv[walk ? 4 : 5];
    if (dataDir == "-") dataDir.clear();
    for (int i = walk ? 5 : 6; i + 1 < argc; i += 2) {
        const std::string key = argv[i];
        const uint32_t val = (uint32_t)atoll(argv[i + 1]);
        if (key == "--transB") opt.tiling.transB = val;
        else if (key == "--experts") opt.tiling.expertNum = val;
        else if (key == "--rank") opt.rank = val;
        else if (key == "--ranks") opt.tiling.rankSize = val ? val : 1;
        else if (key == "--topk") opt.tiling.topK = val ? val : 1;
        else if (key == "--fp16") opt.fp16Out = val;
        else if (key == "--warmup") opt.warmup = val;
        else if (key == "--iters") opt.iters = val;
        else { ERROR_LOG("unknown option %s", key.c_str()); return -1; }
    }
    int rc = cch_init(0);
    if (rc != CCH_OK) {
        ERROR_LOG("cch_init failed: %s", cch_last_error());
        return -1;
    }
    if (!walk) {
        opt.tiling.m = (uint32_t)atoll(argv[2]);
        opt.tiling.k = (uint32_t)atoll(argv[3]);
        opt.tiling.n = (uint32_t)atoll(argv[4]);
        return RunOne(kernelName, opt, dataDir);
    }
    // The reference's run.sh scripts read test_shapes.csv line by line (header "M,K,N[,TA,TB]") and
    // start the operator once per shape; here one process walks the list.  With a data directory,
    // shape M,K,N reads and writes <data_dir>/<M>_<K>_<N>/.
    std::ifstream csv(argv[3]);
    if (!csv) {
        ERROR_LOG("cannot read shape list %s", argv[3]);
        return -1;
    }
    std::string line;
    int shapes = 0;
    while (std::getline(csv, line)) {
        std::vector<uint32_t> v;
        std::stringstream ss(line);
        std::string cell;
        bool numeric = true;
        while (std::getline(ss, cell, ',')) {
            char *end = nullptr;
            const unsigned long long x = strtoull(cell.c_str(), &end, 10);
            while (end && (*end == ' ' || *end == '\r' || *end == '\t')) end++;
            if (end == cell.c_str() || (end && *end)) { numeric = false; break; }
            v.push_back((uint32_t)x);
        }
        if (!numeric || v.empty()) continue;   // header or blank line
        if (v.size() < 3) {
            ERROR_LOG("shape list %s: line \"%s\" has fewer than three columns", argv[3], line.c_str());
            return -1;
        }
        RunOptions one = opt;
        one.tiling.m = v[0];
        one.tiling.k = v[1];
        one.tiling.n = v[2];
        if (v.size() >= 5) {
            one.tiling.transA = v[3];
            one.tiling.transB = v[4];
        }
        INFO_LOG("Processing test case: M=%u, K=%u, N=%u", v[0], v[1], v[2]);
        const std::string dir = dataDir.empty() ? dataDir
                                                : dataDir + "/" + std::to_string(v[0]) + "_" + std::to_string(v[1]) + "_" + std::to_string(v[2]);
        if (RunOne(kernelName, one, dir) != 0) return -1;
        shapes++;
    }
    INFO_LOG("%d shapes finished", shapes);
    return shapes > 0 ? 0 : -1;
}
