// The host-side operators of the hot path, registered under the reference's registry names.
// Each one knows its buffer sizes and data files for ONE rank's already-landed slice: the
// communication stage of the reference operator is dropped, so rankSize only selects file names
// and output offsets.  File names follow the reference's <op>_host.h files (cited per class);
// all files are raw little-endian arrays without header.
#include <algorithm>
#include <cstdlib>
#include <vector>

#include "operator_registry.h"

namespace {

// Device buffer of `bytes`, filled from `path` (if `dataDir` is non-empty) or with `fillByte`.
// `minFileBytes` > 0 accepts a shorter file (the rest keeps the fill value).
uint8_t *LoadOrFill(size_t bytes, const std::string &dataDir, const std::string &name, int fillByte,
                    size_t *fileBytes = nullptr)
{
    void *dev = nullptr;
    CCH_CHECK(cch_malloc(&dev, bytes));
    if (bytes == 0 || dev == nullptr) return static_cast<uint8_t *>(dev);
    if (dataDir.empty()) {
        CCH_CHECK(cch_memset(dev, fillByte, bytes));
        return static_cast<uint8_t *>(dev);
    }
    void *host = nullptr;
    CCH_CHECK(cch_malloc_host(&host, bytes));
    if (host == nullptr) return static_cast<uint8_t *>(dev);
    memset(host, fillByte, bytes);
    size_t got = 0;
    ReadFile(dataDir + "/" + name, host, bytes, &got);
    if (fileBytes) *fileBytes = got;
    CCH_CHECK(cch_memcpy_h2d(dev, host, bytes));
    CCH_CHECK(cch_free_host(host));
    return static_cast<uint8_t *>(dev);
}

uint8_t *DeviceAlloc(size_t bytes)
{
    void *dev = nullptr;
    CCH_CHECK(cch_malloc(&dev, bytes));
    return static_cast<uint8_t *>(dev);
}

void DumpDevice(const uint8_t *dev, size_t bytes, const std::string &path, size_t offset = 0)
{
    if (bytes == 0) return;
    void *host = nullptr;
    CCH_CHECK(cch_malloc_host(&host, bytes));
    if (host == nullptr) return;
    CCH_CHECK(cch_memcpy_d2h(host, dev, bytes));
    WriteFile(path, host, bytes, offset);
    CCH_CHECK(cch_free_host(host));
}

std::string R(uint32_t rank) { return std::to_string(rank); }
size_t ScaleCols(size_t k) { return 2 * ((k + 63) / 64); }  // E8M0 bytes per row: block count padded to even

// ---------------------------------------------------------------------------------------------
// MX quantisation, bf16 -> FP8 E4M3 + E8M0 (reference examples/ascend950_mx_quant_allgather/
// mx_quant_allgather_host.h:7-119).  ptrA = input, ptrB = scales, ptrC = payload.
// Here `n` is the quantised (row) length, as in the reference.
class MxQuantAllGatherOperator : public CatccosOperator {
public:
    void AllocateDeviceSpace(KernelParams &params, const CocTilingParams &t, uint32_t rankId, std::string dataFile) override
    {
        const size_t m = t.m, n = t.n;
        // constant fill: bf16 1.0 = 0x3F80 cannot be made by memset, 0x3C3C (~0.0115) can
        uint8_t *in = LoadOrFill(m * n * 2, dataFile, "rank_" + R(rankId) + "_input.bin", 0x3C);
        uint8_t *out = DeviceAlloc(m * n);
        uint8_t *scale = DeviceAlloc(m * ScaleCols(n));
        params.SetKernelParams(in, scale, out);
    }
    void WriteResultFile(const KernelParams &params, const CocTilingParams &t, uint32_t rankId, std::string dataFile) override
    {
        const size_t m = t.m, n = t.n;
        DumpDevice(params.ptrC, m * n, dataFile + "/rank_" + R(rankId) + "_output.bin");
        DumpDevice(params.ptrB, m * ScaleCols(n), dataFile + "/rank_" + R(rankId) + "_mxscale.bin");
    }
    size_t GetWorkspaceSize(const CocTilingParams &) override { return 0; }
    CocCommType GetActualKernelType(const CocTilingParams &) override { return MX_QUANT_ALLGATHER; }
    bool CheckCocTilingParams(uint32_t, const CocTilingParams &t) override { return t.m > 0 && t.n > 0 && t.n % MX_BLOCK_SIZE == 0; }
};

// ---------------------------------------------------------------------------------------------
// int8 matmul + dequant (reference examples/allgather_matmul_dequant/allgather_matmul_dequant_host.h:16-128).
// ptrA = A int8 [m,k], ptrB = B int8 ([k,n] or, with transB, [n,k]), ptrC = out bf16 [m,n],
// custom[0] = per-channel fp32 [n], custom[1] = per-token fp32 [m].
// scale_gm.bin may hold fp32[n] or the reference's 64-bit fix-pipe words (low 32 bits = the fp32
// scale, examples/utils/gen_allgather_fixpipe_quant_data.py:57-60); pertoken_scale_gm_rank<r>.bin
// is this build's addition (fp32[m]; absent = all ones).
class AllGatherMatmulDequantOperator : public CatccosOperator {
public:
    void AllocateDeviceSpace(KernelParams &params, const CocTilingParams &t, uint32_t rankId, std::string dataFile) override
    {
        const size_t m = t.m, k = t.k, n = t.n;
        uint8_t *a = LoadOrFill(m * k, dataFile, "a_gm_rank" + R(rankId) + ".bin", 1);
        uint8_t *b = LoadOrFill(k * n, dataFile, "b_gm_rank" + R(rankId) + ".bin", 1);
        uint8_t *d = DeviceAlloc(m * n * 2);
        std::vector<float> perCh(n, 1.0f), perTok(m, 1.0f);
        if (!dataFile.empty()) {
            std::vector<uint64_t> raw(n, 0);
            size_t got = 0;
            if (ReadFile(dataFile + "/scale_gm.bin", raw.data(), n * 8, &got)) {
                if (got == n * 8) {
                    for (size_t i = 0; i < n; i++) {
                        const uint32_t lo = static_cast<uint32_t>(raw[i]);
                        memcpy(&perCh[i], &lo, 4);
                    }
                } else if (got == n * 4) {
                    memcpy(perCh.data(), raw.data(), n * 4);
                } else {
                    ERROR_LOG("scale_gm.bin has %zu bytes, expected %zu or %zu", got, n * 4, n * 8);
                }
            }
            struct stat st;
            const std::string tokFile = dataFile + "/pertoken_scale_gm_rank" + R(rankId) + ".bin";
            if (stat(tokFile.c_str(), &st) == 0) ReadFile(tokFile, perTok.data(), m * 4);
        }
        uint8_t *chDev = DeviceAlloc(n * 4), *tokDev = DeviceAlloc(m * 4);
        CCH_CHECK(cch_memcpy_h2d(chDev, perCh.data(), n * 4));
        CCH_CHECK(cch_memcpy_h2d(tokDev, perTok.data(), m * 4));
        params.SetKernelParams(a, b, d, chDev, tokDev);
    }
    void WriteResultFile(const KernelParams &params, const CocTilingParams &t, uint32_t rankId, std::string dataFile) override
    {
        DumpDevice(params.ptrC, static_cast<size_t>(t.m) * t.n * 2, dataFile + "/output_rank" + R(rankId) + ".bin");
    }
    size_t GetWorkspaceSize(const CocTilingParams &) override { return 0; }  // no B padding pass on this path
    CocCommType GetActualKernelType(const CocTilingParams &) override { return ALLGATHER_MATMUL_DEQUANT; }
    bool CheckCocTilingParams(uint32_t, const CocTilingParams &t) override { return t.m > 0 && t.n > 0 && t.k > 0; }
};

// ---------------------------------------------------------------------------------------------
// MXFP8 dense GEMM (reference examples/ascend950_mxfp8_matmul_reduce_scatter/
// ascend950_mxfp8_matmul_reduce_scatter_host.h:28-142).  ptrA/ptrB payloads, ptrC = out bf16,
// custom[0] = scaleA [m, 2*ceil(k/64)], custom[1] = scaleB (layout by transB).
// The result goes to output.bin at offset rank * bytes, as every rank of the reference does.
class Ascend950MxFp8MatmulReduceScatterOperator : public CatccosOperator {
public:
    void AllocateDeviceSpace(KernelParams &params, const CocTilingParams &t, uint32_t rankId, std::string dataFile) override
    {
        const size_t m = t.m, k = t.k, n = t.n, sc = ScaleCols(k);
        const std::string p = "rank_" + R(rankId) + "_";
        uint8_t *a = LoadOrFill(m * k, dataFile, p + "a.bin", 0x38);  // E4M3 1.0
        uint8_t *b = LoadOrFill(k * n, dataFile, p + "b.bin", 0x38);
        uint8_t *sa = LoadOrFill(m * sc, dataFile, p + "a_scale.bin", 127);
        uint8_t *sb = LoadOrFill(n * sc, dataFile, p + "b_scale.bin", 127);
        uint8_t *d = DeviceAlloc(m * n * 2);
        params.SetKernelParams(a, b, d, sa, sb);
    }
    void WriteResultFile(const KernelParams &params, const CocTilingParams &t, uint32_t rankId, std::string dataFile) override
    {
        const size_t bytes = static_cast<size_t>(t.m) * t.n * 2;
        DumpDevice(params.ptrC, bytes, dataFile + "/output.bin", rankId * bytes);
    }
    size_t GetWorkspaceSize(const CocTilingParams &) override { return 0; }
    CocCommType GetActualKernelType(const CocTilingParams &) override { return ASCEND950_MXFP8_MATMUL_REDUCE_SCATTER; }
    bool CheckCocTilingParams(uint32_t, const CocTilingParams &t) override { return t.m > 0 && t.n > 0 && t.k > 0 && t.k % MX_BLOCK_SIZE == 0; }
};

// ---------------------------------------------------------------------------------------------
// MoE grouped int8 matmul + dequant + SwiGLU (reference examples/dispatch_gmm_dequant_swiglu/
// dispatch_gmm_dequant_swiglu_host.h:15-119), two file sets:
//  * the reference's own (expert_idx_<r>.bin present): a_gm_<r>.bin bf16 tokens [m,k], expert_idx_<r>.bin
//    int32 [m,topK], scale_gm_<r>.bin per-channel scales as 64-bit fix-pipe words (low 32 bits = fp32,
//    gen_data_dispatch_gmm_dequant_swiglu.py:75-76) or plain fp32.  Routing (stable sort of the flat
//    expert indices, as moe_init_routing does), dynamic int8 quantisation with the expert-sorted row
//    gather and the grouped matmul all run on the device, over m * topK rows.
//    ptrA = tokens, ptrB = W, ptrC = out bf16 [m*topK, n/2], custom[0] = per-channel fp32 [E,n],
//    custom[1] = expert idx (as in the reference), then derived: custom[2] = per-token fp32 [m*topK],
//    custom[3] = rows per expert, custom[4] = flat entry at each sorted position [m*topK], custom[5] = int8
//    rows, custom[6] = sorted position of each flat entry, custom[7] = routing workspace.
//  * after the dispatch (no expert_idx file): a_gm_<r>.bin holds the int8 tokens this rank received,
//    grouped by local expert ([m,k]); group_list_<r>.bin int32[expertNum] their counts;
//    pertoken_scale_<r>.bin fp32[m].  ptrA = tokens, ptrB = W int8 [E,k,n] (transB: [E,n,k]),
//    ptrC = out bf16 [m,n/2], custom[0] = per-channel fp32 [E,n], custom[1] = group list,
//    custom[2] = per-token fp32 [m].
class DispatchGmmDequantSwigluOperator : public CatccosOperator {
public:
    void AllocateDeviceSpace(KernelParams &params, const CocTilingParams &t, uint32_t rankId, std::string dataFile) override
    {
        const size_t m = t.m, k = t.k, n = t.n, e = t.expertNum, topK = t.topK ? t.topK : 1;
        struct stat st;
        const std::string idxFile = dataFile + "/expert_idx_" + R(rankId) + ".bin";
        fromTokens_ = !dataFile.empty() && stat(idxFile.c_str(), &st) == 0;
        uint8_t *b = LoadOrFill(e * k * n, dataFile, "b_gm_" + R(rankId) + ".bin", 1);
        std::vector<float> perCh(e * n, 1.0f);
        if (!dataFile.empty()) {
            std::vector<uint64_t> raw(e * n, 0);
            size_t got = 0;
            if (ReadFile(dataFile + "/scale_gm_" + R(rankId) + ".bin", raw.data(), e * n * 8, &got)) {
                if (got == e * n * 8) {
                    for (size_t i = 0; i < e * n; i++) {
                        const uint32_t lo = static_cast<uint32_t>(raw[i]);
                        memcpy(&perCh[i], &lo, 4);
                    }
                } else if (got == e * n * 4) {
                    memcpy(perCh.data(), raw.data(), e * n * 4);
                } else {
                    ERROR_LOG("scale_gm_%u.bin has %zu bytes, expected %zu or %zu", rankId, got, e * n * 4, e * n * 8);
                }
            }
        }
        uint8_t *chDev = DeviceAlloc(e * n * 4);
        CCH_CHECK(cch_memcpy_h2d(chDev, perCh.data(), e * n * 4));
        if (fromTokens_) {
            const size_t rows = m * topK;
            uint8_t *x = LoadOrFill(m * k * 2, dataFile, "a_gm_" + R(rankId) + ".bin", 0);
            std::vector<int32_t> expertIdx(rows, 0);
            ReadFile(idxFile, expertIdx.data(), rows * 4);
            // buffers of the device-side routing (stable sort by expert), filled by the launcher
            const size_t wsBytes = static_cast<size_t>(cch_moe_init_routing_workspace_bytes(static_cast<int64_t>(rows), static_cast<int>(e)));
            uint8_t *idxDev = DeviceAlloc(rows * 4), *tokDev = DeviceAlloc(rows * 4), *grpDev = DeviceAlloc(e * 4);
            uint8_t *srcDev = DeviceAlloc(rows * 4), *q = DeviceAlloc(rows * k), *d = DeviceAlloc(rows * (n / 2) * 2);
            uint8_t *posDev = DeviceAlloc(rows * 4), *wsDev = DeviceAlloc(wsBytes);
            CCH_CHECK(cch_memcpy_h2d(idxDev, expertIdx.data(), rows * 4));
            params.SetKernelParams(x, b, d, chDev, idxDev, tokDev, grpDev, srcDev, q, posDev, wsDev);
            return;
        }
        uint8_t *a = LoadOrFill(m * k, dataFile, "a_gm_" + R(rankId) + ".bin", 1);
        uint8_t *d = DeviceAlloc(m * (n / 2) * 2);
        std::vector<float> perTok(m, 1.0f);
        std::vector<int32_t> groups(e, 0);
        for (size_t i = 0; i < e; i++) groups[i] = static_cast<int32_t>(m / e + (i < m % e ? 1 : 0));
        if (!dataFile.empty()) {
            ReadFile(dataFile + "/pertoken_scale_" + R(rankId) + ".bin", perTok.data(), m * 4);
            ReadFile(dataFile + "/group_list_" + R(rankId) + ".bin", groups.data(), e * 4);
        }
        uint8_t *tokDev = DeviceAlloc(m * 4), *grpDev = DeviceAlloc(e * 4);
        CCH_CHECK(cch_memcpy_h2d(tokDev, perTok.data(), m * 4));
        CCH_CHECK(cch_memcpy_h2d(grpDev, groups.data(), e * 4));
        params.SetKernelParams(a, b, d, chDev, grpDev, tokDev);
    }
    void WriteResultFile(const KernelParams &params, const CocTilingParams &t, uint32_t rankId, std::string dataFile) override
    {
        const size_t rows = static_cast<size_t>(t.m) * (fromTokens_ ? (t.topK ? t.topK : 1) : 1);
        DumpDevice(params.ptrC, rows * (t.n / 2) * 2, dataFile + "/output_" + R(rankId) + ".bin");
    }
    size_t GetWorkspaceSize(const CocTilingParams &) override { return 0; }
    CocCommType GetActualKernelType(const CocTilingParams &) override { return DISPATCH_GMM_DEQUANT_SWIGLU; }
    bool CheckCocTilingParams(uint32_t, const CocTilingParams &t) override
    {
        return t.m > 0 && t.k > 0 && t.n > 0 && t.n % 2 == 0 && t.expertNum > 0 &&
               static_cast<uint64_t>(t.m) * (t.topK ? t.topK : 1) < (1ull << 31);
    }

private:
    bool fromTokens_ = false;
};

// ---------------------------------------------------------------------------------------------
// MX grouped matmul, FP4 and FP8 payload (reference examples/ascend950_fp4_mx_alltoallv_grouped_matmul/
// ascend950_fp4_mx_alltoallv_grouped_matmul_host.h:7-165 and its fp8 twin).  ptrA = tokens received
// (grouped by local expert, m rows), ptrB = W [E,...], ptrC = out bf16 [m,n], custom[0] = scaleA,
// custom[1] = scaleB, custom[2] = local_tokens_per_expert (unused on one rank),
// custom[3] = global_tokens_per_local_expert int32 [rankSize, E_loc]; with the source-rank
// dimension collapsed its first row is the group list.
template <bool FP4, CocCommType KIND> class MxAllToAllVGroupedMatmulOperator : public CatccosOperator {
public:
    void AllocateDeviceSpace(KernelParams &params, const CocTilingParams &t, uint32_t rankId, std::string dataFile) override
    {
        const size_t m = t.m, k = t.k, n = t.n, e = t.expertNum, sc = ScaleCols(k), pack = FP4 ? 2 : 1;
        const int one = FP4 ? 0x22 : 0x38;  // payload 1.0 in either format
        uint8_t *a = LoadOrFill(m * k / pack, dataFile, "input_a_" + R(rankId) + ".bin", one);
        uint8_t *b = LoadOrFill(e * k * n / pack, dataFile, "input_b_" + R(rankId) + ".bin", one);
        uint8_t *sa = LoadOrFill(m * sc, dataFile, "input_a_scale_" + R(rankId) + ".bin", 127);
        uint8_t *sb = LoadOrFill(e * n * sc, dataFile, "input_b_scale_" + R(rankId) + ".bin", 127);
        uint8_t *d = DeviceAlloc(m * n * 2);
        std::vector<int32_t> groups(e, 0);
        for (size_t i = 0; i < e; i++) groups[i] = static_cast<int32_t>(m / e + (i < m % e ? 1 : 0));
        if (!dataFile.empty()) ReadFile(dataFile + "/global_tokens_per_local_expert_" + R(rankId) + ".bin", groups.data(), e * 4);
        uint8_t *localDev = DeviceAlloc(e * 4), *grpDev = DeviceAlloc(e * 4);
        CCH_CHECK(cch_memcpy_h2d(localDev, groups.data(), e * 4));
        CCH_CHECK(cch_memcpy_h2d(grpDev, groups.data(), e * 4));
        params.SetKernelParams(a, b, d, sa, sb, localDev, grpDev);
    }
    void WriteResultFile(const KernelParams &params, const CocTilingParams &t, uint32_t rankId, std::string dataFile) override
    {
        DumpDevice(params.ptrC, static_cast<size_t>(t.m) * t.n * 2, dataFile + "/output_" + R(rankId) + ".bin");
    }
    size_t GetWorkspaceSize(const CocTilingParams &) override { return 0; }
    CocCommType GetActualKernelType(const CocTilingParams &) override { return KIND; }
    bool CheckCocTilingParams(uint32_t, const CocTilingParams &t) override
    {
        return t.m > 0 && t.k > 0 && t.n > 0 && t.k % 64 == 0 && t.expertNum > 0 && (!FP4 || t.n % 2 == 0);
    }
};
using Ascend950Fp4MxAllToAllVGroupedMatmulOperator = MxAllToAllVGroupedMatmulOperator<true, ASCEND950_FP4_MX_ALLTOALLV_GROUPED_MATMUL>;
using Ascend950Fp8MxAllToAllVGroupedMatmulOperator = MxAllToAllVGroupedMatmulOperator<false, ASCEND950_FP8_MX_ALLTOALLV_GROUPED_MATMUL>;

// ---------------------------------------------------------------------------------------------
// MX grouped matmul whose results leave in send-buffer order, FP8 and FP4 payload (reference
// examples/ascend950_fp8_mx_grouped_matmul_alltoallv/ascend950_fp8_mx_grouped_matmul_alltoallv_host.h:
// 16-160 and its fp4 twin): the down projection of the MoE layer.  ptrA = tokens grouped by local
// expert and, inside an expert, by the rank they came from (m rows), ptrB = W [E,...], ptrC = out
// bf16 [rankSize * m, n] zero-filled, region r holding the rows that go back to rank r in expert
// order; custom[0] = scaleA, custom[1] = scaleB, custom[2] = local_tokens_per_expert (unused on one
// rank), custom[3] = global_tokens_per_local_expert int32 [rankSize, E].  Derived here, as the
// reference's scheduler derives them on the device (block_scheduler_reducescatter_alltoallv.hpp:
// 211-256): custom[4] = rows per expert, custom[5] = destination row of every row of A.
// The output is bf16 or, through the FP16 launchers (the type the reference registers this operator
// for), IEEE half; both are two bytes per element.
template <bool FP4, CocCommType KIND> class MxGroupedMatmulAllToAllVOperator : public CatccosOperator {
public:
    void AllocateDeviceSpace(KernelParams &params, const CocTilingParams &t, uint32_t rankId, std::string dataFile) override
    {
        const size_t m = t.m, k = t.k, n = t.n, ranks = t.rankSize ? t.rankSize : 1, sc = ScaleCols(k), pack = FP4 ? 2 : 1;
        const size_t e = t.expertNum / (t.epSize ? t.epSize : 1);
        const int one = FP4 ? 0x22 : 0x38;  // payload 1.0 in either format
        uint8_t *a = LoadOrFill(m * k / pack, dataFile, "a_gm_" + R(rankId) + ".bin", one);
        uint8_t *b = LoadOrFill(e * k * n / pack, dataFile, "b_gm_" + R(rankId) + ".bin", one);
        uint8_t *sa = LoadOrFill(m * sc, dataFile, "a_scale_" + R(rankId) + ".bin", 127);
        uint8_t *sb = LoadOrFill(e * n * sc, dataFile, "b_scale_" + R(rankId) + ".bin", 127);
        const size_t outBytes = ranks * m * n * 2;
        uint8_t *d = DeviceAlloc(outBytes);
        CCH_CHECK(cch_memset(d, 0, outBytes));
        std::vector<int32_t> local(t.expertNum, 0), global(ranks * e, 0);
        for (size_t r = 0; r < ranks; r++)
            for (size_t i = 0; i < e; i++) global[r * e + i] = static_cast<int32_t>(m / (ranks * e));
        if (!dataFile.empty()) {
            ReadFile(dataFile + "/local_tokens_per_expert_" + R(rankId) + ".bin", local.data(), local.size() * 4);
            ReadFile(dataFile + "/global_tokens_per_local_expert_" + R(rankId) + ".bin", global.data(), global.size() * 4);
        }
        // rows per expert, and where each row goes: chunk (expert i, rank r) of A -> region r, after
        // the chunks of experts 0..i-1 for that rank
        std::vector<int32_t> groups(e, 0), rowMap(m, -1);
        size_t src = 0;
        for (size_t i = 0; i < e; i++) {
            for (size_t r = 0; r < ranks; r++) {
                const int64_t cnt = std::max<int32_t>(global[r * e + i], 0);
                int64_t dst = static_cast<int64_t>(r * m);
                for (size_t j = 0; j < i; j++) dst += std::max<int32_t>(global[r * e + j], 0);
                for (int64_t x = 0; x < cnt && src < m; x++) rowMap[src++] = static_cast<int32_t>(dst + x);
                groups[i] += static_cast<int32_t>(cnt);
            }
        }
        uint8_t *localDev = DeviceAlloc(local.size() * 4), *globalDev = DeviceAlloc(global.size() * 4);
        uint8_t *grpDev = DeviceAlloc(e * 4), *mapDev = DeviceAlloc(m * 4);
        CCH_CHECK(cch_memcpy_h2d(localDev, local.data(), local.size() * 4));
        CCH_CHECK(cch_memcpy_h2d(globalDev, global.data(), global.size() * 4));
        CCH_CHECK(cch_memcpy_h2d(grpDev, groups.data(), e * 4));
        CCH_CHECK(cch_memcpy_h2d(mapDev, rowMap.data(), m * 4));
        params.SetKernelParams(a, b, d, sa, sb, localDev, globalDev, grpDev, mapDev);
    }
    void WriteResultFile(const KernelParams &params, const CocTilingParams &t, uint32_t rankId, std::string dataFile) override
    {
        const size_t ranks = t.rankSize ? t.rankSize : 1;
        DumpDevice(params.ptrC, ranks * t.m * static_cast<size_t>(t.n) * 2, dataFile + "/output_" + R(rankId) + ".bin");
    }
    size_t GetWorkspaceSize(const CocTilingParams &) override { return 0; }
    CocCommType GetActualKernelType(const CocTilingParams &) override { return KIND; }
    bool CheckCocTilingParams(uint32_t, const CocTilingParams &t) override
    {
        return t.m > 0 && t.k > 0 && t.n > 0 && t.k % 64 == 0 && t.expertNum > 0 && (!FP4 || t.n % 2 == 0) &&
               static_cast<uint64_t>(t.rankSize ? t.rankSize : 1) * t.m < (1ull << 31);
    }
};
using Ascend950Fp8MxGroupedMatmulAllToAllVOperator = MxGroupedMatmulAllToAllVOperator<false, ASCEND950_FP8_MX_GROUPED_MATMUL_ALLTOALLV>;
using Ascend950Fp4MxGroupedMatmulAllToAllVOperator = MxGroupedMatmulAllToAllVOperator<true, ASCEND950_FP4_MX_GROUPED_MATMUL_ALLTOALLV>;

// ---------------------------------------------------------------------------------------------
// The MXFP8 MoE FFN of one rank from routing to combine (reference examples/ascend950_dispatch_ffn_combine/
// ascend950_dispatch_ffn_combine_host.h:15-194; files as examples/utils/gen_data_moe.py:460-616 writes them):
//   in_routing_matrix_a_<r>.bin      bf16 [m,k] tokens            in_routing_expert_idx_<r>.bin  int32 [m,topK]
//   in_gmm_matrix_b_<r>.bin          E4M3 [E,n,k] (W1 transposed) in_gmm_matrix_b_scale_<r>.bin  E8M0 [E,n,2*ceil(k/64)]
//   in_gmm_matrix_b2_<r>.bin         E4M3 [E,k,n/2]               in_gmm_matrix_b2_scale_<r>.bin E8M0 [E,k,2*ceil(n/128)]
//   in_gather_gate_weight_<r>.bin    fp32 [m,topK]                output_<r>.bin                 bf16 [m,k]
// Pointer roles as the reference's main.cpp:203-210 reads them back: ptrA = tokens, ptrB = W1, ptrC = out,
// custom[0] = W2, [1] = expert_idx, [2] = gate weights, [3] = W1 scales, [4] = W2 scales.  The buffers the
// reference carves out of its workspace (:165-176) follow: [5] expanded_row_idx (row of each routed token after
// the sort), [6] its inverse, [7] tokens per expert, [8] packed MXFP8 rows after dispatch, [9]/[10] the
// quantised activation and its scales, [11] GMM2's output rows, [12] the routing sort's workspace.
// One rank holds every expert here: the two all-to-all exchanges are the identity.
class Ascend950DispatchFFNCombineOperator : public CatccosOperator {
public:
    void AllocateDeviceSpace(KernelParams &params, const CocTilingParams &t, uint32_t rankId, std::string dataFile) override
    {
        const size_t m = t.m, k = t.k, n = t.n, h = n / 2, e = t.expertNum, topK = t.topK ? t.topK : 1, rows = m * topK;
        const std::string r = R(rankId);
        uint8_t *a = DeviceAlloc(m * k * 2), *idx = DeviceAlloc(rows * 4), *probs = DeviceAlloc(rows * 4);
        {
            // constant inputs of the perf mode: tokens 1.0, routes round-robin over the experts, equal gate weights
            std::vector<uint16_t> ones(m * k, 0x3F80);
            std::vector<int32_t> routes(rows);
            std::vector<float> gate(rows, 1.0f / static_cast<float>(topK));
            for (size_t i = 0; i < rows; i++) routes[i] = static_cast<int32_t>(i % e);
            if (!dataFile.empty()) {
                ReadFile(dataFile + "/in_routing_matrix_a_" + r + ".bin", ones.data(), m * k * 2);
                ReadFile(dataFile + "/in_routing_expert_idx_" + r + ".bin", routes.data(), rows * 4);
                ReadFile(dataFile + "/in_gather_gate_weight_" + r + ".bin", gate.data(), rows * 4);
            }
            CCH_CHECK(cch_memcpy_h2d(a, ones.data(), m * k * 2));
            CCH_CHECK(cch_memcpy_h2d(idx, routes.data(), rows * 4));
            CCH_CHECK(cch_memcpy_h2d(probs, gate.data(), rows * 4));
        }
        uint8_t *b = LoadOrFill(e * n * k, dataFile, "in_gmm_matrix_b_" + r + ".bin", 0x38);
        uint8_t *b2 = LoadOrFill(e * k * h, dataFile, "in_gmm_matrix_b2_" + r + ".bin", 0x38);
        uint8_t *sb = LoadOrFill(e * n * ScaleCols(k), dataFile, "in_gmm_matrix_b_scale_" + r + ".bin", 127);
        uint8_t *sb2 = LoadOrFill(e * k * ScaleCols(h), dataFile, "in_gmm_matrix_b2_scale_" + r + ".bin", 127);
        uint8_t *c = DeviceAlloc(m * k * 2);
        CCH_CHECK(cch_memset(c, 0, m * k * 2));
        const size_t wsBytes = static_cast<size_t>(cch_moe_init_routing_workspace_bytes(static_cast<int64_t>(rows), static_cast<int>(e)));
        uint8_t *s2d = DeviceAlloc(rows * 4), *d2s = DeviceAlloc(rows * 4), *cnt = DeviceAlloc(e * 4);
        uint8_t *packed = DeviceAlloc(rows * (k + ScaleCols(k))), *act = DeviceAlloc(rows * h), *actScale = DeviceAlloc(rows * ScaleCols(h));
        uint8_t *y = DeviceAlloc(rows * k * 2), *ws = DeviceAlloc(wsBytes);
        params.SetKernelParams(a, b, c, b2, idx, probs, sb, sb2, s2d, d2s, cnt, packed, act, actScale, y, ws);
    }
    void WriteResultFile(const KernelParams &params, const CocTilingParams &t, uint32_t rankId, std::string dataFile) override
    {
        DumpDevice(params.ptrC, static_cast<size_t>(t.m) * t.k * 2, dataFile + "/output_" + R(rankId) + ".bin");
    }
    size_t GetWorkspaceSize(const CocTilingParams &) override { return 0; }
    CocCommType GetActualKernelType(const CocTilingParams &) override { return ASCEND950_DISPATCH_FFN_COMBINE; }
    bool CheckCocTilingParams(uint32_t rankSize, const CocTilingParams &t) override
    {
        if (rankSize > 1) {
            ERROR_LOG("Ascend950DispatchFFNCombine: this build runs one rank that holds every expert");
            return false;
        }
        // the reference's own shape rule (ascend950_dispatch_ffn_combine_host.h:180-184)
        if (t.k % 256 != 0 || t.n % 512 != 0) {
            ERROR_LOG("MXFP8 FFN requires K %% 256 == 0 and N %% 512 == 0");
            return false;
        }
        const uint32_t topK = t.topK ? t.topK : 1;
        return t.m > 0 && t.k > 0 && t.n > 0 && t.expertNum > 0 && topK <= t.expertNum &&
               static_cast<uint64_t>(t.m) * topK < (1ull << 31);
    }
};

}  // namespace

REGISTER_OPERATOR("MxQuantAllGather", MxQuantAllGatherOperator)
REGISTER_OPERATOR("AllGatherMatmulDequant", AllGatherMatmulDequantOperator)
REGISTER_OPERATOR("Ascend950MxFp8MatmulReduceScatter", Ascend950MxFp8MatmulReduceScatterOperator)
REGISTER_OPERATOR("DispatchGmmDequantSwiglu", DispatchGmmDequantSwigluOperator)
REGISTER_OPERATOR("Ascend950Fp4MxAllToAllVGroupedMatmul", Ascend950Fp4MxAllToAllVGroupedMatmulOperator)
REGISTER_OPERATOR("Ascend950Fp8MxAllToAllVGroupedMatmul", Ascend950Fp8MxAllToAllVGroupedMatmulOperator)
REGISTER_OPERATOR("Ascend950Fp8MxGroupedMatmulAllToAllV", Ascend950Fp8MxGroupedMatmulAllToAllVOperator)
REGISTER_OPERATOR("Ascend950Fp4MxGroupedMatmulAllToAllV", Ascend950Fp4MxGroupedMatmulAllToAllVOperator)
REGISTER_OPERATOR("Ascend950DispatchFFNCombine", Ascend950DispatchFFNCombineOperator)
