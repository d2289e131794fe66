// Launcher ABI: one function per (operator kind, data type) with the signature the reference's
// harness calls (tests/dynamic_tiling/include/launch_map.h:15-59), looked up by
// (commType << 8) | dataType.  `stream` is a hipStream_t; blockNum, fftsAddr, workSpace and
// symmetricPtr belong to the dropped communication half and are ignored.
#ifndef CATCCOS_HOST_LAUNCH_MAP_H
#define CATCCOS_HOST_LAUNCH_MAP_H

#include <unordered_map>

#include "info.h"

using KernelFuncPtr = void (*)(void *stream, uint32_t blockNum, uint64_t fftsAddr, KernelParams &params,
                               uint8_t *workSpace, uint8_t *symmetricPtr, CocTilingParams &tiling, uint32_t transA,
                               uint32_t transB);

class KernelDispatcher {
public:
    static KernelFuncPtr GetKernelFunc(CocCommType commType, CocDataType dataType)
    {
        auto &map = Map();
        auto it = map.find(Key(commType, dataType));
        return it == map.end() ? nullptr : it->second;
    }
    static void RegisterKernelFunc(CocCommType commType, CocDataType dataType, KernelFuncPtr func)
    {
        Map().insert({Key(commType, dataType), func});
    }

private:
    static int Key(CocCommType commType, CocDataType dataType) { return (commType << 8) | dataType; }
    static std::unordered_map<int, KernelFuncPtr> &Map()
    {
        static std::unordered_map<int, KernelFuncPtr> map;
        return map;
    }
};

// The launchers this build provides (names as in the reference's impl/kernel_*.cpp).
void LaunchAscend950BF16QuantAllGatherFP8E4M3FN(void *, uint32_t, uint64_t, KernelParams &, uint8_t *, uint8_t *,
                                                CocTilingParams &, uint32_t, uint32_t);
void LaunchAllGatherMatmulDequantINT8(void *, uint32_t, uint64_t, KernelParams &, uint8_t *, uint8_t *, CocTilingParams &,
                                      uint32_t, uint32_t);
void LaunchAscend950MxFp8MatmulReduceScatterFP8E4M3FN(void *, uint32_t, uint64_t, KernelParams &, uint8_t *, uint8_t *,
                                                      CocTilingParams &, uint32_t, uint32_t);
void LaunchDispatchGmmDequantSwigluINT8(void *, uint32_t, uint64_t, KernelParams &, uint8_t *, uint8_t *,
                                        CocTilingParams &, uint32_t, uint32_t);
void LaunchAscend950Fp4MxAllToAllVGroupedMatmulBF16(void *, uint32_t, uint64_t, KernelParams &, uint8_t *, uint8_t *,
                                                    CocTilingParams &, uint32_t, uint32_t);
void LaunchAscend950Fp8MxAllToAllVGroupedMatmulBF16(void *, uint32_t, uint64_t, KernelParams &, uint8_t *, uint8_t *,
                                                    CocTilingParams &, uint32_t, uint32_t);

void LaunchAscend950Fp4MxAllToAllVGroupedMatmulFP16(void *, uint32_t, uint64_t, KernelParams &, uint8_t *, uint8_t *,
                                                    CocTilingParams &, uint32_t, uint32_t);
void LaunchAscend950Fp8MxAllToAllVGroupedMatmulFP16(void *, uint32_t, uint64_t, KernelParams &, uint8_t *, uint8_t *,
                                                    CocTilingParams &, uint32_t, uint32_t);

void LaunchAscend950Fp8MxGroupedMatmulAllToAllVBF16(void *, uint32_t, uint64_t, KernelParams &, uint8_t *, uint8_t *,
                                                    CocTilingParams &, uint32_t, uint32_t);
void LaunchAscend950Fp4MxGroupedMatmulAllToAllVBF16(void *, uint32_t, uint64_t, KernelParams &, uint8_t *, uint8_t *,
                                                    CocTilingParams &, uint32_t, uint32_t);

void LaunchAscend950Fp8MxGroupedMatmulAllToAllVFP16(void *, uint32_t, uint64_t, KernelParams &, uint8_t *, uint8_t *,
                                                    CocTilingParams &, uint32_t, uint32_t);
void LaunchAscend950Fp4MxGroupedMatmulAllToAllVFP16(void *, uint32_t, uint64_t, KernelParams &, uint8_t *, uint8_t *,
                                                    CocTilingParams &, uint32_t, uint32_t);
void LaunchAscend950DispatchFFNCombineBF16(void *, uint32_t, uint64_t, KernelParams &, uint8_t *, uint8_t *, CocTilingParams &,
                                           uint32_t, uint32_t);

#endif  // CATCCOS_HOST_LAUNCH_MAP_H
