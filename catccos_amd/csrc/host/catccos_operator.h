// Abstract operator of the host surface: owns the per-operator knowledge of buffer sizes,
// data-file names and tiling validity (reference utils/catccos_operator.h:31-44).
#ifndef CATCCOS_HOST_OPERATOR_H
#define CATCCOS_HOST_OPERATOR_H

#include <functional>
#include <memory>
#include <string>

#include "info.h"

class CatccosOperator {
public:
    virtual ~CatccosOperator() = default;
    virtual bool CheckCocTilingParams(uint32_t rankSize, const CocTilingParams &cocTiling) = 0;
    // Allocates every device buffer of the operator and fills the inputs from `dataFile` (a
    // directory), or with constants when it is empty.  The caller frees with FreeDeviceSpace.
    virtual void AllocateDeviceSpace(KernelParams &params, const CocTilingParams &cocTiling, uint32_t rankId,
                                     std::string dataFile = "") = 0;
    virtual void WriteResultFile(const KernelParams &params, const CocTilingParams &cocTiling, uint32_t rankId,
                                 std::string dataFile = "") = 0;
    virtual size_t GetWorkspaceSize(const CocTilingParams &cocTiling) = 0;
    virtual CocCommType GetActualKernelType(const CocTilingParams &cocTiling) = 0;
};

using OperatorCreator = std::function<std::unique_ptr<CatccosOperator>()>;

#endif  // CATCCOS_HOST_OPERATOR_H
