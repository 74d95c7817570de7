// Plugin base class of the host layer (reference: utils/catccos_operator.h:35-54).
#ifndef CATCCOS_OPERATOR_H
#define CATCCOS_OPERATOR_H

#include <cstring>
#include <functional>
#include <iostream>
#include <memory>
#include <string>
#include <unordered_map>
#include <vector>

#include "info.h"
#include "padding.h"
#include "utils.h"

// 16-bit storage stand-in for half / bfloat16 host buffers (sizes only; no arithmetic on the host)
using fp16_t = uint16_t;
using float32_t = float;

class CatccosOperator {
public:
    virtual ~CatccosOperator() = default;

    // common shape/rank check first, then the operator's own
    bool ValidateCocTilingParams(uint32_t rankSize, const CocTilingParams& cocTiling)
    {
        if (!CheckCommonCocTilingParams(rankSize, cocTiling)) {
            return false;
        }
        return CheckCocTilingParams(rankSize, cocTiling);
    }

    // Bytes of symmetric (peer-visible) staging the caller provides.  One GPU has no peers; the
    // reference's figure is kept so callers that size one allocation from it stay unchanged.
    virtual size_t GetSymmetricSize(const CocTilingParams&) { return SHMEM_BUFF_BYTES; }

    virtual bool CheckCocTilingParams(uint32_t rankSize, const CocTilingParams& cocTiling) = 0;
    // Allocates every device input/output, fills inputs from <dataFile>/<name>_<rank>.bin (or defaults
    // when dataFile is empty) and records the pointers in params.  The caller frees (FreeDeviceSpace).
    virtual void AllocateDeviceSpace(KernelParams& params, const CocTilingParams& cocTiling, uint32_t rankId,
                                     std::string dataFile = "") = 0;
    virtual void WriteResultFile(const KernelParams& params, const CocTilingParams& cocTiling, uint32_t rankId,
                                 std::string dataFile = "") = 0;
    virtual size_t GetWorkspaceSize(const CocTilingParams& cocTiling) = 0;
    virtual CocCommType GetActualKernelType(const CocTilingParams& cocTiling) = 0;
};

using OperatorCreator = std::function<std::unique_ptr<CatccosOperator>()>;

#endif  // CATCCOS_OPERATOR_H
