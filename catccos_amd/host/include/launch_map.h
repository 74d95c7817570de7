// Uniform launch entry per (operator, data type), the shape of the reference's generic driver table
// (tests/dynamic_tiling/include/launch_map.h:16-59): one function-pointer signature for every operator so a
// driver can loop over shapes and operators without knowing their argument lists.
#pragma once

#include <map>

#include "operator_registry.h"

// blockNum and fftsAddr are accepted for signature compatibility and ignored (no cube/vector core split
// and no cross-core flags on a GPU); symmetric is unused with one rank.  Failures are reported through
// LaunchStatus() because the signature returns void.
using KernelFuncPtr = void (*)(void* stream, uint32_t blockNum, uint64_t fftsAddr, KernelParams& params, uint8_t* workspace,
                               uint8_t* symmetric, CocTilingParams& cocTiling, uint32_t transA, uint32_t transB);

inline int& LaunchStatus()
{
    static thread_local int status = CMX_OK;
    return status;
}

inline uint32_t LaunchKey(CocCommType type, CocDataType dtype) { return (static_cast<uint32_t>(type) << 8) | static_cast<uint32_t>(dtype); }

std::map<uint32_t, KernelFuncPtr>& LaunchMap();
KernelFuncPtr GetKernelFunc(CocCommType type, CocDataType dtype);
