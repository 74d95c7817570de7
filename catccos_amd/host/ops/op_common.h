// Helpers shared by the operator classes: device buffers filled from raw .bin files.
#pragma once

#include <string>
#include <vector>

#include "operator_registry.h"
#include "quant_size_utils.h"

namespace mxops {

inline std::string RankFile(const std::string& dir, const std::string& stem, uint32_t rankId, bool prefixRank)
{
    // two naming schemes are in use: "<stem>_<rank>.bin" and "rank_<rank>_<stem>.bin"
    return prefixRank ? dir + "/rank_" + std::to_string(rankId) + "_" + stem + ".bin"
                      : dir + "/" + stem + "_" + std::to_string(rankId) + ".bin";
}

// Device buffer of `bytes`, filled from `path` (must have exactly that size; throws otherwise) or, when
// `path` is empty, with `fillByte`.
inline uint8_t* DeviceBufferFromFile(size_t bytes, const std::string& path, int fillByte = 0)
{
    uint8_t* dev = mxrt::DeviceAlloc(bytes);
    if (path.empty()) {
        MX_CHECK(cmx_rt_memset(dev, fillByte, bytes));
        return dev;
    }
    std::vector<uint8_t> host(bytes);
    try {
        ReadFileOrThrow(path, host.data(), bytes);
    } catch (...) {
        MX_CHECK(cmx_rt_free(dev));
        throw;
    }
    MX_CHECK(cmx_rt_memcpy_h2d(dev, host.data(), bytes));
    return dev;
}

inline uint8_t* DeviceBufferFromValues(const void* host, size_t bytes)
{
    uint8_t* dev = mxrt::DeviceAlloc(bytes);
    MX_CHECK(cmx_rt_memcpy_h2d(dev, host, bytes));
    return dev;
}

inline bool DeviceBufferToFile(const uint8_t* dev, size_t bytes, const std::string& path, size_t offset = 0)
{
    std::vector<uint8_t> host(bytes);
    MX_CHECK(cmx_rt_memcpy_d2h(host.data(), dev, bytes));
    return WriteFile(path, host.data(), bytes, offset);
}

inline size_t ScaleCols(size_t k) { return RoundUp<size_t>(CeilDev(static_cast<int32_t>(k), 32), 2); }

}  // namespace mxops
