// Workspace-region sizing of the MoE FFN operator (reference:
// include/catccos/detail/ascend950_moe_ready.hpp:21-56).  On the reference device two bf16 staging regions
// double as per-expert ready counters (one 64-byte line each), so a region is at least as large as its
// counters; the published workspace size keeps that rule so both implementations report the same bytes.
#ifndef CATCCOS_DETAIL_ASCEND950_MOE_READY_HPP
#define CATCCOS_DETAIL_ASCEND950_MOE_READY_HPP

#include <cstdint>

namespace Catccos::Detail {

struct Ascend950MoeReady {
    static constexpr uint32_t kCacheLineBytes = 64;
    static constexpr uint32_t kStride = kCacheLineBytes / sizeof(int32_t);

    static constexpr uint64_t Align(uint64_t bytes, uint64_t alignment = 512)
    {
        return (bytes + alignment - 1) / alignment * alignment;
    }
    static constexpr uint64_t CounterBytes(uint32_t localExperts)
    {
        return uint64_t{localExperts} * kCacheLineBytes;
    }
    // counters of the dispatch region sit behind a [ranks, localExperts] int32 offset table
    static constexpr uint64_t DispatchOffset(uint32_t ranks, uint32_t localExperts)
    {
        return Align(uint64_t{ranks} * localExperts * sizeof(int32_t), kCacheLineBytes);
    }
    static constexpr uint64_t SwigluRegionBytes(uint64_t stagingBytes, uint32_t localExperts)
    {
        const uint64_t counters = CounterBytes(localExperts);
        return Align(stagingBytes > counters ? stagingBytes : counters);
    }
    static constexpr uint64_t DispatchRegionBytes(uint64_t stagingBytes, uint32_t ranks, uint32_t localExperts)
    {
        const uint64_t counters = DispatchOffset(ranks, localExperts) + CounterBytes(localExperts);
        return Align(stagingBytes > counters ? stagingBytes : counters);
    }
};

}  // namespace Catccos::Detail
#endif
