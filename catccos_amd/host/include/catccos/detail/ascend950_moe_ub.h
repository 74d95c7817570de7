// Shape limits the reference operator enforces through its 256 KiB on-chip buffer accounting
// (reference: include/catccos/detail/ascend950_moe_ub.h:19-64).  The GPU kernels have no such limit;
// the predicate is kept so a driver can reject exactly the shapes the reference rejects.
#ifndef CATCCOS_DETAIL_ASCEND950_MOE_UB_H
#define CATCCOS_DETAIL_ASCEND950_MOE_UB_H

#include <algorithm>
#include <cstdint>

namespace Catccos::Detail {

struct Ascend950MoeUb {
    static constexpr uint64_t kCapacityBytes = 256 * 1024;

    static constexpr uint64_t Align(uint64_t bytes, uint64_t alignment)
    {
        return (bytes + alignment - 1) / alignment * alignment;
    }
    static constexpr uint64_t ScaleBytes(uint32_t hidden) { return Align((uint64_t{hidden} + 31) / 32, 2); }

    // input quantizer: two stages of (bf16 row + fp8 row + scales + two u16 scratch rows of scales)
    static constexpr uint64_t InputQuantBytes(uint32_t hidden)
    {
        return 2 * (3 * uint64_t{hidden} + 5 * ScaleBytes(hidden));
    }
    // dispatch: ping-pong buffers of two packed rows [codes | scales | pad to 32 B]
    static constexpr uint64_t DispatchBytes(uint32_t hidden)
    {
        const uint64_t packedRow = Align(uint64_t{hidden} + ScaleBytes(hidden), 32);
        return 2 * Align(2 * packedRow, 64);
    }
    // combine: 18 hidden-sized (512-aligned) buffers + 256 B + two 32-byte-aligned index/weight queues
    static constexpr uint64_t UnpermuteBytes(uint32_t m, uint32_t hidden, uint32_t topK, uint32_t aivNum)
    {
        if (aivNum == 0) {
            return kCapacityBytes + 1;
        }
        const uint64_t rowsPerCore = std::max<uint64_t>(1, std::min<uint64_t>(m / aivNum, 600));
        return 18 * Align(hidden, 512) + 256 + 2 * Align(rowsPerCore * topK * sizeof(uint32_t), 32);
    }
    static constexpr bool Fits(uint32_t m, uint32_t hidden, uint32_t topK, uint32_t aivNum)
    {
        return InputQuantBytes(hidden) <= kCapacityBytes && DispatchBytes(hidden) <= kCapacityBytes &&
               UnpermuteBytes(m, hidden, topK, aivNum) <= kCapacityBytes;
    }
};

}  // namespace Catccos::Detail
#endif
