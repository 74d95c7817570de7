// Overflow-checked buffer sizes for the quantizing operators (reference: utils/quant_size_utils.h:20-46).
#ifndef QUANT_SIZE_UTILS_H
#define QUANT_SIZE_UTILS_H

#include <cstddef>
#include <cstdint>
#include <initializer_list>
#include <limits>
#include <stdexcept>

// Product of the factors; throws std::overflow_error when it would not fit a signed offset / file size.
inline size_t CheckedBufferSize(std::initializer_list<size_t> factors)
{
    const size_t limit = static_cast<size_t>(std::numeric_limits<ptrdiff_t>::max());
    size_t product = 1;
    for (size_t f : factors) {
        if (f != 0 && product > limit / f) {
            throw std::overflow_error("Quant buffer size exceeds the addressable range");
        }
        product *= f;
    }
    return product;
}

// The multi-rank quantizers number their 2^20-element tiles in a 20-bit flag field per rank.
inline void CheckQuantBlockCount(size_t elementCount, uint32_t rankSize)
{
    if (rankSize == 0) {
        throw std::invalid_argument("Quant rank size must be positive");
    }
    const size_t tileElements = size_t{1} << 20;
    const size_t maxTiles = (size_t{1} << 20) - 1;
    const size_t perRank = (elementCount + rankSize - 1) / rankSize;
    if (perRank > maxTiles * tileElements) {
        throw std::overflow_error("Quant block count exceeds the synchronization flag range");
    }
}

#endif  // QUANT_SIZE_UTILS_H
