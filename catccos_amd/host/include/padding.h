// Alignment helpers (reference: utils/padding.h:16-42 plus the RoundUp / CeilDiv spellings the example
// hosts take from the matmul library's alignment header).
#ifndef PADDING_H
#define PADDING_H

#include <cstddef>
#include <cstdint>

#include "utils.h"

template <class T>
constexpr T Roundup(const T& val, const T align)
{
    return (val + align - 1) / align * align;
}

template <class T>
constexpr T RoundUp(const T& val, const T align)
{
    return Roundup<T>(val, align);
}

template <uint32_t Div, class T>
constexpr T CeilDiv(const T& val)
{
    return (val + Div - 1) / Div;
}

template <class T>
constexpr T CeilDiv(const T& val, const T div)
{
    return div == 0 ? val : (val + div - 1) / div;
}

// A matrix needs a padded copy when its contiguous dimension is not a multiple of the alignment,
// or when that dimension is too long for one strided transfer.
inline bool IsNeedPadding(uint32_t rows, uint32_t cols, uint32_t trans, uint32_t alignByElement)
{
    const uint32_t contiguous = trans ? rows : cols;
    return contiguous >= 65536 || contiguous % alignByElement != 0;
}

inline size_t GetWorkspaceLen(uint32_t shape0, uint32_t shape1, size_t blockRows, size_t blockCols)
{
    return Roundup(static_cast<size_t>(shape0), blockRows) * Roundup(static_cast<size_t>(shape1), blockCols);
}

#endif  // PADDING_H
