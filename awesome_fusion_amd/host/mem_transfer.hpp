// Host float matrices -> device wire formats, as /root/reference/bfAintBGemm/mem_transfer.hpp:6-32:
//   mem_transfer<bfloat16, float, ...>  element-wise fp32 -> bf16 by truncation (:12-21)
//   mem_transfer<int8_t,   float, ...>  static_cast<int8_t>(x) + 128 stored in a byte: excess-128 (:23-32)
// Added for this build: round-to-nearest-even activations and scales, and 4-bit packing.
#pragma once
#include <cstddef>
#include <cstdint>

#include "datatype.hpp"
#include "simple_device_mem.hpp"

template <typename Y, typename X, typename YLocation, typename XLocation>
void mem_transfer(YLocation& dst, XLocation& src, std::size_t size);

template <>
inline void mem_transfer<bfloat16, float, SimpleHostMem, SimpleHostMem>(SimpleHostMem& dst, SimpleHostMem& src, std::size_t size)
{
    bfloat16* d = static_cast<bfloat16*>(dst.GetBuffer());
    const float* s = static_cast<const float*>(src.GetBuffer());
    for (std::size_t i = 0; i < size; i++) d[i] = type_convert<bfloat16, float>(s[i]);
}

template <>
inline void mem_transfer<std::int8_t, float, SimpleHostMem, SimpleHostMem>(SimpleHostMem& dst, SimpleHostMem& src, std::size_t size)
{
    std::int8_t* d = static_cast<std::int8_t*>(dst.GetBuffer());
    const float* s = static_cast<const float*>(src.GetBuffer());
    for (std::size_t i = 0; i < size; i++) d[i] = static_cast<std::int8_t>(type_convert<std::int8_t, float>(s[i]) + 128);
}

// fp32 -> bf16 with round to nearest even (the rounding the library's contract uses for A and scales).
inline void mem_transfer_bf16_rne(SimpleHostMem& dst, SimpleHostMem& src, std::size_t size)
{
    bfloat16* d = static_cast<bfloat16*>(dst.GetBuffer());
    const float* s = static_cast<const float*>(src.GetBuffer());
    for (std::size_t i = 0; i < size; i++) d[i] = bf16_convert_rtn<bfloat16, float>(s[i]);
}

// 4-bit weights: float matrix [rows, ld] of integers in [-8,7] -> rows of ld/2 bytes; byte j holds
// column 2j in its low nibble and 2j+1 in its high nibble, each as q + 8 (the 4-bit sibling of +128).
inline void mem_transfer_int4(SimpleHostMem& dst, SimpleHostMem& src, std::size_t rows, std::size_t cols, std::size_t ld)
{
    std::uint8_t* d = static_cast<std::uint8_t*>(dst.GetBuffer());
    const float* s = static_cast<const float*>(src.GetBuffer());
    for (std::size_t r = 0; r < rows; r++)
        for (std::size_t j = 0; j < cols / 2; j++) {
            const unsigned lo = unsigned(static_cast<int>(s[r * ld + 2 * j]) + 8) & 0xfu;
            const unsigned hi = unsigned(static_cast<int>(s[r * ld + 2 * j + 1]) + 8) & 0xfu;
            d[r * (ld / 2) + j] = std::uint8_t(lo | (hi << 4));
        }
}
