// Layout tags of the GEMM operands (names as in /root/reference/bfAintBGemm/gemm_tensor_layout.hpp:5-28).
// The reference instantiates RowMajor only (bfAintBGemm.cc:17-23: A, B, scale and C are "rrr");
// ColumnMajor exists there as a name.  The library implements the row-major case.
#pragma once
#include <cstddef>
#include <ostream>
#include <type_traits>

namespace gemm_layout {

struct BaseTensorLayout {};

namespace gemm {
template <bool kRowsContiguous>
struct MajorTag : BaseTensorLayout {
    static constexpr bool rows_contiguous = kRowsContiguous;
    static constexpr const char* name = kRowsContiguous ? "RowMajor" : "ColumnMajor";
};
using RowMajor = MajorTag<true>;
using ColumnMajor = MajorTag<false>;
}  // namespace gemm

template <typename L>
typename std::enable_if<std::is_base_of<BaseTensorLayout, L>::value, std::ostream&>::type operator<<(std::ostream& os, const L&)
{
    os << L::name;
    return os;
}

// Elements spanned by a matrix stored with a leading dimension (the lambda at bfAintBGemm.cc:68-76).
template <typename L>
inline std::size_t matrix_space_size(std::size_t n_row, std::size_t n_col, std::size_t stride, L)
{
    return L::rows_contiguous ? (n_row - 1) * stride + n_col : (n_col - 1) * stride + n_row;
}

}  // namespace gemm_layout
