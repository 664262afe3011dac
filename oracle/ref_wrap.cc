// TEST INFRASTRUCTURE ONLY.
// C-callable doors onto the reference's own host code, compiled from the headers where they lie
// (-I/root/reference/bfAintBGemm); nothing of the reference is copied here.  The resulting
// library (oracle/_ref/libbfaintb_ref.so) is used to pin the restatement in bfaintb_oracle.c and,
// when present, as the CPU baseline timed by the benchmark.
#include <cstddef>
#include <cstdint>
#include <cstdio>
#include <cmath>
#include <type_traits>
#include <ostream>

#include "host_ref.hpp"            // gemm_rrr
#include "datatype.hpp"            // type_convert, bf16_convert_rtn
#include "validation.hpp"          // valid_vector
#include "mem_transfer.hpp"        // mem_transfer specialisations (need SimpleHostMem)
#include "gemm_tensor_layout.hpp"  // layout tags

extern "C" {

void ref_gemm_rrr(float* c, const float* a, const float* b, const float* scale, std::size_t m, std::size_t n,
                  std::size_t k, std::size_t lda, std::size_t ldb, std::size_t ldc)
{
    gemm_rrr(c, a, b, scale, m, n, k, lda, ldb, ldc);
}

uint16_t ref_f32_to_bf16_rtz(float x) { return type_convert<bhalf_t, float>(x); }
float ref_bf16_to_f32(uint16_t x) { return type_convert<float, bhalf_t>(x); }
uint16_t ref_f32_to_bf16_rne(float x) { return bf16_convert_rtn<bhalf_t, float>(x); }

// Array doors: values travel by pointer, so signalling NaNs are not quieted on the way.
void ref_f32_to_bf16_rtz_n(uint16_t* dst, const float* src, std::size_t n)
{
    for(std::size_t i = 0; i < n; i++) dst[i] = type_convert<bhalf_t, float>(src[i]);
}
void ref_f32_to_bf16_rne_n(uint16_t* dst, const float* src, std::size_t n)
{
    for(std::size_t i = 0; i < n; i++) dst[i] = bf16_convert_rtn<bhalf_t, float>(src[i]);
}
void ref_bf16_to_f32_n(float* dst, const uint16_t* src, std::size_t n)
{
    for(std::size_t i = 0; i < n; i++) dst[i] = type_convert<float, bhalf_t>(src[i]);
}

// mem_transfer works on SimpleHostMem objects that own their storage; stage through them.
void ref_mem_transfer_bf16(uint16_t* dst, const float* src, std::size_t n)
{
    SimpleHostMem d(n * sizeof(bfloat16)), s(n * sizeof(float));
    __builtin_memcpy(s.GetBuffer(), src, n * sizeof(float));
    mem_transfer<bfloat16, float, SimpleHostMem, SimpleHostMem>(d, s, n);
    __builtin_memcpy(dst, d.GetBuffer(), n * sizeof(bfloat16));
}

void ref_mem_transfer_int8(uint8_t* dst, const float* src, std::size_t n)
{
    SimpleHostMem d(n), s(n * sizeof(float));
    __builtin_memcpy(s.GetBuffer(), src, n * sizeof(float));
    mem_transfer<int8_t, float, SimpleHostMem, SimpleHostMem>(d, s, n);
    __builtin_memcpy(dst, d.GetBuffer(), n);
}

int ref_valid_vector_bf16(const float* ref, const uint16_t* pred, int n, float nrms)
{
    return valid_vector<bfloat16>(ref, pred, n, nrms) ? 1 : 0;
}

const char* ref_row_major_name() { return gemm_layout::gemm::RowMajor::name; }
const char* ref_column_major_name() { return gemm_layout::gemm::ColumnMajor::name; }

}  // extern "C"
