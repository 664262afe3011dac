// Device-side building blocks shared by every bfAintBGemm kernel for gfx950.
//
// The arithmetic restated here is the reference kernel's dequantisation
// (/root/reference/bfAintBGemm/bf16gemm_kernel_gfx90a.s:18-55): integer code -> fp32, times the
// column's scale, narrowed to bf16.  Differences by contract: scales are bf16 (so the product is
// exact in fp32), the narrowing rounds to nearest even (v_cvt_pk_bf16_f32) instead of truncating,
// and 4-bit codes exist.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace bfaintb {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2_t;
typedef __attribute__((ext_vector_type(4))) float f32x4_t;
typedef __attribute__((ext_vector_type(16))) float f32x16_t;

constexpr int kCounterSlots = 4096;  // arrival counters at the head of a workspace (uint32 each)

struct GemmParams {
    uint16_t* c;
    const uint16_t* a;
    const uint8_t* b;
    const uint16_t* scale;
    uint32_t m, n, k;
    uint32_t lda;        // elements
    uint32_t ldb_bytes;  // bytes per row of packed weights
    uint32_t ldc;        // elements
    uint32_t lds;        // elements per scale row (= n)
    uint32_t group_size; // rows of k per scale group; 0 = one group
    // split-K (decode variant only)
    uint32_t k_per_wg;   // rows of k one workgroup covers (multiple of 128)
    uint32_t splits;     // workgroups along k
    float* partials;     // [splits][m][n] fp32
    uint32_t* counters;  // [column blocks]
};

__device__ __forceinline__ float bf16_bits_to_f32(uint32_t bits16) { return __uint_as_float(bits16 << 16); }

// Two fp32 -> one dword of two bf16 (lo in bits 15:0), round to nearest even.
__device__ __forceinline__ uint32_t pack_bf16_rne(float lo, float hi)
{
    bf16x2_t v;
    v[0] = (__bf16)lo;
    v[1] = (__bf16)hi;
    return __builtin_bit_cast(uint32_t, v);
}

// Byte `I` of a dword as fp32 (v_cvt_f32_ubyteI).
template <int I>
__device__ __forceinline__ float ubyte_to_f32(uint32_t x)
{
    return (float)((x >> (8 * I)) & 0xffu);
}

// A column's scale prepared for dequantisation: w = fma(code, s, o) with o = -bias*s.
// code*s is exact inside the fma (<= 8 significant bits each), o is exact (bias is a power of
// two) and the sum (code-bias)*s has at most 16 significant bits, so the fma returns exactly
// float(q)*float(s), which is then rounded once to bf16.
struct ColScale {
    float s, o;
};

template <int BITS>
__device__ __forceinline__ ColScale make_col_scale(uint32_t scale_bf16_bits)
{
    ColScale cs;
    cs.s = bf16_bits_to_f32(scale_bf16_bits);
    cs.o = (BITS == 8 ? -128.0f : -8.0f) * cs.s;
    return cs;
}

__device__ __forceinline__ float dequant_code(float code, const ColScale& cs) { return __builtin_fmaf(code, cs.s, cs.o); }

}  // namespace bfaintb
