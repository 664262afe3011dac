// The harness's own host GEMM: what `bfAintBGemm 1 ...` validates the device result against.
// Same name, signature and arithmetic as the reference's (/root/reference/bfAintBGemm/host_ref.hpp:3-25,
// called at bfAintBGemm.cc:200-209): every output is one fp32 sum over k in ascending order of
// a[m][k] * (b[k][n] * scale[n]), the weight scaled first.  Leading dimensions in elements; entries of c
// past column n of a row are left alone.  Build with -ffp-contract=off: a fused multiply-add would round
// differently from the two operations written here.
#pragma once
#include <cstddef>

static inline void gemm_rrr(float* ptr_c, const float* ptr_a, const float* ptr_b, const float* ptr_scale, std::size_t m,
                            std::size_t n, std::size_t k, std::size_t lda, std::size_t ldb, std::size_t ldc)
{
    for (std::size_t row = 0; row < m; ++row) {
        const float* a_row = ptr_a + row * lda;
        float* c_row = ptr_c + row * ldc;
        for (std::size_t col = 0; col < n; ++col) {
            const float s = ptr_scale[col];
            const float* b_col = ptr_b + col;  // walks down column `col`: stride ldb
            float sum = 0.0f;
            for (std::size_t kk = 0; kk < k; ++kk) sum += a_row[kk] * (b_col[kk * ldb] * s);
            c_row[col] = sum;
        }
    }
}
