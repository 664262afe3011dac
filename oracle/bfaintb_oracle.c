/*
 * TEST INFRASTRUCTURE ONLY — CPU restatement of the reference's bfAintBGemm arithmetic.
 *
 * Nothing in the shipped library or the host driver may include, link or call this file.
 * It exists so that tests, the smoke check and the benchmark's CPU-baseline leg have an
 * independent statement of what the GPU path must produce.
 *
 * Every function names the reference lines it follows (paths under
 * /root/reference/bfAintBGemm/).  Build with -ffp-contract=off: the reference's inner
 * statement is a separate fp32 multiply, multiply and add, each rounded.
 *
 * Pinning status (what checks each function, all in tests/test_oracle_*.py):
 *   orc_bf16_to_f32, orc_f32_to_bf16_rtz   exhaustive 2^16 round trip, known answers, the
 *                                          reference's own converters compiled from its headers
 *   orc_f32_to_bf16_rne                    tie/carry/Inf/NaN known answers, torch.bfloat16 on
 *                                          2^20 random bit patterns, the reference's compiled routine
 *   orc_int8_to_excess128                  closed form (q+128)&0xFF for all 256 values, compiled reference
 *   orc_magic_dequant_int8                 exhaustive identity with u-128 for all 256 bytes
 *   orc_gemm_rrr                           compiled reference (bit-for-bit), closed forms, fp64 brute
 *                                          force, exact-integer regime, numpy float32 sequential sum
 *   orc_gemm_rrr_fast                      bit-for-bit against orc_gemm_rrr
 *   orc_valid_vector                       hand-built vectors, compiled reference
 *   orc_dequant, orc_pack_int4, orc_check_ulp
 *                                          no counterpart in the reference (it has no int4, no group
 *                                          scales and no ULP criterion): pinned by brute force in numpy
 *                                          and by the exactness argument (8-bit integer times 8-bit
 *                                          significand fits fp32) checked exhaustively.
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#define ORC_API __attribute__((visibility("default")))

/* ---- number formats: datatype.hpp ------------------------------------------------------- */

/* bf16 -> fp32: place the 16 bits in the high half (datatype.hpp:31-42). */
ORC_API float orc_bf16_to_f32(uint16_t x)
{
    uint32_t u = (uint32_t)x << 16;
    float f;
    memcpy(&f, &u, 4);
    return f;
}

/* fp32 -> bf16 by truncation, the conversion mem_transfer uses (datatype.hpp:44-55). */
ORC_API uint16_t orc_f32_to_bf16_rtz(float x)
{
    uint32_t u;
    memcpy(&u, &x, 4);
    return (uint16_t)(u >> 16);
}

/* fp32 -> bf16 round-to-nearest-even with signalling-NaN preservation (datatype.hpp:80-121). */
ORC_API uint16_t orc_f32_to_bf16_rne(float x)
{
    uint32_t u;
    memcpy(&u, &x, 4);
    if ((~u & 0x7f800000u) != 0u) {
        /* zero, subnormal or normal: add 0x7fff plus the parity of the kept mantissa */
        u += 0x7fffu + ((u >> 16) & 1u);
    } else if ((u & 0xffffu) != 0u) {
        /* NaN whose payload lives only in the dropped half: keep it a NaN */
        u |= 0x10000u;
    }
    return (uint16_t)(u >> 16);
}

ORC_API void orc_bf16_to_f32_n(float* dst, const uint16_t* src, size_t n)
{
    for (size_t i = 0; i < n; ++i) dst[i] = orc_bf16_to_f32(src[i]);
}

/* mem_transfer<bfloat16,float>: element-wise truncation (mem_transfer.hpp:12-21). */
ORC_API void orc_mem_transfer_bf16(uint16_t* dst, const float* src, size_t n)
{
    for (size_t i = 0; i < n; ++i) dst[i] = orc_f32_to_bf16_rtz(src[i]);
}

/* The build's activation conversion: RNE instead of truncation (same loop, other rounding). */
ORC_API void orc_f32_to_bf16_rne_n(uint16_t* dst, const float* src, size_t n)
{
    for (size_t i = 0; i < n; ++i) dst[i] = orc_f32_to_bf16_rne(src[i]);
}

/* ---- weight wire formats: mem_transfer.hpp ---------------------------------------------- */

/* float -> int8 -> +128, stored in a byte: excess-128 (mem_transfer.hpp:23-32, line 30). */
ORC_API uint8_t orc_int8_to_excess128(float x)
{
    int8_t q = (int8_t)x;                 /* type_convert<int8_t,float> is a static_cast */
    return (uint8_t)(int8_t)(q + 128);    /* the sum is an int; storing it in int8_t wraps */
}

ORC_API void orc_mem_transfer_int8(uint8_t* dst, const float* src, size_t n)
{
    for (size_t i = 0; i < n; ++i) dst[i] = orc_int8_to_excess128(src[i]);
}

/*
 * int4 packing (no counterpart in the reference, which has 8-bit weights only).
 * Two weights per byte along N: byte j of row k holds column 2j in its low nibble and column
 * 2j+1 in its high nibble, each stored excess-8 (q+8 in 0..15), mirroring the excess-128
 * byte format of mem_transfer.hpp:30.  q is row-major [k, ldq]; dst rows are ldb_bytes apart.
 */
ORC_API void orc_pack_int4(uint8_t* dst, const int8_t* q, size_t k, size_t n, size_t ldq, size_t ldb_bytes)
{
    for (size_t i = 0; i < k; ++i)
        for (size_t j = 0; j < n / 2; ++j) {
            unsigned lo = (unsigned)(q[i * ldq + 2 * j] + 8) & 0xFu;
            unsigned hi = (unsigned)(q[i * ldq + 2 * j + 1] + 8) & 0xFu;
            dst[i * ldb_bytes + j] = (uint8_t)(lo | (hi << 4));
        }
}

/*
 * The kernel-side integer decode of the reference: splice the byte under 0x4B000000 (2^23) and
 * subtract 2^23+128 (bf16gemm_kernel_gfx90a.s:19-27 with the constants of lines 204-210).
 * Returns exactly (float)(u - 128).
 */
ORC_API float orc_magic_dequant_int8(uint8_t u)
{
    uint32_t bits = 0x4B000000u | (uint32_t)u;
    float f;
    memcpy(&f, &bits, 4);
    return f - 8388736.0f;
}

/* stored code -> signed integer value */
static inline int orc_decode_q(const uint8_t* b, size_t row, size_t col, size_t ldb_bytes, int bits)
{
    if (bits == 8) return (int)b[row * ldb_bytes + col] - 128;
    uint8_t byte = b[row * ldb_bytes + (col >> 1)];
    return (int)((col & 1) ? (byte >> 4) : (byte & 0xF)) - 8;
}

/*
 * Dequantization oracle: W[k,n] = bf16( float(q[k,n]) * float(scale[g(k), n]) ).
 * Device statement: bf16gemm_kernel_gfx90a.s:18-55 (integer -> fp32, one fp32 multiply by the
 * column's scale, pack to bf16) — there with fp32 scales and truncation; here the scale dtype and
 * rounding are parameters:
 *   scale_is_f32 = 0: scale is bf16 [groups, lds]   (the build's default contract)
 *                  1: scale is fp32 [groups, lds]   (the reference's dtype, bfAintBGemm.cc:27)
 *   rtz          = 0: round to nearest even          (build default)
 *                  1: truncate                       (what v_pack_b32_f16 op_sel:[1,1] does, asm:34-35)
 * group_size = 0 means one scale per column; otherwise g(k) = k / group_size.
 * ldb is in weight ELEMENTS (bfAintBGemm.cc:48-49); a 4-bit row is ldb/2 bytes.
 */
ORC_API void orc_dequant(uint16_t* w, const uint8_t* b, const void* scale, size_t k, size_t n, size_t ldb,
                         size_t ldw, size_t lds, int bits, size_t group_size, int scale_is_f32, int rtz)
{
    size_t ldb_bytes = bits == 8 ? ldb : ldb / 2;
    for (size_t i = 0; i < k; ++i) {
        size_t g = group_size ? i / group_size : 0;
        for (size_t j = 0; j < n; ++j) {
            float s = scale_is_f32 ? ((const float*)scale)[g * lds + j]
                                   : orc_bf16_to_f32(((const uint16_t*)scale)[g * lds + j]);
            float qf = (float)orc_decode_q(b, i, j, ldb_bytes, bits);
            float p = qf * s;
            w[i * ldw + j] = rtz ? orc_f32_to_bf16_rtz(p) : orc_f32_to_bf16_rne(p);
        }
    }
}

/* ---- the reference GEMM: host_ref.hpp ---------------------------------------------------- */

/*
 * gemm_rrr (host_ref.hpp:3-25): row-major A[m,lda], B[k,ldb], C[m,ldc], one fp32 scale per
 * column; for each output, acc starts at 0 and k runs upward; the weight is scaled first
 * (b*scale), then multiplied by a, then added — three separately rounded fp32 operations.
 */
ORC_API void orc_gemm_rrr(float* c, const float* a, const float* b, const float* scale, size_t m, size_t n,
                          size_t k, size_t lda, size_t ldb, size_t ldc)
{
    for (size_t im = 0; im < m; ++im)
        for (size_t in = 0; in < n; ++in) {
            float acc = 0;
            float s = scale[in];
            for (size_t ik = 0; ik < k; ++ik) acc += a[im * lda + ik] * (b[ik * ldb + in] * s);
            c[im * ldc + in] = acc;
        }
}

/*
 * Same arithmetic, same order per output element, but the loops are interchanged so that the
 * innermost walk is along a row of B (contiguous) over a block of columns that each keep their own
 * accumulator.  Every c[m,n] still sees acc = 0; acc += a*(b*s) for k = 0..K-1 in order, so the
 * result equals orc_gemm_rrr bit for bit; only the speed differs.  Used for large parity cases.
 */
#define ORC_NB 512
__attribute__((target_clones("avx2", "default")))
ORC_API void orc_gemm_rrr_fast(float* c, const float* a, const float* b, const float* scale, size_t m,
                               size_t n, size_t k, size_t lda, size_t ldb, size_t ldc)
{
    float acc[ORC_NB];
    for (size_t n0 = 0; n0 < n; n0 += ORC_NB) {
        size_t nb = n - n0 < ORC_NB ? n - n0 : ORC_NB;
        const float* s = scale + n0;
        for (size_t im = 0; im < m; ++im) {
            for (size_t j = 0; j < nb; ++j) acc[j] = 0.0f;
            const float* arow = a + im * lda;
            for (size_t ik = 0; ik < k; ++ik) {
                float av = arow[ik];
                const float* brow = b + ik * ldb + n0;
                for (size_t j = 0; j < nb; ++j) acc[j] += av * (brow[j] * s[j]);
            }
            for (size_t j = 0; j < nb; ++j) c[im * ldc + n0 + j] = acc[j];
        }
    }
}

/*
 * The GEMM oracle for bf16 inputs: gemm_rrr(C, float(A_bf16), float(W_bf16), ones).  With unit
 * scales b*1.0f == b exactly, so this is host_ref.hpp:15-24 fed the values the device really
 * multiplies (bf16 activations, bf16 dequantized weights).  Widening bf16 -> fp32 is exact.
 * Column-blocked like orc_gemm_rrr_fast; per-element operation order is unchanged.
 */
__attribute__((target_clones("avx2", "default")))
ORC_API void orc_gemm_bf16(float* c, const uint16_t* a, const uint16_t* w, size_t m, size_t n, size_t k,
                           size_t lda, size_t ldw, size_t ldc)
{
    float acc[ORC_NB];
    float wrow[ORC_NB];
    for (size_t n0 = 0; n0 < n; n0 += ORC_NB) {
        size_t nb = n - n0 < ORC_NB ? n - n0 : ORC_NB;
        for (size_t im = 0; im < m; ++im) {
            for (size_t j = 0; j < nb; ++j) acc[j] = 0.0f;
            for (size_t ik = 0; ik < k; ++ik) {
                float av = orc_bf16_to_f32(a[im * lda + ik]);
                const uint16_t* wr = w + ik * ldw + n0;
                for (size_t j = 0; j < nb; ++j) {
                    uint32_t u = (uint32_t)wr[j] << 16;
                    memcpy(&wrow[j], &u, 4);
                }
                for (size_t j = 0; j < nb; ++j) acc[j] += av * wrow[j];
            }
            for (size_t j = 0; j < nb; ++j) c[im * ldc + n0 + j] = acc[j];
        }
    }
}

/* fp64-accumulated variant of the same sum, to tell which side of a disagreement is nearer the
 * exact value.  Not a restatement of reference code. */
ORC_API void orc_gemm_bf16_f64(double* c, const uint16_t* a, const uint16_t* w, size_t m, size_t n, size_t k,
                               size_t lda, size_t ldw, size_t ldc)
{
    double acc[ORC_NB];
    for (size_t n0 = 0; n0 < n; n0 += ORC_NB) {
        size_t nb = n - n0 < ORC_NB ? n - n0 : ORC_NB;
        for (size_t im = 0; im < m; ++im) {
            for (size_t j = 0; j < nb; ++j) acc[j] = 0.0;
            for (size_t ik = 0; ik < k; ++ik) {
                double av = (double)orc_bf16_to_f32(a[im * lda + ik]);
                const uint16_t* wr = w + ik * ldw + n0;
                for (size_t j = 0; j < nb; ++j) acc[j] += av * (double)orc_bf16_to_f32(wr[j]);
            }
            for (size_t j = 0; j < nb; ++j) c[im * ldc + n0 + j] = acc[j];
        }
    }
}

/* ---- validation: validation.hpp ---------------------------------------------------------- */

/*
 * valid_vector<bfloat16> (validation.hpp:7-46): fp32 running sums s0 += (r-p)^2 and
 * s1 += 2 r^2 (the 2.0 literal makes that product a double before it is narrowed), a per-element
 * count of |r-p|/r > 1e-3 (division by the signed reference: a zero reference with a zero
 * prediction gives NaN, which does not count; negative references never count), and the verdict
 * sqrt(s0/s1) < nrms && pp_err == 0.  The diagnostics printf of the reference is not reproduced;
 * the counters are returned instead.
 */
ORC_API int orc_valid_vector(const float* ref, const uint16_t* pred, int n, float nrms, int* pp_err_out,
                             float* nrms_out)
{
    float s0 = 0.0f, s1 = 0.0f;
    int pp_err = 0;
    for (int i = 0; i < n; ++i) {
        float ri = ref[i];
        float pi = orc_bf16_to_f32(pred[i]);
        float d = ri - pi;
        float dd = d * d;
        float rr = (float)(2.0 * ri * ri);
        s0 += dd;
        s1 += rr;
        float delta = fabsf(ri - pi) / ri;
        if (delta > 1e-3) pp_err++; /* compared against the double literal, as in the reference */
    }
    if (pp_err_out) *pp_err_out = pp_err;
    if (nrms_out) *nrms_out = sqrtf(s0 / s1);
    return (sqrtf(s0 / s1) < nrms) && (pp_err == 0); /* C++ picks the float overload of sqrt here */
}

/*
 * The build's acceptance criterion for bf16 output (not in the reference): an element passes if
 * |pred - ref| <= max_ulp * ulp_bf16(ref), where ulp_bf16(ref) is the spacing of bf16 numbers in
 * ref's binade (2^(e-7) for 2^e <= |ref| < 2^(e+1), never below the bf16 subnormal spacing), or,
 * where |ref| < small_abs, if |pred - ref| <= small_rel * |ref|.
 * Returns the number of failing elements; reports the worst error in ULPs and its index.
 */
ORC_API long orc_check_ulp(const float* ref, const uint16_t* pred, size_t n, double max_ulp, double small_abs,
                           double small_rel, double* worst_ulp_out, size_t* worst_idx_out)
{
    long bad = 0;
    double worst = 0.0;
    size_t worst_idx = 0;
    for (size_t i = 0; i < n; ++i) {
        double r = (double)ref[i];
        double p = (double)orc_bf16_to_f32(pred[i]);
        double err = fabs(p - r);
        int e;
        double ulp;
        if (r == 0.0) {
            ulp = ldexp(1.0, -133);
        } else {
            frexp(fabs(r), &e); /* |r| = f * 2^e with f in [0.5,1): binade exponent is e-1 */
            int ee = e - 1;
            if (ee < -126) ee = -126;
            ulp = ldexp(1.0, ee - 7);
        }
        double u = err / ulp;
        int ok = (u <= max_ulp) || (fabs(r) < small_abs && err <= small_rel * fabs(r));
        if (!(p == p) || !(r == r)) ok = 0;
        if (!ok) bad++;
        if (u > worst || !(u == u)) {
            worst = u;
            worst_idx = i;
        }
    }
    if (worst_ulp_out) *worst_ulp_out = worst;
    if (worst_idx_out) *worst_idx_out = worst_idx;
    return bad;
}
