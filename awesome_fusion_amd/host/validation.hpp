// Acceptance checks of the harness.
// valid_vector<T> keeps the reference's criterion (/root/reference/bfAintBGemm/validation.hpp:7-46):
// NRMS = sqrt(sum (r-p)^2 / sum 2 r^2) below `nrms` AND no element with |r-p|/r > 1e-3 (signed
// division: a zero reference with a zero prediction is NaN and passes, a negative reference never
// fails per element); it prints the same summary line.  valid_vector_ulp is this build's bound for
// bf16 outputs of real-valued data: |r-p| <= max_ulp bf16 ULPs of r, or |r-p| <= small_rel*|r|
// where |r| < small_abs.
#pragma once
#include <cmath>
#include <cstdint>
#include <cstdio>

#include "datatype.hpp"

#define PER_PIXEL_CHECK
#define ASSERT_ON_FAIL

template <typename T>
inline bool valid_vector(const float* ref, const T* pred, int n, float nrms = 1e-3)
{
    float s0 = 0.0f, s1 = 0.0f;
    int pp_err = 0;
    for (int i = 0; i < n; ++i) {
        const float ri = ref[i];
        const float pi = type_convert<float>(pred[i]);
        const float d = ri - pi;
        s0 += d * d;
        s1 += static_cast<float>(2.0 * ri * ri);
#ifdef PER_PIXEL_CHECK
        const float delta = std::fabs(ri - pi) / ri;
        if (delta > 1e-3) {
#ifdef ASSERT_ON_FAIL
            if (pp_err < 100) std::printf("diff at %4d, ref:%lf, pred:%lf(0x%04x), d:%lf\n", i, ri, pi, (unsigned)pred[i], delta);
#endif
            pp_err++;
        }
#endif
    }
    std::printf("pp_crr:%d, pp_err:%d, crr_ratio:%.3f, nrms:%lf, s0:%lf, s1:%lf\n", n - pp_err, pp_err,
                (float)(n - pp_err) / (float)n, (float)std::sqrt((float)(s0 / s1)), s0, s1);
    return (std::sqrt(s0 / s1) < nrms) && (pp_err == 0);
}

struct UlpReport {
    long failing = 0;
    long cancelling = 0;  // outside the plain bound, inside the bound widened by the summation noise
    double worst_ulp = 0.0;
    long worst_index = 0;
};

// `noise`, if given, is a per-element bound on what the rounding of an fp32 sum may contribute on either
// side (the caller passes a few times 2^-24 * sum_k |a*w| for outputs near zero, and 0 elsewhere): an output
// that cancels to almost nothing can differ from the reference by more than two of ITS ULPs whatever order
// the device adds in.  Such elements are counted separately; the caller decides how many it tolerates.
inline UlpReport valid_vector_ulp(const float* ref, const bfloat16* pred, long n, double max_ulp = 2.0, double small_abs = 1e-3,
                                  double small_rel = 1e-2, const float* noise = nullptr)
{
    UlpReport rep;
    for (long i = 0; i < n; ++i) {
        const double r = ref[i], p = type_convert<float>(pred[i]);
        const double err = std::fabs(p - r);
        int e = 0;
        double ulp = std::ldexp(1.0, -133);
        if (r != 0.0) {
            (void)std::frexp(std::fabs(r), &e);
            ulp = std::ldexp(1.0, (e - 1 < -126 ? -126 : e - 1) - 7);
        }
        const double u = err / ulp;
        bool ok = (u <= max_ulp) || (std::fabs(r) < small_abs && err <= small_rel * std::fabs(r));
        if (!(p == p) || !(r == r)) ok = false;
        else if (!ok && noise != nullptr && err <= max_ulp * ulp + noise[i]) { ok = true; rep.cancelling++; }
        if (!ok) rep.failing++;
        if (u > rep.worst_ulp || !(u == u)) { rep.worst_ulp = u; rep.worst_index = i; }
    }
    return rep;
}
