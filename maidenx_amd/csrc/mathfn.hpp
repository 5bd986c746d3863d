// f32 math used by the elementwise kernels.
//
// The reference's CPU backend calls the platform libm (glibc expf/tanhf/powf...) through
// Rust's f32 methods.  These kernels are HBM-bound, so the transcendental functions are
// evaluated in f64 and rounded once: the result is the correctly rounded f32 value except
// for inputs whose exact result lies within ~1e-12 (relative) of a rounding boundary, which
// keeps it within 1 ulp of any libm whose own error is below 1 ulp.
// Everything here compiles for host and device so it can be checked on the CPU.
#pragma once
#include <cmath>
#include <cstdint>

#if defined(__HIPCC__)
#define MXH_HD __host__ __device__ inline
#else
#define MXH_HD inline
#endif

namespace mxh {

MXH_HD double bits2d(uint64_t b) {
    union { uint64_t u; double d; } c;
    c.u = b;
    return c.d;
}

// exp(r) for |r| <= 0.35 : Taylor to degree 11 (truncation below 1e-14 relative)
MXH_HD double exp_poly(double r) {
    double p = 1.0 / 39916800.0;
    p = fma(p, r, 1.0 / 3628800.0);
    p = fma(p, r, 1.0 / 362880.0);
    p = fma(p, r, 1.0 / 40320.0);
    p = fma(p, r, 1.0 / 5040.0);
    p = fma(p, r, 1.0 / 720.0);
    p = fma(p, r, 1.0 / 120.0);
    p = fma(p, r, 1.0 / 24.0);
    p = fma(p, r, 1.0 / 6.0);
    p = fma(p, r, 0.5);
    p = fma(p, r, 1.0);
    p = fma(p, r, 1.0);
    return p;
}

// e^x as a double, for |x| < 700
MXH_HD double exp_d(double x) {
    double n = rint(x * 1.4426950408889634);
    double r = fma(-n, 0.6931471803691238, x);      // ln2 high part (its low 21 bits are zero)
    r = fma(-n, 1.9082149292705877e-10, r);         // ln2 low part
    double s = bits2d((uint64_t)(1023 + (int64_t)n) << 52);
    return exp_poly(r) * s;
}

MXH_HD float m_exp(float x) {
    if (!(x == x)) return x + x;
    if (x > 89.0f) return INFINITY;
    if (x < -104.0f) return 0.0f;
    return (float)exp_d((double)x);
}

MXH_HD float m_tanh(float x) {
    if (!(x == x)) return x + x;
    double a = fabs((double)x);
    double t;
    if (a < 0.02) {
        double a2 = a * a;   // odd Taylor series, truncation below 1e-15 relative here
        t = a * fma(a2, fma(a2, fma(a2, fma(a2, 62.0 / 2835.0, -17.0 / 315.0), 2.0 / 15.0), -1.0 / 3.0), 1.0);
    } else if (a < 20.0) {
        double e = exp_d(2.0 * a);
        t = 1.0 - 2.0 / (e + 1.0);
    } else {
        t = 1.0;
    }
    float r = (float)t;
    return x < 0.0f ? -r : r;
}

MXH_HD float m_pow(float x, float c) { return (float)pow((double)x, (double)c); }
MXH_HD float m_ln(float x) { return (float)log((double)x); }
MXH_HD float m_log2(float x) { return (float)log2((double)x); }
MXH_HD float m_log10(float x) { return (float)log10((double)x); }
MXH_HD float m_sin(float x) { return (float)sin((double)x); }
MXH_HD float m_cos(float x) { return (float)cos((double)x); }
MXH_HD float m_tan(float x) { return (float)tan((double)x); }
MXH_HD float m_exp2(float x) { return (float)exp2((double)x); }

}  // namespace mxh
