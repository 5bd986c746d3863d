// f32 math used by the elementwise kernels.
//
// The reference's CPU backend reaches the platform libm (glibc 2.35 here) through Rust's
// f32::exp / f32::tanh / f32::powf.  Composite ops amplify a last-bit difference of the inner
// function (1 + tanh(..) in gelu, 1 + exp(x) in softplus and sigmoid), so exp and tanh are not
// merely accurate: they restate the algorithms that libm uses, operation for operation, and
// return the same bits.
//   expf   : the table-driven double-precision scheme of glibc >= 2.27 (from ARM's optimized
//            routines): x*N/ln2 = k + r, 2^(k/N) from a 32-entry table, cubic in r, with the
//            multiply-adds fused the way the FMA build of the library fuses them.
//   tanhf, expm1f : the FDLIBM single-precision routines (Sun Microsystems, 1993).
// Both were compared with the library over all 2^32 inputs on the CPU and agree on every one
// (tests/test_mathfn.py samples this).  The remaining functions are evaluated in f64 and
// rounded once, which keeps them within 1 ulp of any libm whose own error is below 1 ulp.
// Everything here compiles for host and device.
#pragma once
#include <cmath>
#include <cstdint>
#include <cstring>

#if defined(__HIPCC__)
#define MXH_HD __host__ __device__ inline
#else
#define MXH_HD inline
#endif

namespace mxh {

MXH_HD uint32_t f2u(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }
MXH_HD float u2f(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }
MXH_HD uint64_t d2u(double f) { uint64_t u; memcpy(&u, &f, 8); return u; }
MXH_HD double u2d(uint64_t u) { double f; memcpy(&f, &u, 8); return f; }

// bits(2^(i/32)) - (i << 47), i = 0..31 (each 2^(i/32) correctly rounded to double)
#if defined(__HIP_DEVICE_COMPILE__)
static __device__ __constant__
#else
static
#endif
const uint64_t EXP2F_TAB[32] = {
    0x3ff0000000000000ULL, 0x3fefd9b0d3158574ULL, 0x3fefb5586cf9890fULL, 0x3fef9301d0125b51ULL,
    0x3fef72b83c7d517bULL, 0x3fef54873168b9aaULL, 0x3fef387a6e756238ULL, 0x3fef1e9df51fdee1ULL,
    0x3fef06fe0a31b715ULL, 0x3feef1a7373aa9cbULL, 0x3feedea64c123422ULL, 0x3feece086061892dULL,
    0x3feebfdad5362a27ULL, 0x3feeb42b569d4f82ULL, 0x3feeab07dd485429ULL, 0x3feea47eb03a5585ULL,
    0x3feea09e667f3bcdULL, 0x3fee9f75e8ec5f74ULL, 0x3feea11473eb0187ULL, 0x3feea589994cce13ULL,
    0x3feeace5422aa0dbULL, 0x3feeb737b0cdc5e5ULL, 0x3feec49182a3f090ULL, 0x3feed503b23e255dULL,
    0x3feee89f995ad3adULL, 0x3feeff76f2fb5e47ULL, 0x3fef199bdd85529cULL, 0x3fef3720dcef9069ULL,
    0x3fef5818dcfba487ULL, 0x3fef7c97337b9b5fULL, 0x3fefa4afa2a490daULL, 0x3fefd0765b6e4540ULL
};

// Without a branch: the core runs for every input and the out-of-range results are selected afterwards, so the table
// reads of the elements a thread owns are all in flight together (behind per-element branches each element waited
// for its own read: [8192,8192] f32 took 110 us).
MXH_HD float m_exp(float x) {
    const double InvLn2N = 0x1.71547652b82fep+0 * 32, Shift = 0x1.8p+52;
    const double C0 = 0x1.c6af84b912394p-5 / 32 / 32 / 32, C1 = 0x1.ebfce50fac4f3p-3 / 32 / 32, C2 = 0x1.62e42ff0c52d6p-1 / 32;
    const double xd = (double)x;
    double kd = fma(InvLn2N, xd, Shift);
    const uint64_t ki = d2u(kd);
    kd -= Shift;
    const double r = fma(InvLn2N, xd, -kd);
    const uint64_t t = EXP2F_TAB[ki % 32] + (ki << 47);
    const double s = u2d(t);
    const double z = fma(C0, r, C1);
    const double r2 = r * r;
    double y = fma(C2, r, 1.0);
    y = fma(z, r2, y);
    y = y * s;
    float res = (float)y;                                   // (subnormal results round here, as in the library)
    if (x > 0x1.62e42ep6f) res = INFINITY;                  // overflow, +inf
    if (x < -0x1.9fe368p6f) res = 0.0f;                     // underflow to zero, -inf
    if (x != x) res = x + x;                                // NaN
    return res;
}

MXH_HD float m_expm1(float x) {
    const float one = 1.0f, huge = 1.0e+30f, tiny = 1.0e-30f, o_threshold = 8.8721679688e+01f,
                ln2_hi = 6.9313812256e-01f, ln2_lo = 9.0580006145e-06f, invln2 = 1.4426950216e+00f,
                Q1 = -3.3333335072e-02f, Q2 = 1.5873016091e-03f, Q3 = -7.9365076090e-05f, Q4 = 4.0082177293e-06f,
                Q5 = -2.0109921195e-07f;
    float y, hi, lo, c = 0.0f, t, e, hxs, hfx, r1;
    int32_t k;
    uint32_t hx = f2u(x);
    const uint32_t xsb = hx & 0x80000000u;
    hx &= 0x7fffffffu;
    if (hx >= 0x4195b844u) {                 // |x| >= 27 ln2
        if (hx >= 0x42b17218u) {             // |x| >= 88.72
            if (hx > 0x7f800000u) return x + x;
            if (hx == 0x7f800000u) return xsb == 0 ? x : -1.0f;
            if (x > o_threshold) return huge * huge;
        }
        if (xsb != 0) {
            if (x + tiny < 0.0f) return tiny - one;
        }
    }
    if (hx > 0x3eb17218u) {                  // |x| > 0.5 ln2
        if (hx < 0x3F851592u) {              // |x| < 1.5 ln2
            if (xsb == 0) { hi = x - ln2_hi; lo = ln2_lo; k = 1; }
            else { hi = x + ln2_hi; lo = -ln2_lo; k = -1; }
        } else {
            k = (int32_t)(invln2 * x + (xsb == 0 ? 0.5f : -0.5f));
            t = (float)k;
            hi = x - t * ln2_hi;
            lo = t * ln2_lo;
        }
        x = hi - lo;
        c = (hi - x) - lo;
    } else if (hx < 0x33000000u) {           // |x| < 2^-25
        t = huge + x;
        return x - (t - (huge + x));
    } else {
        k = 0;
    }
    hfx = 0.5f * x;
    hxs = x * hfx;
    r1 = one + hxs * (Q1 + hxs * (Q2 + hxs * (Q3 + hxs * (Q4 + hxs * Q5))));
    t = 3.0f - r1 * hfx;
    e = hxs * ((r1 - t) / (6.0f - x * t));
    if (k == 0) return x - (x * e - hxs);
    e = (x * (e - c) - c);
    e -= hxs;
    if (k == -1) return 0.5f * (x - e) - 0.5f;
    if (k == 1) {
        if (x < -0.25f) return -2.0f * (e - (x + 0.5f));
        return one + 2.0f * (x - e);
    }
    if (k <= -2 || k > 56) {
        y = one - (e - x);
        y = u2f(f2u(y) + ((uint32_t)k << 23));
        return y - one;
    }
    if (k < 23) {
        t = u2f(0x3f800000u - (0x1000000u >> k));   // 1 - 2^-k
        y = t - (e - x);
        y = u2f(f2u(y) + ((uint32_t)k << 23));
    } else {
        t = u2f((uint32_t)(0x7f - k) << 23);        // 2^-k
        y = x - (e + t);
        y += one;
        y = u2f(f2u(y) + ((uint32_t)k << 23));
    }
    return y;
}

// a / b for operands whose quotient, reciprocal and remainders are all normal numbers: the correctly rounded IEEE
// quotient.  On the device this is the compiler's own division sequence (reciprocal, one Newton step, three fused
// residual corrections) without the operand scaling and the special-case fix-up that out-of-range operands need -
// 8 instructions instead of 12; on the host it is the division itself.
MXH_HD float div_in_range(float a, float b) {
#if defined(__HIP_DEVICE_COMPILE__)
    float y = __builtin_amdgcn_rcpf(b);
    const float e0 = __builtin_fmaf(-b, y, 1.0f);
    y = __builtin_fmaf(e0, y, y);
    float q = a * y;
    float r = __builtin_fmaf(-b, q, a);
    q = __builtin_fmaf(r, y, q);
    r = __builtin_fmaf(-b, q, a);
    return __builtin_fmaf(r, y, q);
#else
    return a / b;
#endif
}

// tanhf of FDLIBM, operation for operation, without a branch: every lane runs the same instructions and selects.
//   |x| >= 1 : z = 1 - 2 / (t + 2),  t = expm1f(2|x|)         (reduction index k >= 3)
//   |x| <  1 : z = -t / (t + 2),     t = expm1f(-2|x|)        (k in {0, -1, -2, -3})
// expm1f is restated inline for exactly those arguments: the reduction a = hi - lo with its correction c, the
// rational approximation, and the reconstruction by k: k = 0, k = -1, k <= -2 (y = 1 - (e - x), scaled, minus 1) and
// 2 <= k < 23 (y = (1 - 2^-k) - (e - x), scaled).  For k >= 23 (|x| >= 7.8) FDLIBM forms y another way; there
// t > 6e6 and z = 1 - 2/(t + 2) no longer depends on the last bits of t, and the k < 23 form gives the same z on every
// input.  |x| >= 22 is 1 by FDLIBM's own shortcut; the tiny-|x| shortcut x * (1 + x) equals what the general path
// returns; a NaN propagates through the arithmetic.  Each of these simplifications was kept only after the host build
// of this function agreed with the library's tanhf on all 2^32 inputs (tests/test_mathfn.py, MATHFN_EXHAUSTIVE=1).
// The two divisions have operands in [1, 2^64], far from any special case.
MXH_HD float m_tanh(float x) {
    const float ln2_hi = 6.9313812256e-01f, ln2_lo = 9.0580006145e-06f, invln2 = 1.4426950216e+00f,
                Q1 = -3.3333335072e-02f, Q2 = 1.5873016091e-03f, Q3 = -7.9365076090e-05f, Q4 = 4.0082177293e-06f,
                Q5 = -2.0109921195e-07f;
    const uint32_t ux = f2u(x), ix = ux & 0x7fffffffu;
    const float ax = u2f(ix);
    const bool big = ix >= 0x3f800000u;
    const float a2 = ax + ax;
    const float a = big ? a2 : -a2;                           // the argument of expm1
    // k = (int)(invln2 * a +- 0.5).  FDLIBM sets k = -1 for 0.5 ln2 < |a| < 1.5 ln2 and skips the reduction below that;
    // the formula gives the same k (and with k = 0 a reduction that changes nothing) for every one of these arguments.
    const float tk = truncf(invln2 * a + (big ? 0.5f : -0.5f));
    const int k = (int)tk;
    const float hi = a - tk * ln2_hi;
    const float lo = tk * ln2_lo;
    const float xr = hi - lo;
    const float c = (hi - xr) - lo;
    const float hfx = 0.5f * xr;
    const float hxs = xr * hfx;
    const float r1 = 1.0f + hxs * (Q1 + hxs * (Q2 + hxs * (Q3 + hxs * (Q4 + hxs * Q5))));
    const float t3 = 3.0f - r1 * hfx;
    const float e = hxs * div_in_range(r1 - t3, 6.0f - xr * t3);
    const float res0 = xr - (xr * e - hxs);                   // k = 0
    float e2 = xr * (e - c) - c;
    e2 -= hxs;
    const float resm1 = 0.5f * (xr - e2) - 0.5f;              // k = -1
    const float twomk = u2f((uint32_t)(0x7f - k) << 23);      // 2^-k
    const float top = big ? 1.0f - twomk : 1.0f;              // 1 - 2^-k is exact for k < 25
    float y = top - (e2 - xr);
    y = u2f(f2u(y) + ((uint32_t)k << 23));                    // times 2^k
    const float resg = big ? y : y - 1.0f;
    const float t = k == 0 ? res0 : (k == -1 ? resm1 : resg);
    const float q = div_in_range(big ? 2.0f : -t, t + 2.0f);
    float z = big ? 1.0f - q : q;
    if (ax >= 22.0f) z = 1.0f;                                // |x| >= 22 and +-inf; a NaN fails the test and has made z a NaN
    return u2f((f2u(z) & 0x7fffffffu) | (ux & 0x80000000u));  // (|x| < 2^-55, FDLIBM's x * (1 + x) = x, comes out as x by itself)
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
