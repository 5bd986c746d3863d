// Host build of maidenx_amd/csrc/mathfn.hpp for the CPU tests: compares the backend's exp / tanh /
// expm1 restatements with the platform libm the reference's CPU path calls.
// Build: g++ -O2 -shared -fPIC -fopenmp -ffp-contract=off -mfma (see tests/test_mathfn.py).
#include <cmath>
#include <cstdint>
#include <cstring>

#include "../../maidenx_amd/csrc/mathfn.hpp"

static inline bool same(float a, float b) { return mxh::f2u(a) == mxh::f2u(b) || (a != a && b != b); }

// Walks bit patterns start, start+stride, ... (count of them) and returns the number of inputs
// on which the restatement and libm differ; which: 0 = exp, 1 = tanh, 2 = expm1.
extern "C" long mathfn_mismatches(int which, uint32_t start, uint32_t stride, long count, float* first_bad) {
    long bad = 0;
#pragma omp parallel for reduction(+ : bad) schedule(static)
    for (long i = 0; i < count; ++i) {
        float x = mxh::u2f(start + (uint32_t)i * stride);
        float ref, got;
        if (which == 0) { ref = expf(x); got = mxh::m_exp(x); }
        else if (which == 1) { ref = tanhf(x); got = mxh::m_tanh(x); }
        else { ref = expm1f(x); got = mxh::m_expm1(x); }
        if (!same(ref, got)) {
            ++bad;
#pragma omp critical
            if (first_bad) *first_bad = x;
        }
    }
    return bad;
}

extern "C" void mathfn_eval(int which, const float* x, float* y, long n) {
    for (long i = 0; i < n; ++i)
        y[i] = which == 0 ? mxh::m_exp(x[i]) : which == 1 ? mxh::m_tanh(x[i]) : which == 2 ? mxh::m_expm1(x[i])
             : which == 3 ? mxh::m_pow(x[i], 2.0f) : mxh::m_ln(x[i]);
}
