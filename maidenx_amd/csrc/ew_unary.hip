// extern "C" entry points of the unary families (plain, with a by-value constant, and the
// bool-producing forms).  Each replaces the `cuda_<op>_<dtype>` symbol of
// crates/maidenx_cuda/src/ops/unary.rs:21-77; a null input means "in place on the output"
// (crates/maidenx_cuda/kernels/ops/unary.cu:20).
#include "elementwise.hpp"
#include "lut16.hpp"
#include "ops.hpp"

using namespace mxh;

static inline float F_host(float v) { return v; }
static inline float F_host(bf16_t v) { return bf2f(v); }
static inline float F_host(f16_t v) { return h2f(v); }

#define MXH_UNARY(NAME, OP, T, SUF, O)                                                                        \
    extern "C" void hip_##NAME##_##SUF(size_t num_els, size_t num_dims, const size_t* md, const T* in, O* out) { MXH_API; \
        ew_unary(num_els, num_dims, md, in, out, OP<T>{});                                                    \
    }
// The long-running functions: for the 16-bit dtypes a large call is a table lookup (lut16.hpp), f32 always computes.
template <class Op>
static inline bool by_table(size_t num_els, size_t num_dims, const size_t* md, const void* in, void* out) {
    if constexpr (sizeof(typename Op::In) == 2) return lut16_unary<Op>(num_els, num_dims, md, in, out);
    else return false;
}
#define MXH_UNARY_L(NAME, OP, T, SUF, O)                                                                      \
    extern "C" void hip_##NAME##_##SUF(size_t num_els, size_t num_dims, const size_t* md, const T* in, O* out) { MXH_API; \
        if (by_table<OP<T>>(num_els, num_dims, md, in, out)) return;                                          \
        ew_unary(num_els, num_dims, md, in, out, OP<T>{});                                                    \
    }
#define MXH_UNARY_C(NAME, OP, T, SUF, O)                                                                      \
    extern "C" void hip_##NAME##_##SUF(size_t num_els, size_t num_dims, const size_t* md, const T* in, T c,   \
                                       O* out) { MXH_API;                                                     \
        ew_unary(num_els, num_dims, md, in, out, OP<T>{c});                                                   \
    }

// x^2 (the square of MSE and variance) is the product: a product of two floats is exact in double, so rounding it
// once is bit for bit what the double pow() path returns - without the 200 instructions of pow.  x^1 (the factor
// x^(c-1) in the backward of that square) is x.
#define MXH_POW(T, SUF)                                                                                       \
    extern "C" void hip_pow_##SUF(size_t num_els, size_t num_dims, const size_t* md, const T* in, T c, T* out) { MXH_API; \
        if (F_host(c) == 2.0f) ew_unary(num_els, num_dims, md, in, out, OpSquare<T>{});                       \
        else if (F_host(c) == 1.0f) ew_unary(num_els, num_dims, md, in, out, OpIdentity<T>{});                \
        else ew_unary(num_els, num_dims, md, in, out, OpPow<T>{c});                                           \
    }

#define MXH_ALL_FOR(T, SUF)                                                                                   \
    MXH_UNARY(neg, OpNeg, T, SUF, T) MXH_UNARY(abs, OpAbs, T, SUF, T) MXH_UNARY(sign, OpSign, T, SUF, T)      \
    MXH_UNARY(square, OpSquare, T, SUF, T) MXH_UNARY(sqrt, OpSqrt, T, SUF, T)                                 \
    MXH_UNARY(relu, OpRelu, T, SUF, T) MXH_UNARY_L(sigmoid, OpSigmoid, T, SUF, T)                             \
    MXH_UNARY_L(tanh, OpTanh, T, SUF, T) MXH_UNARY_L(gelu, OpGelu, T, SUF, T)                                 \
    MXH_UNARY_L(sin, OpSin, T, SUF, T) MXH_UNARY_L(cos, OpCos, T, SUF, T) MXH_UNARY_L(tan, OpTan, T, SUF, T)  \
    MXH_UNARY_L(ln, OpLn, T, SUF, T) MXH_UNARY_L(log10, OpLog10, T, SUF, T) MXH_UNARY_L(log2, OpLog2, T, SUF, T) \
    MXH_UNARY_L(exp, OpExp, T, SUF, T) MXH_UNARY_L(exp10, OpExp10, T, SUF, T) MXH_UNARY_L(exp2, OpExp2, T, SUF, T) \
    MXH_UNARY_L(softplus, OpSoftplus, T, SUF, T) MXH_UNARY(recip, OpRecip, T, SUF, T)                         \
    MXH_UNARY(logical_not, OpLogicalNot, T, SUF, bool_t)                                                      \
    MXH_UNARY_C(add_scalar, OpAddScalar, T, SUF, T) MXH_UNARY_C(sub_scalar, OpSubScalar, T, SUF, T)           \
    MXH_UNARY_C(mul_scalar, OpMulScalar, T, SUF, T) MXH_UNARY_C(div_scalar, OpDivScalar, T, SUF, T)           \
    MXH_UNARY_C(maximum_scalar, OpMaximumScalar, T, SUF, T) MXH_UNARY_C(minimum_scalar, OpMinimumScalar, T, SUF, T) \
    MXH_POW(T, SUF) MXH_UNARY_C(leaky_relu, OpLeakyRelu, T, SUF, T)                                           \
    MXH_UNARY_C(elu, OpElu, T, SUF, T)                                                                        \
    MXH_UNARY_C(eq_scalar, OpEqScalar, T, SUF, bool_t) MXH_UNARY_C(ne_scalar, OpNeScalar, T, SUF, bool_t)     \
    MXH_UNARY_C(lt_scalar, OpLtScalar, T, SUF, bool_t) MXH_UNARY_C(le_scalar, OpLeScalar, T, SUF, bool_t)     \
    MXH_UNARY_C(gt_scalar, OpGtScalar, T, SUF, bool_t) MXH_UNARY_C(ge_scalar, OpGeScalar, T, SUF, bool_t)

namespace mxh {
const uint16_t* lut16_exp_bf16() { return lut16_table<OpExp<bf16_t>>(); }
const uint16_t* lut16_exp_f16() { return lut16_table<OpExp<f16_t>>(); }
}  // namespace mxh

MXH_ALL_FOR(float, f32)
MXH_ALL_FOR(bf16_t, bf16)
MXH_ALL_FOR(f16_t, f16)
