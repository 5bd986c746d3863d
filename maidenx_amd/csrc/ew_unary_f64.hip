// Unary entry points for f64 and bool (crates/maidenx_cuda/src/ops/unary.rs:97-104, 152-159); see ops_wide.hpp for
// which forms are built.
#include "ops_wide.hpp"

MXH_WIDE_SIGNED(double, f64)
MXH_WU(relu, WRelu, double, double, f64, double)
MXH_WU(recip, WRecip, double, double, f64, double)
MXH_WUC(leaky_relu, WLeakyRelu, double, double, f64, double)
MXH_WU(sigmoid, WSigmoid, double, double, f64, double) MXH_WU(tanh, WTanh, double, double, f64, double)
MXH_WU(gelu, WGelu, double, double, f64, double) MXH_WU(sin, WSin, double, double, f64, double)
MXH_WU(cos, WCos, double, double, f64, double) MXH_WU(tan, WTan, double, double, f64, double)
MXH_WU(ln, WLn, double, double, f64, double) MXH_WU(log10, WLog10, double, double, f64, double)
MXH_WU(log2, WLog2, double, double, f64, double) MXH_WU(exp, WExp, double, double, f64, double)
MXH_WU(exp10, WExp10, double, double, f64, double) MXH_WU(exp2, WExp2, double, double, f64, double)
MXH_WU(softplus, WSoftplus, double, double, f64, double)
MXH_WUC(elu, WElu, double, double, f64, double)      // (pow comes with MXH_WIDE_SIGNED)

MXH_WIDE_COMMON(mxh::b8_t, uint8_t, bool)
MXH_WU(neg, WNeg, mxh::b8_t, uint8_t, bool, uint8_t)
MXH_WU(abs, WSame, mxh::b8_t, uint8_t, bool, uint8_t)
MXH_WU(sign, WSame, mxh::b8_t, uint8_t, bool, uint8_t)
MXH_WU(square, WSame, mxh::b8_t, uint8_t, bool, uint8_t)
MXH_WU(sqrt, WSame, mxh::b8_t, uint8_t, bool, uint8_t)
MXH_WU(relu, WSame, mxh::b8_t, uint8_t, bool, uint8_t)
MXH_WU(sigmoid, WSame, mxh::b8_t, uint8_t, bool, uint8_t)
MXH_WU(tanh, WSame, mxh::b8_t, uint8_t, bool, uint8_t)
MXH_WUC(pow, WPow, mxh::b8_t, uint8_t, bool, uint8_t)
