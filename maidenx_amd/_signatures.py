"""ctypes signatures of the `<prefix><op>_<dtype>` symbol families declared in include/maidenx_hip.h.

The same table describes the reference's CPU symbols (crates/maidenx_cpu/src/ops/*.rs), which have
identical argument lists, so a CPU restatement built with another prefix can be bound with it too.
"""
import ctypes as C

SZ, P = C.c_size_t, C.c_void_p
CONST = {"f32": C.c_float, "f64": C.c_double, "bf16": C.c_uint16, "f16": C.c_uint16, "bool": C.c_uint8,
         "u8": C.c_uint8, "u16": C.c_uint16, "u32": C.c_uint32, "u64": C.c_uint64,
         "i8": C.c_int8, "i16": C.c_int16, "i32": C.c_int32, "i64": C.c_int64}

BINARY = ["add", "sub", "mul", "div", "maximum", "minimum", "logical_and", "logical_or", "logical_xor",
          "eq", "ne", "lt", "le", "gt", "ge"]
INPLACE = ["add_inplace", "sub_inplace", "mul_inplace", "div_inplace"]
UNARY = ["neg", "abs", "sign", "square", "sqrt", "relu", "sigmoid", "tanh", "gelu", "sin", "cos", "tan", "ln",
         "log10", "log2", "exp", "exp10", "exp2", "softplus", "recip", "logical_not"]
UNARY_CONST = ["add_scalar", "sub_scalar", "mul_scalar", "div_scalar", "maximum_scalar", "minimum_scalar", "pow",
               "leaky_relu", "elu", "eq_scalar", "ne_scalar", "lt_scalar", "le_scalar", "gt_scalar", "ge_scalar"]
REDUCE = ["sum", "mean", "max", "min"]
BOOL_OUT = {"logical_and", "logical_or", "logical_xor", "eq", "ne", "lt", "le", "gt", "ge", "logical_not",
            "eq_scalar", "ne_scalar", "lt_scalar", "le_scalar", "gt_scalar", "ge_scalar"}


def signatures(dtypes=("f32", "bf16", "f16")):
    """name (without prefix) -> argtypes list."""
    sig = {}
    for dt in dtypes:
        c = CONST[dt]
        for op in BINARY:
            sig[f"{op}_{dt}"] = [SZ, SZ, P, P, P, P]
        for op in INPLACE:
            sig[f"{op}_{dt}"] = [SZ, SZ, P, P, P]
        for op in UNARY:
            sig[f"{op}_{dt}"] = [SZ, SZ, P, P, P]
        for op in UNARY_CONST:
            sig[f"{op}_{dt}"] = [SZ, SZ, P, P, c, P]
        for op in REDUCE:
            sig[f"{op}_{dt}"] = [SZ, SZ, SZ, P, P, P]
        sig[f"sum_to_shape_{dt}"] = [SZ, SZ, P, P, P]
        sig[f"fold_{dt}"] = [SZ, SZ, P, P, P]
        sig[f"softmax_{dt}"] = [SZ, SZ, SZ, P, P, P]
        for mode in ("reflection", "replication"):
            sig[f"pad_with_{mode}_{dt}"] = [SZ, SZ, SZ, P, P, P]
            sig[f"pad_with_{mode}_backward_{dt}"] = [SZ, SZ, SZ, P, P, P]
        sig[f"matmul_{dt}"] = [SZ, P, P, P, P]
        sig[f"matmul_backward_{dt}"] = [SZ, SZ, P, P, P, P, P, P]
        sig[f"pad_with_constant_{dt}"] = [SZ, SZ, SZ, P, P, P, c]
        sig[f"pad_with_constant_backward_{dt}"] = [SZ, SZ, SZ, P, P, P]
        sig[f"conv2d_im2col_{dt}"] = [SZ, P, P, P]
        sig[f"conv2d_col2im_{dt}"] = [SZ, P, P, P]
    return sig


WIDE_DTYPES = ("f64", "bool", "u8", "u16", "u32", "u64", "i8", "i16", "i32", "i64")


def binary_signatures(dtypes=WIDE_DTYPES):
    """The binary / comparison / logical / in-place families for the dtypes that only they cover so far."""
    sig = {}
    for dt in dtypes:
        for op in BINARY:
            sig[f"{op}_{dt}"] = [SZ, SZ, P, P, P, P]
        for op in INPLACE:
            sig[f"{op}_{dt}"] = [SZ, SZ, P, P, P]
    return sig


PLAIN_DTYPES = ("f32", "f64", "bool", "u8", "u16", "u32", "u64", "i8", "i16", "i32", "i64")


def cast_signatures():
    """Conversions between every pair of the plain-number dtypes."""
    return {f"cast_{a}_{b}": [SZ, P, P] for a in PLAIN_DTYPES for b in PLAIN_DTYPES if a != b}


def wide_util_signatures():
    """fill / copy_strided for the dtypes beyond f32, bf16, f16 (fill_bool is with those)."""
    sig = {}
    for dt in WIDE_DTYPES:
        if dt != "bool":
            sig[f"fill_{dt}"] = [SZ, P, CONST[dt]]
        sig[f"copy_strided_{dt}"] = [SZ, SZ, P, P, P]
    return sig


WIDE_CONST_OPS = ["add_scalar", "sub_scalar", "mul_scalar", "div_scalar", "maximum_scalar", "minimum_scalar",
                  "eq_scalar", "ne_scalar", "lt_scalar", "le_scalar", "gt_scalar", "ge_scalar"]


def wide_unary_ops(dt):
    """(plain ops, ops with a constant) built for a dtype beyond f32 / bf16 / f16."""
    plain, const = ["logical_not"], list(WIDE_CONST_OPS)
    if dt == "bool":
        plain += ["neg", "abs", "sign", "square", "sqrt", "relu", "sigmoid", "tanh"]
        const += ["pow"]
    else:
        plain += ["sign", "square", "sqrt"]
        if dt != "f64":
            const += ["pow"]
        if dt[0] in "if":
            plain += ["neg", "abs"]
        if dt == "f64":
            plain += ["relu", "recip", "sigmoid", "tanh", "gelu", "sin", "cos", "tan", "ln", "log10", "log2", "exp", "exp10", "exp2", "softplus"]
            const += ["leaky_relu", "pow", "elu"]
    return plain, const


def wide_unary_signatures(dtypes=WIDE_DTYPES):
    sig = {}
    for dt in dtypes:
        plain, const = wide_unary_ops(dt)
        for op in plain:
            sig[f"{op}_{dt}"] = [SZ, SZ, P, P, P]
        for op in const:
            sig[f"{op}_{dt}"] = [SZ, SZ, P, P, CONST[dt], P]
    return sig


REDUCE_WIDE_DTYPES = ("f64", "u8", "u16", "u32", "u64", "i8", "i16", "i32", "i64")


def wide_reduce_signatures(dtypes=REDUCE_WIDE_DTYPES):
    """sum / max / min / sum_to_shape and matmul / matmul_backward for f64 and the integers, mean for f64."""
    sig = {}
    for dt in dtypes:
        for op in ("sum", "max", "min") + (("mean",) if dt == "f64" else ()):
            sig[f"{op}_{dt}"] = [SZ, SZ, SZ, P, P, P]
        sig[f"sum_to_shape_{dt}"] = [SZ, SZ, P, P, P]
        sig[f"matmul_{dt}"] = [SZ, P, P, P, P]
        sig[f"matmul_backward_{dt}"] = [SZ, SZ, P, P, P, P, P, P]
        sig[f"fold_{dt}"] = [SZ, SZ, P, P, P]
        sig[f"pad_with_constant_{dt}"] = [SZ, SZ, SZ, P, P, P, CONST[dt]]
        sig[f"pad_with_constant_backward_{dt}"] = [SZ, SZ, SZ, P, P, P]
        for mode in ("reflection", "replication"):
            sig[f"pad_with_{mode}_{dt}"] = [SZ, SZ, SZ, P, P, P]
            sig[f"pad_with_{mode}_backward_{dt}"] = [SZ, SZ, SZ, P, P, P]
        if dt == "f64":
            sig["softmax_f64"] = [SZ, SZ, SZ, P, P, P]
            sig["conv2d_im2col_f64"] = [SZ, P, P, P]
            sig["conv2d_col2im_f64"] = [SZ, P, P, P]
    return sig


INDEX_WIDE_DTYPES = ("bool", "u8", "u16", "u32", "u64", "i8", "i16", "i32", "i64")


def index_signatures(dtypes=("f32", "bf16", "f16", "f64"), wide=INDEX_WIDE_DTYPES):
    """Index ops (host loops in the reference's tensor layer, device entry points here).  `wide`: the dtypes that have
    everything but the weighted bincount (whose weights are floats)."""
    sig = {}
    for dt in tuple(dtypes) + tuple(wide):
        for it in ("i32", "i64"):
            sig[f"index_select_{dt}_{it}"] = [SZ, SZ, P, SZ, SZ, SZ, P, P, P]
            sig[f"gather_{dt}_{it}"] = [SZ, SZ, P, P, P, P, P]
            sig[f"index_add_{dt}_{it}"] = [SZ, SZ, P, P, SZ, SZ, SZ, P, P, P]
            sig[f"scatter_add_{dt}_{it}"] = [SZ, SZ, P, P, P, P, P, P]
            if dt in dtypes:
                sig[f"bincount_weighted_{dt}_{it}"] = [SZ, SZ, SZ, P, SZ, SZ, P, SZ, P]
        sig[f"index_put_{dt}"] = [SZ, P, SZ, P, SZ, P, P, P]
    for it in ("i32", "i64"):
        sig[f"bincount_{it}"] = [SZ, SZ, SZ, P, SZ, P]
    return sig


def extension_signatures():
    """Entry points of the HIP library that have no counterpart symbol in the reference."""
    sig = index_signatures()
    for dt in ("f32", "bf16", "f16", "bool"):
        sig[f"fill_{dt}"] = [SZ, P, CONST[dt]]
    for dt in ("f32", "bf16", "f16"):
        sig[f"copy_strided_{dt}"] = [SZ, SZ, P, P, P]
        sig[f"adam_step_{dt}"] = [SZ, P, P, P, P] + [CONST[dt]] * 8
    for a, b in (("bool", "f32"), ("bool", "bf16"), ("f32", "bf16"), ("bf16", "f32"), ("f32", "bool"), ("bf16", "bool"),
                 ("bool", "f16"), ("f32", "f16"), ("f16", "f32"), ("f16", "bool")):
        sig[f"cast_{a}_{b}"] = [SZ, P, P]
    sig["sum_f32_noalloc"] = [SZ, SZ, SZ, P, P, P]
    sig["mse_loss_f32"] = [SZ, P, P, P]
    sig["mse_loss_backward_f32"] = [SZ, P, P, P, P, P]
    sig["sgd_step_f32"] = [SZ, P, P, C.c_float]
    sig["conv2d_cols_matmul_f32"] = [P, C.c_int, P, P, SZ, P, P]
    sig["conv2d_col2im_add_f32"] = [SZ, P, P, P]
    sig.update(cast_signatures())
    sig.update(wide_util_signatures())
    sig.update(wide_unary_signatures())
    sig.update(wide_reduce_signatures())
    return sig
