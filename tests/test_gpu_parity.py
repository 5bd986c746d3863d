"""GPU parity: the HIP backend, called through its C ABI, against the CPU oracle on the same seeded
inputs.  Bars: bit-exact for data movement, comparisons and single IEEE operations; <= 1 ulp for
f32 transcendentals (tanh-based ones are reported, see test); reductions and matmuls against an
f64 evaluation of the same inputs, f32 <= 1e-5 and bf16 <= 1e-2 of the sum of magnitudes."""
import numpy as np
import pytest

import layouts as LY
from helpers import (NP, PLAIN, cast_inputs, In, InOut, Out, bf16_to_f32, const_arg, contiguous_strides, f32_to_bf16, meta_binary, meta_conv,
                     layout, meta_matmul, meta_pad, u64, meta_reduce, meta_sum_to_shape, meta_unary, rng, to_float, to_storage,
                     ulp_diff_f32)

pytestmark = pytest.mark.gpu

DTS = ["f32", "bf16", "f16"]
INT_DTS = ["u8", "u16", "u32", "u64", "i8", "i16", "i32", "i64"]


def both(oracle, hip, name, *args_builder):
    """Run the same call on both backends; args_builder() must build fresh argument objects."""
    (build,) = args_builder
    return oracle.call(name, *build()), hip.call(name, *build())


def same_bits(a, b):
    return np.array_equal(np.ascontiguousarray(a).view(np.uint8), np.ascontiguousarray(b).view(np.uint8))


# ---------------------------------------------------------------------------------------------------
# elementwise
# ---------------------------------------------------------------------------------------------------
BIN_LAYOUTS = {
    "contig": lambda: (LY.contiguous([37, 64]), LY.contiguous([37, 64])),
    "contig_big": lambda: (LY.contiguous([1 << 18]), LY.contiguous([1 << 18])),
    "offset_misaligned": lambda: (LY.contiguous([33, 20], off=1), LY.contiguous([33, 20], off=3)),
    "rhs_row_bcast": lambda: (LY.contiguous([96, 256]), LY.broadcast([96, 256], [1, 256])),
    "rhs_row_bcast_odd": lambda: (LY.contiguous([17, 30], off=1), LY.broadcast([17, 30], [1, 30])),
    "lhs_col_bcast": lambda: (LY.broadcast([64, 48], [64, 1]), LY.contiguous([64, 48])),
    "lhs_transposed": lambda: (LY.permuted([192, 160], [1, 0]), LY.contiguous([192, 160])),
    "lhs_transposed_supertiles": lambda: (LY.permuted([1024, 1024], [1, 0]), LY.contiguous([1024, 1024])),
    "lhs_transposed_ragged": lambda: (LY.permuted([70, 45], [1, 0], off=1), LY.contiguous([70, 45])),
    "both_transposed": lambda: (LY.permuted([100, 130], [1, 0]), LY.permuted([100, 130], [1, 0], off=2)),
    "nhwc_view_plus_bias": lambda: (LY.permuted([2, 64, 12, 12], [0, 3, 1, 2]), LY.broadcast([2, 64, 12, 12], [1, 64, 1, 1])),
    "scalar_bcast": lambda: (LY.contiguous([1000]), LY.broadcast([1000], [1])),
    "batched_transpose3d": lambda: (LY.permuted([3, 40, 50], [0, 2, 1]), LY.contiguous([3, 40, 50])),
    "rank5": lambda: (LY.permuted([2, 3, 4, 5, 6], [4, 2, 0, 3, 1]), LY.broadcast([2, 3, 4, 5, 6], [2, 1, 4, 1, 6])),
    "one_element": lambda: (LY.contiguous([1]), LY.contiguous([1])),
}


def special_values(r, n, dt):
    x = r.standard_normal(n).astype(np.float32)
    k = min(n, 8)
    x[:k] = np.array([0.0, -0.0, np.inf, -np.inf, np.nan, 1.0, -1.0, 3e38], dtype=np.float32)[:k]
    return to_storage(x, dt)


@pytest.mark.parametrize("dt", DTS)
@pytest.mark.parametrize("lname", list(BIN_LAYOUTS))
def test_binary_ops_bit_exact(oracle, hip, lname, dt):
    ll, rl = BIN_LAYOUTS[lname]()
    r = rng(hash(lname) % 1000)
    ls, rs = special_values(r, ll["size"], dt), special_values(r, rl["size"], dt)
    # make zeros meet zeros / non-zeros for the division rule
    n = int(np.prod(ll["dims"]))
    md = meta_binary(ll["dims"], ll["strides"], rl["strides"], ll["off"], rl["off"])
    for op in ["add", "sub", "mul", "div", "maximum", "minimum"]:
        (o,), (h,) = both(oracle, hip, f"{op}_{dt}", lambda: (n, len(ll["dims"]), md, In(ls), In(rs), Out(n, dt)))
        if op in ("maximum", "minimum") and dt == "f32":
            # f32::max may return either zero for (+0, -0): compare values, NaN-aware
            assert np.array_equal(o, h, equal_nan=True), op
        else:
            fo, fh = to_float(o, dt), to_float(h, dt)
            assert np.array_equal(np.isnan(fo), np.isnan(fh)), op
            assert same_bits(np.where(np.isnan(fo), 0, fo), np.where(np.isnan(fh), 0, fh)), op
    for op in ["eq", "ne", "lt", "le", "gt", "ge", "logical_and", "logical_or", "logical_xor"]:
        (o,), (h,) = both(oracle, hip, f"{op}_{dt}", lambda: (n, len(ll["dims"]), md, In(ls), In(rs), Out(n, "bool")))
        assert np.array_equal(o, h), op


@pytest.mark.parametrize("dt", DTS)
@pytest.mark.parametrize("lname", ["contig", "offset_misaligned", "rhs_row_bcast", "scalar_bcast", "nhwc_view_plus_bias"])
def test_inplace_ops_bit_exact(oracle, hip, lname, dt):
    ll, rl = BIN_LAYOUTS[lname]()
    lc = LY.contiguous(ll["dims"], off=ll["off"])       # accumulators are contiguous tensors
    r = rng(5)
    ls = to_storage(r.standard_normal(lc["size"]).astype(np.float32), dt)
    rs = to_storage(r.standard_normal(rl["size"]).astype(np.float32), dt)
    n = int(np.prod(lc["dims"]))
    md = meta_binary(lc["dims"], lc["strides"], rl["strides"], lc["off"], rl["off"])
    for op in ["add_inplace", "sub_inplace", "mul_inplace", "div_inplace"]:
        (o,), (h,) = both(oracle, hip, f"{op}_{dt}", lambda: (n, len(lc["dims"]), md, InOut(ls.copy()), In(rs)))
        assert same_bits(o, h), op


def test_inplace_with_transposed_rhs(oracle, hip):
    # accumulate_grad of a transposed operand: lhs contiguous, rhs a transposed view
    lc, rl = LY.contiguous([130, 70]), LY.permuted([130, 70], [1, 0])
    r = rng(6)
    ls = r.standard_normal(lc["size"]).astype(np.float32)
    rs = r.standard_normal(rl["size"]).astype(np.float32)
    md = meta_binary(lc["dims"], lc["strides"], rl["strides"], 0, 0)
    (o,), (h,) = both(oracle, hip, "add_inplace_f32", lambda: (130 * 70, 2, md, InOut(ls.copy()), In(rs)))
    assert same_bits(o, h)


UN_LAYOUTS = {
    "contig": lambda: LY.contiguous([5000]),
    "offset": lambda: LY.contiguous([77, 13], off=1),
    "transposed": lambda: LY.permuted([150, 200], [1, 0]),
    "transposed_whole_tiles": lambda: LY.permuted([160, 256], [1, 0]),      # the vector form of the tile kernel, also for bool outputs
    "bcast": lambda: LY.broadcast([40, 50], [1, 50]),
    "perm4d": lambda: LY.permuted([2, 5, 6, 7], [3, 1, 0, 2]),
}
EXACT_UNARY = ["neg", "abs", "sign", "square", "sqrt", "relu", "recip"]
ULP1_UNARY = ["exp", "sigmoid", "sin", "cos", "ln", "log2", "exp2", "softplus", "exp10", "log10", "tan"]


@pytest.mark.parametrize("dt", DTS)
@pytest.mark.parametrize("lname", list(UN_LAYOUTS))
def test_unary_exact_ops(oracle, hip, lname, dt):
    lay = UN_LAYOUTS[lname]()
    r = rng(3)
    st = special_values(r, lay["size"], dt)
    n = int(np.prod(lay["dims"]))
    md = meta_unary(lay["dims"], lay["strides"], lay["off"])
    for op in EXACT_UNARY:
        (o,), (h,) = both(oracle, hip, f"{op}_{dt}", lambda: (n, len(lay["dims"]), md, In(st), Out(n, dt)))
        fo, fh = to_float(o, dt), to_float(h, dt)
        assert np.array_equal(np.isnan(fo), np.isnan(fh)), op
        assert same_bits(np.where(np.isnan(fo), 0, fo), np.where(np.isnan(fh), 0, fh)), op
    (o,), (h,) = both(oracle, hip, f"logical_not_{dt}", lambda: (n, len(lay["dims"]), md, In(st), Out(n, "bool")))
    assert np.array_equal(o, h)
    for op, c in [("add_scalar", 0.75), ("sub_scalar", 0.3), ("mul_scalar", 0.01), ("div_scalar", 3.0), ("div_scalar", 0.0),
                  ("maximum_scalar", 0.1), ("minimum_scalar", -0.2), ("leaky_relu", 0.1)]:
        (o,), (h,) = both(oracle, hip, f"{op}_{dt}", lambda: (n, len(lay["dims"]), md, In(st), const_arg(c, dt), Out(n, dt)))
        fo, fh = to_float(o, dt), to_float(h, dt)
        assert np.array_equal(np.isnan(fo), np.isnan(fh)), op
        assert np.array_equal(np.where(np.isnan(fo), 0, fo), np.where(np.isnan(fh), 0, fh)), (op, c)
    for op in ["eq_scalar", "ne_scalar", "lt_scalar", "le_scalar", "gt_scalar", "ge_scalar"]:
        (o,), (h,) = both(oracle, hip, f"{op}_{dt}", lambda: (n, len(lay["dims"]), md, In(st), const_arg(0.0, dt), Out(n, "bool")))
        assert np.array_equal(o, h), op


def test_unary_in_place_when_input_is_null(hip, oracle):
    r = rng(8)
    x = r.standard_normal(1000).astype(np.float32)
    (want,) = oracle.call("square_f32", 1000, 1, meta_unary([1000], [1]), In(x), Out(1000, "f32"))
    (got,) = hip.call("square_f32", 1000, 1, meta_unary([1000], [1]), None, InOut(x.copy()))
    assert same_bits(want, got)


# exp and tanh restate libm's own algorithms, so they and everything built from them with plain
# IEEE operations must come out with identical bits; the rest is evaluated in f64 and rounded once.
BIT_EXACT_TRANSCENDENTAL = ["exp", "tanh", "gelu", "sigmoid"]


@pytest.mark.parametrize("op", ULP1_UNARY + ["tanh", "gelu"])
def test_unary_transcendental_f32_ulp(oracle, hip, op):
    r = rng(17)
    n = 1 << 16
    x = np.concatenate([r.standard_normal(n // 2) * 1.0, r.uniform(-20, 20, n // 4), r.uniform(-90, 90, n // 4)]).astype(np.float32)
    if op in ("ln", "log2", "log10"):
        x = np.abs(x) + 1e-3
    md = meta_unary([n], [1])
    (o,), (h,) = both(oracle, hip, f"{op}_f32", lambda: (n, 1, md, In(x), Out(n, "f32")))
    d = ulp_diff_f32(o, h)
    if op in BIT_EXACT_TRANSCENDENTAL:
        assert np.max(d) == 0, (op, int(np.max(d)), x[np.argmax(d)])
    elif op in ("tan", "log10"):
        # glibc's tanf / log10f are not correctly rounded (documented up to 2 ulp)
        assert np.max(d) <= 2, (op, int(np.max(d)))
    else:
        assert np.max(d) <= 1, (op, int(np.max(d)), x[np.argmax(d)])


def test_elu_f32_bit_exact(oracle, hip):
    r = rng(18)
    n = 1 << 15
    x = (r.standard_normal(n) * 4).astype(np.float32)
    md = meta_unary([n], [1])
    (o,), (h,) = both(oracle, hip, "elu_f32", lambda: (n, 1, md, In(x), const_arg(1.3, "f32"), Out(n, "f32")))
    assert same_bits(o, h)


def test_exp_tanh_f32_subnormal_and_edge_inputs(oracle, hip):
    x = np.array([0.0, -0.0, np.inf, -np.inf, np.nan, 88.7, 88.8, -87.5, -100.0, -103.5, -104.5, 1e-40, -1e-40, 1e-30, 21.9, 22.1,
                  -22.1, 0.5, 1.0, -1.0, 3e-9, 0.3465, 1.04, -0.3466], dtype=np.float32)
    md = meta_unary([x.size], [1])
    for op in ("exp", "tanh", "gelu", "sigmoid", "softplus"):
        (o,), (h,) = both(oracle, hip, f"{op}_f32", lambda: (x.size, 1, md, In(x), Out(x.size, "f32")))
        lim = 0 if op != "softplus" else 1
        assert np.max(ulp_diff_f32(o, h)) <= lim, (op, o, h)
        assert np.array_equal(np.signbit(o), np.signbit(h)), op


def test_pow_f32_ulp(oracle, hip):
    r = rng(19)
    n = 1 << 15
    x = r.standard_normal(n).astype(np.float32)
    md = meta_unary([n], [1])
    for c in (2.0, 1.0, 3.0, 0.5, -1.0):
        (o,), (h,) = both(oracle, hip, "pow_f32", lambda: (n, 1, md, In(x), const_arg(c, "f32"), Out(n, "f32")))
        assert np.max(ulp_diff_f32(o, h)) <= 1, c


def test_pow_square_is_the_correctly_rounded_product(oracle, hip):
    """pow(x, 2) takes the product path: the correctly rounded square (what a double pow rounded once gives),
    special values included; the oracle's powf may differ from it by one ulp at most."""
    r = rng(23)
    x = np.concatenate([r.standard_normal(4096).astype(np.float32) * np.float32(10.0) ** r.integers(-25, 20, 4096).astype(np.float32),
                        np.array([0.0, -0.0, np.inf, -np.inf, np.nan, 1e-30, -1e-30, 1e-23, 3e19, -3e19, 1.8446744e19, 1e-45], np.float32)])
    n = x.size
    md = meta_unary([n], [1])
    (o,), (h,) = both(oracle, hip, "pow_f32", lambda: (n, 1, md, In(x), const_arg(2.0, "f32"), Out(n, "f32")))
    with np.errstate(all="ignore"):
        want = x * x
    assert np.array_equal(np.isnan(want), np.isnan(h))
    ok = ~np.isnan(want)
    assert np.array_equal(want[ok].view(np.uint32), h[ok].view(np.uint32))
    fin = ok & np.isfinite(o)
    assert np.max(ulp_diff_f32(o[fin], h[fin])) <= 1
    (h1,) = hip.call("pow_f32", n, 1, md, In(x), const_arg(1.0, "f32"), Out(n, "f32"))          # x^1 is x
    assert np.array_equal(x[ok].view(np.uint32), h1[ok].view(np.uint32)) and np.array_equal(np.isnan(x), np.isnan(h1))
    for dt in ("bf16", "f16"):
        bits = np.arange(1 << 16, dtype=np.uint16)
        mdb = meta_unary([bits.size], [1])
        for c in (2.0, 1.0):
            (ob,), (hb,) = both(oracle, hip, f"pow_{dt}", lambda: (bits.size, 1, mdb, In(bits), const_arg(c, dt), Out(bits.size, dt)))
            fo = to_float(ob, dt)
            okb = ~np.isnan(fo)
            assert np.array_equal(ob[okb], hb[okb]), (dt, c)


@pytest.mark.parametrize("dt", ["bf16", "f16"])
@pytest.mark.parametrize("op", ["exp", "tanh", "gelu", "sigmoid"])
def test_unary_transcendental_16bit(oracle, hip, op, dt):
    # all 2^16 inputs: f32 evaluation (bit-identical) then the same single rounding
    bits = np.arange(1 << 16, dtype=np.uint16)
    md = meta_unary([bits.size], [1])
    (o,), (h,) = both(oracle, hip, f"{op}_{dt}", lambda: (bits.size, 1, md, In(bits), Out(bits.size, dt)))
    fo, fh = to_float(o, dt), to_float(h, dt)
    assert np.array_equal(np.isnan(fo), np.isnan(fh))
    ok = ~np.isnan(fo)
    assert np.array_equal(o[ok], h[ok])


@pytest.mark.parametrize("dt", INT_DTS)
def test_integer_pow_bit_exact(oracle, hip, dt):
    """`(x as f64).powf(c as f64) as T` (unary.rs:565-572): the GPU's exact-integer evaluation against the oracle's libm
    pow and cast - every (x, c) pair of the 8-bit types, boundary sets for the wider ones (the roots of the type's bounds,
    powers of two, 2^53 and its neighbours, negative and huge exponents)."""
    from test_oracle_properties import int_pow_cases
    info = np.iinfo(NP[dt])
    if info.bits == 8:
        xs = np.arange(info.min, info.max + 1).astype(NP[dt])
        cs = range(info.min, info.max + 1)
    else:
        xs, cs = int_pow_cases(dt, rng(97))
    # one call per exponent on a 2-d strided view, so that the strided kernel is exercised as well
    md = meta_unary([xs.size], [1])
    for c in cs:
        (o,), (h,) = both(oracle, hip, f"pow_{dt}", lambda: (xs.size, 1, md, In(xs), int(c), Out(xs.size, dt)))
        assert np.array_equal(o, h), (dt, c, xs[np.nonzero(o != h)[0][:5]], o[o != h][:5], h[o != h][:5])


@pytest.mark.parametrize("op", ["tanh", "gelu"])
def test_tanh_and_gelu_f32_bit_exact_on_16m_inputs(oracle, hip, op):
    """The branch-free tanhf restatement (its two divisions use the reciprocal instruction and fused corrections) against the
    oracle's libm on 2^24 inputs: every exponent from 2^-60 to 2^6 in both signs, dense around the switch points of the
    algorithm (|x| = 0.5 ln 2 / 2, 1.5 ln 2 / 2, 1, 9, 19.6, 22), zeros, infinities, NaN."""
    r = rng(31)
    n = 1 << 24
    x = (r.standard_normal(n) * np.exp2(r.integers(-60, 7, n))).astype(np.float32)
    k = n // 16
    for i, centre in enumerate((0.17328679, 0.51986039, 1.0, 9.0, 19.6, 22.0)):
        x[i * k:(i + 1) * k] = (centre * (1.0 + r.uniform(-2e-3, 2e-3, k))).astype(np.float32) * r.choice(np.array([-1.0, 1.0], np.float32), k)
    x[-8:] = np.array([0.0, -0.0, np.inf, -np.inf, np.nan, 1e-39, -1e-39, 88.0], np.float32)
    oracle.set_threads(0)
    try:
        (o,) = oracle.call(f"{op}_f32", n, 1, meta_unary([n], [1]), In(x), Out(n, "f32"))
    finally:
        oracle.set_threads(1)
    (h,) = hip.call(f"{op}_f32", n, 1, meta_unary([n], [1]), In(x), Out(n, "f32"))
    assert np.array_equal(np.isnan(o), np.isnan(h))
    ok = ~np.isnan(o)
    bad = np.nonzero(o[ok].view(np.uint32) != h[ok].view(np.uint32))[0]
    assert bad.size == 0, (bad.size, x[ok][bad[:5]], o[ok][bad[:5]], h[ok][bad[:5]])


@pytest.mark.parametrize("dt,shape,perm", [("f32", [2056, 2120], [1, 0]), ("f32", [5, 1032, 1024], [0, 2, 1]), ("f32", [3, 1032, 1024], [2, 1, 0]),
                                           ("bf16", [4104, 2120], [1, 0]), ("f16", [3, 2056, 2048], [0, 2, 1])])
def test_unary_on_transposed_views_of_a_thousand_tiles_and_more(oracle, hip, dt, shape, perm):
    """Transposed views of a thousand tiles and more: ragged edge tiles, an outer dim, the 8x8 tile order - bit for bit
    the oracle (exp on the 16-bit dtypes is the table functor's standing grid, the others one block a tile)."""
    r = rng(173)
    n = int(np.prod(shape))
    x = to_storage(r.standard_normal(n).astype(np.float32) * 2, dt)
    base = [shape[perm.index(d)] for d in range(len(shape))]            # the buffer's own shape
    bs = contiguous_strides(base)
    md = meta_unary(shape, [bs[p] for p in perm], 0)
    for op in ("neg", "relu", "exp"):
        (o,), (h,) = both(oracle, hip, f"{op}_{dt}", lambda: (n, len(shape), md, In(x), Out(n, dt)))
        assert same_bits(o, h), op


@pytest.mark.parametrize("dt", ["f32", "bf16", "f16"])
@pytest.mark.parametrize("shape", [[264, 328], [3, 136, 200]])
def test_binary_of_one_transposed_view_given_twice(oracle, hip, dt, shape):
    """x * x, x + x, x - y with x one and the same transposed view (same pointer, same strides): the tile of x is staged
    once and read for both operands; a second view of ANOTHER buffer with the same strides must not be taken for it."""
    r = rng(179)
    n = int(np.prod(shape))
    x, y = In(to_storage(r.standard_normal(n).astype(np.float32), dt)), In(to_storage(r.standard_normal(n).astype(np.float32), dt))
    base = shape[:-2] + [shape[-1], shape[-2]]
    st = contiguous_strides(base)
    st = st[:-2] + [st[-1], st[-2]]
    md = meta_binary(shape, st, st)
    for op in ("mul", "add", "sub"):
        for a, b in ((x, x), (x, y)):
            (o,), (h,) = both(oracle, hip, f"{op}_{dt}", lambda: (n, len(shape), md, a, b, Out(n, dt)))
            assert same_bits(o, h), (op, a is b)


TABLE_OPS = ["sigmoid", "tanh", "gelu", "sin", "cos", "tan", "ln", "log10", "log2", "exp", "exp10", "exp2", "softplus"]


@pytest.mark.parametrize("dt", ["bf16", "f16"])
@pytest.mark.parametrize("op", TABLE_OPS)
def test_large_16bit_unary_calls_go_through_the_table_and_keep_the_bits(oracle, hip, op, dt):
    """A call of 2^20 elements or more on a 16-bit dtype is a table lookup (the table is the op's own kernel run over all
    65536 codes).  Every code, in a shuffled 1.1 M-element input with a ragged tail, must give the bits of the small call
    that computes - contiguous, in place, at an element offset that breaks the 16-byte alignment, and through a
    transposed view - and for the functions the oracle restates bit for bit, the oracle's bits."""
    codes = np.arange(1 << 16, dtype=np.uint16)
    (small,) = hip.call(f"{op}_{dt}", codes.size, 1, meta_unary([codes.size], [1]), In(codes), Out(codes.size, dt))
    n = (1 << 20) + (1 << 16) + 5
    x = np.tile(codes, 18)[:n].copy()
    rng(29).shuffle(x)
    want = small[x]
    (h,) = hip.call(f"{op}_{dt}", n, 1, meta_unary([n], [1]), In(x), Out(n, dt))
    assert np.array_equal(h, want)
    (hi,) = hip.call(f"{op}_{dt}", n, 1, meta_unary([n], [1]), None, InOut(x.copy()))            # null input: in place
    assert np.array_equal(hi, want)
    (ho,) = hip.call(f"{op}_{dt}", n - 3, 1, meta_unary([n - 3], [1], 3), In(x), Out(n - 3, dt))    # odd offset: misaligned
    assert np.array_equal(ho, want[3:])
    rows, cols = 1040, 1024                                                                       # [1040,1024] view of a [1024,1040] buffer
    (ht,) = hip.call(f"{op}_{dt}", rows * cols, 2, meta_unary([rows, cols], [1, rows]), In(x[: rows * cols]), Out(rows * cols, dt))
    assert np.array_equal(ht.reshape(rows, cols), want[: rows * cols].reshape(cols, rows).T)
    # [2,1024,512] view of a [2,512,1024] buffer: an outer dim, and tile counts that take the 8x8 block order
    xb = np.tile(x, 1)[: 2 * 512 * 1024]
    (hb,) = hip.call(f"{op}_{dt}", xb.size, 3, meta_unary([2, 1024, 512], [512 * 1024, 1, 1024]), In(xb), Out(xb.size, dt))
    assert np.array_equal(hb.reshape(2, 1024, 512), want[: xb.size].reshape(2, 512, 1024).transpose(0, 2, 1))
    if op in ("exp", "tanh", "gelu", "sigmoid"):
        (o,) = oracle.call(f"{op}_{dt}", n, 1, meta_unary([n], [1]), In(x), Out(n, dt))
        ok = ~np.isnan(to_float(o, dt))
        assert np.array_equal(np.isnan(to_float(o, dt)), np.isnan(to_float(h, dt)))
        assert np.array_equal(o[ok], h[ok])


# ---------------------------------------------------------------------------------------------------
# reductions
# ---------------------------------------------------------------------------------------------------
RED_CASES = [([64, 96], 0), ([64, 96], 1), ([257, 130], 0), ([257, 130], 1), ([8, 16, 32], 0), ([8, 16, 32], 1), ([8, 16, 32], 2),
             ([5000], 0), ([3, 70000], 1), ([70000, 3], 0), ([1, 40000], 0), ([10000, 1], 1), ([2, 3, 5, 7], 2), ([40000], 0),
             ([300, 2048], 1), ([4, 300000], 1),
             # at least 65536 rows of a few dozen elements: 16 lanes per row (rows of 56, 40, 256 and 64 elements)
             ([1200, 56, 56], 2), ([70000, 40], 1), ([66000, 256], 1), ([65536, 64], 1),
             # narrow rows under a long axis: 256 rows at a time as one wide row, the partial rows folded by a second call
             # (left-over rows, an outer dim whose slices must stay whole, an axis too ragged to regroup)
             ([300000, 5], 0), ([40001, 7], 0), ([2, 16384, 3], 1), ([3, 8200, 6], 1), ([1, 9000, 33], 1), ([5, 8192, 1], 1)]


@pytest.mark.parametrize("dt", DTS)
@pytest.mark.parametrize("shape,dim", RED_CASES)
def test_reductions(oracle, hip, shape, dim, dt):
    r = rng(23)
    n = int(np.prod(shape))
    x = r.uniform(-1, 1, n).astype(np.float32)
    off = 1 if n % 2 else 0
    st = to_storage(np.concatenate([np.full(off, 5.0, np.float32), x]), dt)
    xs = to_float(st, dt)[off:].reshape(shape).astype(np.float64)
    md = meta_reduce(shape, contiguous_strides(shape), dim, off)
    tol = 1e-5 if dt == "f32" else 1e-2
    for op in ["sum", "mean", "max", "min"]:
        (o,), (h,) = both(oracle, hip, f"{op}_{dt}", lambda: (n, len(shape), 1, md, In(st), Out(n // shape[dim], dt)))
        fh = to_float(h, dt).astype(np.float64)
        if op == "mean" and dt == "f16" and shape[dim] > 65504:
            # the count itself overflows f16 (reduction.rs:584: f16::from_f32(x as f32) = inf), so the reference's mean is sum / inf = 0
            assert np.array_equal(to_float(o, dt), to_float(h, dt)) and np.all(fh == 0), op
            continue
        if op in ("max", "min"):
            assert np.array_equal(to_float(o, dt), to_float(h, dt)), op
            continue
        truth = xs.sum(dim) if op == "sum" else xs.mean(dim)
        scale = np.abs(xs).sum(dim) if op == "sum" else np.abs(xs).mean(dim)
        err = np.abs(fh - truth.ravel()) / np.maximum(scale.ravel(), 1e-30)
        assert np.max(err) <= tol, (op, float(np.max(err)))
        if dt == "f32":   # the oracle (sequential f32) obeys the same bound, so the two agree to twice it
            assert np.max(np.abs(fh - o.astype(np.float64)) / np.maximum(scale.ravel(), 1e-30)) <= 2 * tol


def test_reduction_is_deterministic(hip):
    r = rng(29)
    x = r.uniform(-1, 1, 512 * 4096).astype(np.float32)
    md = meta_reduce([512, 4096], [4096, 1], 0)
    outs = [hip.call("sum_f32", x.size, 2, 1, md, In(x), Out(4096, "f32"))[0].copy() for _ in range(3)]
    assert same_bits(outs[0], outs[1]) and same_bits(outs[0], outs[2])


def test_max_seed_and_nan_rule(oracle, hip):
    for data in ([-np.inf, np.nan, -np.inf, np.nan], [np.nan, 2.0, np.nan, -1.0]):
        x = np.array(data, dtype=np.float32)
        (o,), (h,) = both(oracle, hip, "max_f32", lambda: (4, 1, 1, meta_reduce([4], [1], 0), In(x), Out(1, "f32")))
        assert same_bits(o, h)


def test_reduce_strided_input_follows_reference_quirk(oracle, hip):
    # non-contiguous input: the metadata carries the memory stride of the reduced dim as the logical
    # one (tensor/ops/reduction.rs:728-729); the backend must reproduce what the CPU kernel does then
    lay = LY.permuted([6, 8], [1, 0])
    r = rng(31)
    st = r.uniform(-1, 1, lay["size"]).astype(np.float32)
    for dim in (0, 1):
        md = meta_reduce(lay["dims"], lay["strides"], dim, 0)
        (o,), (h,) = both(oracle, hip, "sum_f32", lambda: (48, 2, 1, md, In(st), Out(48 // lay["dims"][dim], "f32")))
        assert np.allclose(o, h, atol=1e-6)


@pytest.mark.parametrize("dt", ["f32", "bf16"])
@pytest.mark.parametrize("dims,perm", [([520, 640], [1, 0]), ([40, 72, 128], [2, 0, 1]), ([6, 300, 200], [0, 2, 1])])
def test_reduce_large_strided_input_is_the_reduction_of_its_logical_copy(oracle, hip, dims, perm, dt):
    """From 2^18 elements a strided input is copied into logical order and reduced as a contiguous tensor: the same
    elements per output as the reference's walk (max and min are order-independent: bit for bit), sums to rounding."""
    lay = LY.permuted(dims, perm)
    r = rng(181)
    st = to_storage(r.uniform(-1, 1, lay["size"]).astype(np.float32), dt)
    n = int(np.prod(lay["dims"]))
    assert n >= 1 << 18
    for dim in range(len(dims)):
        md = meta_reduce(lay["dims"], lay["strides"], dim, 0)
        out_n = n // lay["dims"][dim]
        for op in ("max", "min"):
            (o,), (h,) = both(oracle, hip, f"{op}_{dt}", lambda: (n, len(dims), 1, md, In(st), Out(out_n, dt)))
            assert same_bits(o, h), (op, dim)
        for op in ("sum", "mean"):
            (o,), (h,) = both(oracle, hip, f"{op}_{dt}", lambda: (n, len(dims), 1, md, In(st), Out(out_n, dt)))
            if dt == "f32":
                assert np.allclose(o, h, rtol=1e-5, atol=2e-4), (op, dim)
            else:
                # the reference's bf16 running sum against an f32 sum rounded once: loose, the index sets are pinned by max / min
                assert np.allclose(to_float(o, dt), to_float(h, dt), rtol=0.1, atol=1.0), (op, dim)


STS_CASES = [([64, 96], [64, 96]), ([64, 96], [1, 96]), ([64, 96], [64, 1]), ([8, 64, 128], [1, 64, 1]), ([8, 64, 128], [8, 1, 128]),
             ([2, 3, 4, 5], [1, 3, 1, 5]), ([2, 3, 4, 5], [2, 1, 4, 1]), ([10000, 1], [10000, 1]), ([10000, 1], [1, 1]), ([5], [1]),
             ([300, 700], [1, 1]), ([2, 3, 4, 5, 6], [1, 3, 1, 5, 1]),
             # [reduced, kept, reduced] in one pass: rows cut into chunks (few kept), one block per kept index (many)
             ([40, 3, 256], [1, 3, 1]), ([64, 300, 128], [1, 300, 1]), ([33, 7, 520], [1, 7, 1]), ([2, 4, 260, 2, 64], [1, 1, 260, 1, 1])]


@pytest.mark.parametrize("dt", DTS)
@pytest.mark.parametrize("shape,out_shape", STS_CASES)
def test_sum_to_shape(oracle, hip, shape, out_shape, dt):
    r = rng(37)
    n = int(np.prod(shape))
    st = to_storage(r.uniform(-1, 1, n).astype(np.float32), dt)
    md = meta_sum_to_shape(shape, contiguous_strides(shape), out_shape, 0)
    n_out = int(np.prod(out_shape))
    (o,), (h,) = both(oracle, hip, f"sum_to_shape_{dt}", lambda: (n, len(shape), md, In(st), Out(n_out, dt)))
    xs = to_float(st, dt).reshape(shape).astype(np.float64)
    axes = tuple(i for i, (a, b) in enumerate(zip(shape, out_shape)) if a != b)
    if not axes:
        assert same_bits(o, h)      # identity: 0 + x
        return
    truth = xs.sum(axis=axes).ravel()
    scale = np.abs(xs).sum(axis=axes).ravel()
    tol = 1e-5 if dt == "f32" else 1e-2
    assert np.max(np.abs(to_float(h, dt) - truth) / np.maximum(scale, 1e-30)) <= tol


def test_sum_to_shape_identity_negative_zero(oracle, hip):
    x = np.array([-0.0, 1.0, -2.0, -0.0], dtype=np.float32)
    (o,), (h,) = both(oracle, hip, "sum_to_shape_f32", lambda: (4, 1, meta_sum_to_shape([4], [1], [4]), In(x), Out(4, "f32")))
    assert same_bits(o, h)


def test_sum_to_shape_strided_input(oracle, hip):
    # a stride-0 (broadcast) gradient view, offset 0 — the shape sum(0)'s backward hands over
    lay = LY.broadcast([50, 30], [1, 30])
    r = rng(41)
    st = r.uniform(-1, 1, lay["size"]).astype(np.float32)
    st = np.concatenate([st, np.zeros(50 * 30 - st.size, np.float32)])     # keep the reference's modulo index in bounds
    for out_shape in ([1, 30], [50, 30], [50, 1]):
        md = meta_sum_to_shape(lay["dims"], lay["strides"], out_shape, 0)
        n_out = int(np.prod(out_shape))
        (o,), (h,) = both(oracle, hip, "sum_to_shape_f32", lambda: (1500, 2, md, In(st), Out(n_out, "f32")))
        assert np.allclose(o, h, rtol=1e-5, atol=1e-5), out_shape


@pytest.mark.parametrize("dt", ["f32", "bf16"])
def test_sum_to_shape_of_permuted_views_with_a_reduction(oracle, hip, dt):
    """Permuted views (every index below num_els, so the reference's modulo never applies) are copied into logical order
    by the elementwise identity and reduced; a view whose indices pass num_els keeps the gather with the modulo."""
    r = rng(199)
    cases = [(LY.permuted([72, 200], [1, 0]), [[1, 200], [72, 1], [1, 1]]), (LY.permuted([6, 40, 56], [2, 0, 1]), [[1, 40, 1], [6, 1, 56], [1, 1, 56]]),
             (dict(dims=[30, 40], strides=[1, 32], off=0, size=30 * 40 + 64), [[1, 40], [30, 1]])]
    for lay, outs in cases:
        n = int(np.prod(lay["dims"]))
        st = to_storage(r.uniform(-1, 1, max(lay["size"], n)).astype(np.float32), dt)
        for out_shape in outs:
            md = meta_sum_to_shape(lay["dims"], lay["strides"], out_shape, 0)
            n_out = int(np.prod(out_shape))
            (o,), (h,) = both(oracle, hip, f"sum_to_shape_{dt}", lambda: (n, len(lay["dims"]), md, In(st), Out(n_out, dt)))
            a, b = to_float(o, dt).astype(np.float64), to_float(h, dt).astype(np.float64)
            if dt == "f32":
                assert np.allclose(a, b, rtol=1e-5, atol=1e-5), (lay["dims"], out_shape)
            elif lay["size"] <= n:
                # bf16: the reference's running sum in bf16 drifts by several units; the kernel's f32 sum rounded once is
                # held to the exact sum of the same elements
                logical = to_float(LY.gather(st, lay), dt).astype(np.float64)
                axes = tuple(d for d, (i, k) in enumerate(zip(lay["dims"], out_shape)) if k == 1 and i != 1)
                exact = logical.sum(axis=axes).ravel()
                assert np.all(np.abs(b - exact) <= 2.0 ** -8 * np.abs(exact) + 1e-3), (lay["dims"], out_shape)


@pytest.mark.parametrize("dt", DTS)
def test_sum_to_shape_identity_on_strided_views(oracle, hip, dt):
    """out = 0 + view for views that stay below num_els (one elementwise pass over the view's strides) and for one whose
    indices pass num_els, where the reference's modulo applies (reduction.rs:162-167): the same bits as the oracle."""
    r = rng(83)
    cases = [([40, 30], [0, 1], 0, 40 * 30), ([40, 30], [1, 0], 0, 40 * 30), ([6, 40, 30], [0, 30, 1], 0, 6 * 40 * 30),
             ([30, 40], [1, 30], 0, 30 * 40),                      # a transposed view: its last index is num_els - 1
             ([30, 40], [1, 32], 0, 30 * 40 + 64),                 # rows 32 apart: indices reach 1277 >= 1200, wrapped
             ([8192, 512], [0, 1], 0, 8192 * 512)]                 # a broadcast row as large as a gradient
    for dims, strides, off, size in cases:
        n = int(np.prod(dims))
        st = to_storage(r.standard_normal(size).astype(np.float32), dt)
        st[::7] = to_storage(np.array([-0.0], np.float32), dt)[0]
        md = meta_sum_to_shape(dims, strides, dims, off)
        (o,), (h,) = both(oracle, hip, f"sum_to_shape_{dt}", lambda: (n, len(dims), md, In(st), Out(n, dt)))
        assert same_bits(o, h), (dims, strides)


# ---------------------------------------------------------------------------------------------------
# matmul
# ---------------------------------------------------------------------------------------------------
def matmul_inputs(r, batch, m, k, n, a_perm, b_perm, dt, b_bcast=False):
    a = r.standard_normal((batch, m, k)).astype(np.float32)
    b = (r.standard_normal((1 if b_bcast else batch, k, n)) * 0.02).astype(np.float32)
    a_shape, b_shape = [batch, m, k], [batch, k, n]
    a_st, b_st = contiguous_strides(a_shape), contiguous_strides(b_shape)
    a_store, b_store = a, b
    if a_perm:
        a_store, a_st = np.ascontiguousarray(a.transpose(0, 2, 1)), [m * k, 1, m]
    if b_perm:
        b_store, b_st = np.ascontiguousarray(b.transpose(0, 2, 1)), [k * n, 1, k]
    if b_bcast:
        b_st[0] = 0
    md = meta_matmul([batch, m, n], a_shape, b_shape, a_st, b_st)
    sa, sb = to_storage(a_store.ravel(), dt), to_storage(b_store.ravel(), dt)
    # values as the kernels see them (bf16-rounded)
    av = to_float(to_storage(a.ravel(), dt), dt).reshape(a.shape).astype(np.float64)
    bv = to_float(to_storage(b.ravel(), dt), dt).reshape(b.shape).astype(np.float64)
    return sa, sb, md, av, np.broadcast_to(bv, (batch, k, n))


MM_SHAPES = [# whole k-tiles, last tiles running past the rows and the columns (loaded through bounded descriptors); ragged in all three
             (1, 1000, 1024, 1000), (2, 130, 256, 200), (1, 250, 192, 260), (1, 129, 128, 4), (1, 33, 640, 132), (1, 1000, 1000, 1000),
             # a reduction that is not whole k-tiles, in batches: the operands are copied with the reduction zero-padded
             (2, 130, 1000, 200), (3, 256, 100, 256),
             (1, 300, 8, 256), (3, 128, 5, 264), (1, 4096, 16, 64),      # short reductions, many outputs: a thread per 16-byte vector of them
             (1, 128, 128, 128), (1, 256, 192, 320), (2, 130, 70, 97), (3, 64, 600, 64), (1, 1000, 3, 1), (1, 3, 1000, 1),
             (1, 10000, 3, 1), (1, 1, 257, 1), (2, 37, 19, 53), (1, 512, 64, 64), (1, 100, 576, 64), (4, 16, 16, 16),
             # long reductions with few output tiles (split over the reduction), tall outputs with few columns
             (1, 96, 5000, 64), (1, 130, 4100, 70), (2, 64, 2048, 64), (1, 2048, 576, 64), (1, 1100, 100, 33),
             # few output columns and a long reduction along which both operands are strided (a_perm): tiles, not a wave per output
             (1, 128, 5000, 10), (1, 40, 2100, 12),
             # a handful of outputs, each a long dot product (one block per output)
             (1, 2, 5000, 3), (2, 1, 4096, 1)]


@pytest.mark.parametrize("dt", DTS)
@pytest.mark.parametrize("a_perm,b_perm", [(False, False), (True, False), (False, True), (True, True)])
@pytest.mark.parametrize("shape", MM_SHAPES, ids=lambda s: "x".join(map(str, s)))
def test_matmul_forward(oracle, hip, shape, a_perm, b_perm, dt):
    batch, m, k, n = shape
    r = rng(43)
    sa, sb, md, av, bv = matmul_inputs(r, batch, m, k, n, a_perm, b_perm, dt)
    (h,) = hip.call(f"matmul_{dt}", batch * m * n, md, In(sa), In(sb), Out(batch * m * n, dt))
    truth = np.einsum("bmk,bkn->bmn", av, bv)
    scale = np.einsum("bmk,bkn->bmn", np.abs(av), np.abs(bv))
    tol = 1e-5 if dt == "f32" else 1e-2
    err = np.abs(to_float(h, dt).reshape(truth.shape) - truth) / np.maximum(scale, 1e-30)
    assert np.max(err) <= tol, float(np.max(err))
    if dt == "f32" and batch * m * n * k <= 5_000_000:
        (o,) = oracle.call("matmul_f32", batch * m * n, md, In(sa), In(sb), Out(batch * m * n, "f32"))
        assert np.max(np.abs(o - h).reshape(truth.shape) / np.maximum(scale, 1e-30)) <= 2e-5
        if k <= 16:   # thread-per-output kernel keeps the reference's order: identical bits
            assert same_bits(o, h)


def test_matmul_refuses_operands_whose_inner_extents_disagree(hip):
    """The kernels index b with a's reduction length: a b that says it has fewer rows would be read past its end."""
    md = meta_matmul([8, 16], [8, 16], [4, 16], [16, 1], [16, 1])
    with pytest.raises(Exception):
        hip.call("matmul_f32", 8 * 16, md, In(np.ones(8 * 16, np.float32)), In(np.ones(4 * 16, np.float32)), Out(8 * 16, "f32"))


@pytest.mark.parametrize("dt", DTS)
@pytest.mark.parametrize("layout", ["row-major operands", "a turned", "b turned"])
def test_matmul_of_unaligned_views_matches_the_aligned_product(hip, layout, dt):
    """Operands that start one element into their buffers (no 16-byte alignment) with a reduction of whole k-tiles plus a
    tail: the product copies them, zero-padded, and runs the unchecked kernels.  Same values as the float64 product."""
    m, k, n = 300, 1000, 256
    r = rng(67)
    a = r.standard_normal((m, k)).astype(np.float32)
    b = r.standard_normal((k, n)).astype(np.float32)
    a_store, a_st = (a.T.copy(), [1, m]) if layout == "a turned" else (a, [k, 1])
    b_store, b_st = (b.T.copy(), [1, k]) if layout == "b turned" else (b, [n, 1])
    sa = to_storage(np.concatenate([[0.0], a_store.ravel()]).astype(np.float32), dt)
    sb = to_storage(np.concatenate([[0.0], b_store.ravel()]).astype(np.float32), dt)
    md = meta_matmul([m, n], [m, k], [k, n], a_st, b_st, 1, 1)
    (h,) = hip.call(f"matmul_{dt}", m * n, md, In(sa), In(sb), Out(m * n, dt))
    av = to_float(sa, dt)[1:].reshape(a_store.shape).astype(np.float64)
    bv = to_float(sb, dt)[1:].reshape(b_store.shape).astype(np.float64)
    av = av.T if layout == "a turned" else av
    bv = bv.T if layout == "b turned" else bv
    truth, scale = av @ bv, np.abs(av) @ np.abs(bv)
    tol = 1e-5 if dt == "f32" else 1e-2
    assert np.max(np.abs(to_float(h, dt).reshape(m, n) - truth) / scale) <= tol


@pytest.mark.parametrize("dt", DTS)
@pytest.mark.parametrize("a_perm,b_perm", [(False, False), (True, False), (False, True), (True, True)])
@pytest.mark.parametrize("shape", [(1, 4096, 64, 3072), (1, 4096, 128, 3072), (1, 3072, 320, 4096), (3, 2048, 192, 2048)],
                         ids=lambda s: "x".join(map(str, s)))
def test_matmul_whole_256_tiles(hip, shape, a_perm, b_perm, dt):
    """At least 192 whole 256x256 output tiles: the unchecked 8-wave configuration (1, 2, 5 and 3 k-tiles for bf16),
    for every operand layout."""
    batch, m, k, n = shape
    r = rng(59)
    sa, sb, md, av, bv = matmul_inputs(r, batch, m, k, n, a_perm, b_perm, dt)
    (h,) = hip.call(f"matmul_{dt}", batch * m * n, md, In(sa), In(sb), Out(batch * m * n, dt))
    truth = np.einsum("bmk,bkn->bmn", av, bv)
    scale = np.einsum("bmk,bkn->bmn", np.abs(av), np.abs(bv))
    tol = 1e-5 if dt == "f32" else 1e-2
    err = np.abs(to_float(h, dt).reshape(truth.shape) - truth) / np.maximum(scale, 1e-30)
    assert np.max(err) <= tol, float(np.max(err))


@pytest.mark.parametrize("dt", DTS)
@pytest.mark.parametrize("a_perm,b_perm", [(False, False), (True, False), (False, True), (True, True)])
@pytest.mark.parametrize("shape", [(1, 32768, 64, 192), (1, 100352, 96, 128), (1, 40960, 128, 64 * 9), (1, 65600 * 64 // 64, 32, 64)], ids=lambda s: "x".join(map(str, s)))
def test_matmul_short_reduction_row_panels(hip, shape, a_perm, b_perm, dt):
    """Whole 64-wide tiles and a reduction of a few k-tiles: as many blocks as the chip holds, each walking a run of
    output tiles (the convolution's input gradient is such a product), for every operand layout; tile counts that do and
    do not divide evenly among the blocks, runs that cross from one tile row to the next."""
    batch, m, k, n = shape
    r = rng(61)
    sa, sb, md, av, bv = matmul_inputs(r, batch, m, k, n, a_perm, b_perm, dt)
    (h,) = hip.call(f"matmul_{dt}", batch * m * n, md, In(sa), In(sb), Out(batch * m * n, dt))
    got = to_float(h, dt).reshape(batch, m, n)
    rows = np.unique(np.concatenate([np.arange(0, 130), r.integers(0, m, 600), np.arange(m - 130, m)]))
    truth = np.einsum("bmk,bkn->bmn", av[:, rows], bv)
    scale = np.einsum("bmk,bkn->bmn", np.abs(av[:, rows]), np.abs(bv))
    tol = 1e-5 if dt == "f32" else 1e-2
    err = np.abs(got[:, rows] - truth) / np.maximum(scale, 1e-30)
    assert np.max(err) <= tol, float(np.max(err))
    assert np.isfinite(got).all()


@pytest.mark.parametrize("dt", DTS)
@pytest.mark.parametrize("a_perm,b_perm", [(False, False), (True, False), (False, True)])
@pytest.mark.parametrize("shape", [(1, 1, 300, 256), (1, 2, 4096, 264), (1, 3, 1000, 520), (1, 5, 257, 1024), (1, 8, 2050, 512), (1, 1, 4099, 4096),
                                   (1, 8, 2048, 515), (1, 5, 512, 1000), (1, 4, 8200, 70)],
                         ids=lambda s: "x".join(map(str, s)))
def test_matmul_few_rows(oracle, hip, shape, a_perm, b_perm, dt):
    """One to eight output rows.  Against a row-major right operand: the kernel that streams its rows (a lane per 16-byte
    vector of columns, a wave per run of rows, partial rows folded in chunk order) - ragged reductions, column counts
    that leave lanes of the last wave idle, a left operand given transposed, the right operand as a column slice of a
    wider matrix.  Against a right operand given transposed (a linear layer's x W^T): a wave per output column."""
    batch, m, k, n = shape
    r = rng(67)
    sa, sb, md, av, bv = matmul_inputs(r, batch, m, k, n, a_perm, b_perm, dt)
    (h,) = hip.call(f"matmul_{dt}", m * n, md, In(sa), In(sb), Out(m * n, dt))
    truth = np.einsum("bmk,bkn->bmn", av, bv)
    scale = np.einsum("bmk,bkn->bmn", np.abs(av), np.abs(bv))
    tol = 1e-5 if dt == "f32" else 1e-2
    err = np.abs(to_float(h, dt).reshape(truth.shape) - truth) / np.maximum(scale, 1e-30)
    assert np.max(err) <= tol, float(np.max(err))
    if dt == "f32" and m * n * k <= 5_000_000:
        (o,) = oracle.call("matmul_f32", m * n, md, In(sa), In(sb), Out(m * n, "f32"))
        assert np.max(np.abs(o - h).reshape(truth.shape) / np.maximum(scale, 1e-30)) <= 2e-5
    if b_perm:
        return
    # the right operand as the first n columns of a matrix twice as wide (row stride 2n)
    wide = np.zeros((k, 2 * n), np.float32)
    wide[:, :n] = bv[0]
    wide[:, n:] = 7.0
    mdw = meta_matmul([m, n], [m, k], [k, n], [1, m] if a_perm else [k, 1], [2 * n, 1])
    (hw,) = hip.call(f"matmul_{dt}", m * n, mdw, In(sa), In(to_storage(wide.ravel(), dt)), Out(m * n, dt))
    assert same_bits(h, hw)


def test_matmul_strided_rows_is_the_full_product(oracle, hip):
    """A = big[:, :k], a view whose rows are 3k apart.  The CPU reference drops every term whose operand index reaches
    num_els * k (crates/maidenx_cpu/src/ops/matmul.rs:53-54,109), which cuts the later rows short; the GPU computes the
    whole product.  The oracle, which restates the CPU, differs by exactly those terms."""
    r = rng(71)
    m, k, n, wide = 40, 24, 16, 72
    big = r.standard_normal((m, wide)).astype(np.float32)
    b = r.standard_normal((k, n)).astype(np.float32)
    md = meta_matmul([m, n], [m, k], [k, n], [wide, 1], [n, 1])
    (h,) = hip.call("matmul_f32", m * n, md, In(big.ravel()), In(b.ravel()), Out(m * n, "f32"))
    (o,) = oracle.call("matmul_f32", m * n, md, In(big.ravel()), In(b.ravel()), Out(m * n, "f32"))
    a64, b64 = big[:, :k].astype(np.float64), b.astype(np.float64)
    full = a64 @ b64
    scale = np.abs(a64) @ np.abs(b64)
    assert np.max(np.abs(h.reshape(m, n) - full) / scale) <= 1e-5
    # the guard: a term (i, r) survives when i * wide + r < m * n * k  (and the B index, always small here, does too)
    limit = m * n * k
    keep = (np.arange(m)[:, None] * wide + np.arange(k)[None, :]) < limit
    assert keep.all()                  # (with these sizes every index is below the limit ...)
    truncated = (a64 * keep) @ b64
    assert np.max(np.abs(o.reshape(m, n) - truncated) / scale) <= 1e-5
    # ... so make the guard bite: the same view of a taller matrix with a single output column
    m2, n2 = 400, 1
    big2 = r.standard_normal((m2, wide)).astype(np.float32)
    b2 = r.standard_normal((k, n2)).astype(np.float32)
    md2 = meta_matmul([m2, n2], [m2, k], [k, n2], [wide, 1], [n2, 1])
    (h2,) = hip.call("matmul_f32", m2 * n2, md2, In(big2.ravel()), In(b2.ravel()), Out(m2 * n2, "f32"))
    (o2,) = oracle.call("matmul_f32", m2 * n2, md2, In(big2.ravel()), In(b2.ravel()), Out(m2 * n2, "f32"))
    a2, bb2 = big2[:, :k].astype(np.float64), b2.astype(np.float64)
    keep2 = (np.arange(m2)[:, None] * wide + np.arange(k)[None, :]) < m2 * n2 * k
    assert not keep2.all()
    scale2 = np.abs(a2) @ np.abs(bb2)
    assert np.max(np.abs(h2.reshape(m2, n2) - a2 @ bb2) / scale2) <= 1e-5
    assert np.max(np.abs(o2.reshape(m2, n2) - (a2 * keep2) @ bb2) / scale2) <= 1e-5
    assert np.max(np.abs(o2 - h2)) > 0.1            # rows beyond the limit are all zeros in the oracle's result


def test_matmul_broadcast_batch_uses_stride0(oracle, hip):
    r = rng(47)
    sa, sb, md, av, bv = matmul_inputs(r, 3, 40, 50, 60, False, False, "f32", b_bcast=True)
    (o,), (h,) = both(oracle, hip, "matmul_f32", lambda: (3 * 40 * 60, md, In(sa), In(sb), Out(3 * 40 * 60, "f32")))
    assert np.allclose(o, h, rtol=1e-4, atol=1e-5)


@pytest.mark.parametrize("dt", DTS)
@pytest.mark.parametrize("shape", [(1, 128, 128, 128), (2, 130, 70, 97), (1, 10000, 3, 1), (1, 300, 576, 64), (3, 33, 65, 17), (1, 3000, 96, 64),
                          (1, 4096, 64, 576)],
                         ids=lambda s: "x".join(map(str, s)))
def test_matmul_backward(oracle, hip, shape, dt):
    batch, m, k, n = shape
    r = rng(53)
    sa, sb, md, av, bv = matmul_inputs(r, batch, m, k, n, False, False, dt)
    go = r.standard_normal((batch, m, n)).astype(np.float32)
    sg = to_storage(go.ravel(), dt)
    gv = to_float(sg, dt).reshape(go.shape).astype(np.float64)
    ga, gb = hip.call(f"matmul_backward_{dt}", batch * m * k, batch * k * n, md, In(sg), In(sa), In(sb), Out(batch * m * k, dt),
                      Out(batch * k * n, dt))
    tol = 1e-5 if dt == "f32" else 1e-2
    ta = np.einsum("bmn,bkn->bmk", gv, bv)
    tb = np.einsum("bmk,bmn->bkn", av, gv)
    sa_ = np.einsum("bmn,bkn->bmk", np.abs(gv), np.abs(bv))
    sb_ = np.einsum("bmk,bmn->bkn", np.abs(av), np.abs(gv))
    floor = 2.0 ** -24 if dt == "f16" else 0.0       # f16 results below 6.1e-5 are subnormal: absolute spacing 2^-24
    assert np.max((np.abs(to_float(ga, dt).reshape(ta.shape) - ta) - floor) / np.maximum(sa_, 1e-30)) <= tol
    assert np.max(np.abs(to_float(gb, dt).reshape(tb.shape) - tb) / np.maximum(sb_, 1e-30)) <= tol
    # either gradient may be absent
    (ga2,) = hip.call(f"matmul_backward_{dt}", batch * m * k, batch * k * n, md, In(sg), In(sa), In(sb), Out(batch * m * k, dt), None)
    (gb2,) = hip.call(f"matmul_backward_{dt}", batch * m * k, batch * k * n, md, In(sg), In(sa), In(sb), None, Out(batch * k * n, dt))
    assert same_bits(ga, ga2) and same_bits(gb, gb2)
    # and, in f32, against the CPU restatement of matmul_backward (matmul.rs:124-268) itself where it finishes in a moment
    # (its 16-bit forms accumulate in the storage type, matmul.rs:281-282: their own rounding is the larger error)
    if dt == "f32" and batch * m * k * n <= 5_000_000:
        oa, ob = oracle.call("matmul_backward_f32", batch * m * k, batch * k * n, md, In(sg), In(sa), In(sb), Out(batch * m * k, dt),
                             Out(batch * k * n, dt))
        assert np.max(np.abs(ga.astype(np.float64) - oa).reshape(ta.shape) / np.maximum(sa_, 1e-30)) <= 2e-5
        assert np.max(np.abs(gb.astype(np.float64) - ob).reshape(tb.shape) / np.maximum(sb_, 1e-30)) <= 2e-5


# ---------------------------------------------------------------------------------------------------
# padding, im2col, col2im: bit-exact
# ---------------------------------------------------------------------------------------------------
PAD_CASES = [([2, 3, 8, 8], [(0, 0), (0, 0), (1, 1), (1, 1)]), ([7], [(3, 0)]), ([5, 6], [(1, 2), (0, 3)]), ([2, 3, 4], [(1, 0), (0, 2), (2, 1)]),
             ([4, 16, 14, 14], [(0, 0), (0, 0), (1, 1), (1, 1)]), ([3, 5], [(0, 0), (0, 0)])]


@pytest.mark.parametrize("dt", DTS + ["f64"])
@pytest.mark.parametrize("shape,pads", PAD_CASES)
def test_pad_constant_forward_backward(oracle, hip, shape, pads, dt):
    r = rng(59)
    out_shape = [s + p[0] + p[1] for s, p in zip(shape, pads)]
    n_in, n_out = int(np.prod(shape)), int(np.prod(out_shape))
    st = to_storage(np.concatenate([[9.0], r.standard_normal(n_in)]).astype(np.float32), dt)
    md = meta_pad(shape, contiguous_strides(shape), 1, out_shape, pads)
    (o,), (h,) = both(oracle, hip, f"pad_with_constant_{dt}",
                      lambda: (n_in, n_out, len(shape), md, In(st), Out(n_out, dt), const_arg(-1.5, dt)))
    assert same_bits(o, h)
    go = to_storage(r.standard_normal(n_out).astype(np.float32), dt)
    go[:1] = to_storage(np.array([-0.0], np.float32), dt)
    (o,), (h,) = both(oracle, hip, f"pad_with_constant_backward_{dt}",
                      lambda: (n_in, n_out, len(shape), md, In(go), InOut(to_storage(np.full(n_in + 2, 7.0, np.float32), dt))))
    assert same_bits(o, h)


def int_values(r, n, dt):
    """Integers over the whole range of the dtype, so that the backward sums wrap."""
    info = np.iinfo(NP[dt])
    return r.integers(info.min, info.max, n, dtype=NP[dt], endpoint=True)


@pytest.mark.parametrize("dt", INT_DTS)
@pytest.mark.parametrize("shape,pads", PAD_CASES[:4] + [([3, 20, 24], [(0, 0), (3, 3), (2, 5)])])
def test_pad_three_modes_integer_dtypes(oracle, hip, shape, pads, dt):
    """Forward modes copy, backward modes add in the storage type with wrap-around: bit-exact whatever the order."""
    r = rng(241)
    out_shape = [s + p[0] + p[1] for s, p in zip(shape, pads)]
    n_in, n_out = int(np.prod(shape)), int(np.prod(out_shape))
    x = np.concatenate([int_values(r, 1, dt), int_values(r, n_in, dt)])
    go = int_values(r, n_out, dt)
    md = meta_pad(shape, contiguous_strides(shape), 1, out_shape, pads)
    (o,), (h,) = both(oracle, hip, f"pad_with_constant_{dt}", lambda: (n_in, n_out, len(shape), md, In(x), Out(n_out, dt), const_arg(5, dt)))
    assert same_bits(o, h)
    assert np.array_equal(h.reshape(out_shape), np.pad(x[1:].reshape(shape), pads, constant_values=5))
    (o,), (h,) = both(oracle, hip, f"pad_with_constant_backward_{dt}",
                      lambda: (n_in, n_out, len(shape), md, In(go), InOut(np.full(n_in + 2, 7, NP[dt]))))
    assert same_bits(o, h)
    for mode, np_mode in (("reflection", "reflect"), ("replication", "edge")):
        if mode == "reflection" and any(s == 1 and (p[0] or p[1]) for s, p in zip(shape, pads)):
            continue
        (o,), (h,) = both(oracle, hip, f"pad_with_{mode}_{dt}", lambda: (n_in, n_out, len(shape), md, In(x), Out(n_out, dt)))
        assert same_bits(o, h)
        assert np.array_equal(h.reshape(out_shape), np.pad(x[1:].reshape(shape), pads, mode=np_mode))
        (o,), (h,) = both(oracle, hip, f"pad_with_{mode}_backward_{dt}",
                          lambda: (n_in, n_out, len(shape), md, In(go), InOut(np.full(n_in + 2, 7, NP[dt]))))
        assert same_bits(o, h)
        # each input position receives the wrapped sum of the output gradients that were read from it
        idx = np.pad(np.arange(n_in).reshape(shape), pads, mode=np_mode).ravel()
        want = np.zeros(n_in, dtype=NP[dt])
        with np.errstate(over="ignore"):
            np.add.at(want, idx, go)
        assert np.array_equal(h[1:n_in + 1], want) and h[0] == 7 and h[-1] == 7


def test_pad_transposed_input(oracle, hip):
    lay = LY.permuted([6, 9], [1, 0])
    r = rng(61)
    st = r.standard_normal(lay["size"]).astype(np.float32)
    pads = [(1, 1), (2, 0)]
    out_shape = [8, 11]
    md = meta_pad(lay["dims"], lay["strides"], 0, out_shape, pads)
    (o,), (h,) = both(oracle, hip, "pad_with_constant_f32", lambda: (54, 88, 2, md, In(st), Out(88, "f32"), 0.0))
    assert same_bits(o, h)
    assert np.array_equal(o.reshape(out_shape), np.pad(LY.gather(st, lay), pads))


CONV_CASES = [(2, 3, 8, 8, 3, 3, 1, 1), (1, 4, 12, 12, 3, 3, 1, 1), (2, 2, 9, 7, 2, 3, 1, 2), (1, 1, 5, 5, 1, 1, 0, 1), (2, 3, 10, 10, 5, 5, 2, 2),
             (3, 8, 14, 14, 3, 3, 1, 1), (1, 2, 6, 6, 3, 3, 0, 1),
             # several bands of output rows per plane: a short last band, stride 2, a tile limited by LDS
             (1, 2, 37, 64, 3, 3, 1, 1), (1, 2, 80, 63, 3, 3, 1, 2), (1, 1, 24, 512, 3, 3, 1, 1), (2, 3, 16, 16, 3, 3, 1, 1),
             # unit stride with 5x5, 1x1 and 2x4 kernels (col2im's compile-time and run-time tap loops)
             (1, 2, 16, 16, 5, 5, 2, 1), (1, 2, 8, 8, 1, 1, 0, 1), (2, 2, 9, 16, 2, 4, 1, 1)]


@pytest.mark.parametrize("dt", DTS + ["f64"])
@pytest.mark.parametrize("case", CONV_CASES, ids=lambda c: "_".join(map(str, c)))
def test_im2col_col2im_bit_exact(oracle, hip, case, dt):
    B, Cc, H, W, kh, kw, p, s = case
    oh, ow = (H + 2 * p - kh) // s + 1, (W + 2 * p - kw) // s + 1
    r = rng(67)
    x = to_storage(r.standard_normal(B * Cc * H * W).astype(np.float32), dt)
    n_col = B * Cc * kh * kw * oh * ow
    md = meta_conv(B, Cc, H, W, kh, kw, oh, ow, p, p, s, s)
    (o,), (h,) = both(oracle, hip, f"conv2d_im2col_{dt}", lambda: (n_col, md, In(x), Out(n_col, dt)))
    assert same_bits(o, h)
    y = to_storage(r.standard_normal(n_col).astype(np.float32), dt)
    for num_els in (n_col, B * Cc * H * W):      # full, and the truncation the reference's Conv2d passes
        (o,), (h,) = both(oracle, hip, f"conv2d_col2im_{dt}", lambda: (num_els, md, In(y), Out(B * Cc * H * W, dt)))
        assert same_bits(o, h), num_els


# (B, C, H, W, kh, kw, pad, stride): ragged tiles, odd widths (element-by-element gather), planes shorter than a tile's
# run of rows, stride 2, whole 64-wide tiles with a 576-term reduction, a reduction long enough for the split
COLS_CASES = CONV_CASES[:7] + [(2, 3, 16, 16, 3, 3, 1, 1), (1, 2, 9, 16, 2, 4, 1, 1), (4, 16, 14, 14, 3, 3, 1, 1), (2, 8, 16, 20, 3, 3, 1, 1),
                               (2, 5, 12, 13, 3, 3, 1, 1), (3, 4, 23, 23, 3, 3, 2, 2), (8, 64, 28, 28, 3, 3, 1, 1), (2, 64, 56, 56, 3, 3, 1, 1)]


@pytest.mark.parametrize("rhs_turned", [False, True])
@pytest.mark.parametrize("transposed", [0, 1])
@pytest.mark.parametrize("n", [64, 24])
@pytest.mark.parametrize("case", COLS_CASES, ids=lambda c: "_".join(map(str, c)))
def test_conv2d_cols_matmul(oracle, hip, case, n, transposed, rhs_turned):
    """The product of the (never stored) column matrix, or of its transpose, with a matrix: against the oracle's im2col
    followed by its matmul, against float64, and bit for bit against the stored way (hip im2col, then hip matmul)
    wherever that runs on the matrix cores too."""
    B, Cc, H, W, kh, kw, p, s = case
    oh, ow = (H + 2 * p - kh) // s + 1, (W + 2 * p - kw) // s + 1
    M, K = B * oh * ow, Cc * kh * kw
    r = rng(73)
    x = r.standard_normal(B * Cc * H * W).astype(np.float32)
    md = meta_conv(B, Cc, H, W, kh, kw, oh, ow, p, p, s, s)
    rows = M if transposed else K                      # of rhs; out is [K, n] or [M, n]
    I = K if transposed else M
    rhs = r.standard_normal((rows, n)).astype(np.float32)
    st = np.ascontiguousarray(rhs.T) if rhs_turned else rhs          # storage; rhs[i, j] at i*rs[0] + j*rs[1]
    rs = u64(1, rows) if rhs_turned else u64(n, 1)
    (h,) = hip.call("conv2d_cols_matmul_f32", md, transposed, In(x), In(st.ravel()), n, rs, Out(I * n, "f32"))
    (cols,) = oracle.call("conv2d_im2col_f32", M * K, md, In(x), Out(M * K, "f32"))
    a = cols.reshape(M, K).T if transposed else cols.reshape(M, K)
    truth = a.astype(np.float64) @ rhs.astype(np.float64)
    scale = np.abs(a).astype(np.float64) @ np.abs(rhs).astype(np.float64)
    err = np.abs(h.reshape(I, n) - truth) / np.maximum(scale, 1e-30)
    assert np.max(err) <= 1e-5, float(np.max(err))
    a_str, b_str = ([1, K] if transposed else [K, 1]), [int(rs[0]), int(rs[1])]
    mm = meta_matmul([I, n], [I, rows], [rows, n], a_str, b_str)
    if I * n * rows <= 5_000_000:
        (o,) = oracle.call("matmul_f32", I * n, mm, In(cols), In(st.ravel()), Out(I * n, "f32"))
        assert np.max(np.abs(o - h).reshape(I, n) / np.maximum(scale, 1e-30)) <= 2e-5
    (hc,) = hip.call("conv2d_im2col_f32", M * K, md, In(x), Out(M * K, "f32"))
    assert same_bits(hc, cols)
    (hs,) = hip.call("matmul_f32", I * n, mm, In(hc), In(st.ravel()), Out(I * n, "f32"))
    outputs = I * n
    on_matrix_cores = rows > 16 and not (I < 16 and n < 16 and rows < 256) and not (outputs <= 64 and rows >= 4096) and \
        not (outputs <= 4096 and (I < 32 or n < 32))
    if on_matrix_cores:
        assert same_bits(hs, h)


@pytest.mark.parametrize("Bn,P,K,J", [(3, 3136, 576, 64), (192, 49, 64, 64), (16, 1000, 96, 64), (2, 4160, 32, 64)])
def test_conv2d_forward_product_is_matmul_then_transposes_then_add(oracle, hip, Bn, P, K, J):
    """hip_conv2d_forward_product_f32 against the three calls it stands for (conv.rs:217-232): the product [B*P, K] x [K, J]
    (w^T as a strided operand), the [B, P, J] -> [B, J, P] view, the bias add through it - bit for bit; and against the
    oracle's product to the GEMM tolerance.  Planes of 49 and 1000 pixels put batch boundaries inside the 64-row tiles."""
    r = rng(900 + P)
    M = Bn * P
    x = r.standard_normal((M, K)).astype(np.float32)
    w = (r.standard_normal((J, K)) * 0.1).astype(np.float32)
    bias = r.standard_normal(J).astype(np.float32)
    (got,) = hip.call("conv2d_forward_product_f32", M, K, J, P, In(x), In(w), In(bias), Out(M * J, "f32"))
    assert hip.last_return == 1
    (prod,) = hip.call("matmul_f32", M * J, meta_matmul([M, J], [M, K], [K, J], [K, 1], [1, K]), In(x), In(w), Out(M * J, "f32"))
    md = meta_binary([Bn, J, P], [P * J, 1, J], [0, 1, 0])
    (want,) = hip.call("add_f32", M * J, 3, md, In(prod), In(bias), Out(M * J, "f32"))
    assert same_bits(got, want)
    ref = (x.astype(np.float64) @ w.astype(np.float64).T).reshape(Bn, P, J).transpose(0, 2, 1) + bias[None, :, None]
    scale = (np.abs(x).astype(np.float64) @ np.abs(w).astype(np.float64).T).max() + np.abs(bias).max()
    assert np.abs(got.reshape(Bn, J, P) - ref).max() <= 1e-5 * scale


def test_conv2d_forward_product_declines_other_shapes(hip):
    """Rows that are not whole tiles, another column count, a ragged reduction, few tiles: 0 and nothing written."""
    x, w, bias = np.zeros(64 * 300 * 40, np.float32), np.zeros(64 * 40, np.float32), np.zeros(64, np.float32)
    for M, K, J, P in ((64 * 300 + 8, 32, 64, 4), (64 * 300, 32, 128, 100), (64 * 300, 40, 64, 100), (64 * 100, 32, 64, 100), (64 * 300, 32, 64, 7)):
        out = np.full(8, -3.0, np.float32)
        (o,) = hip.call("conv2d_forward_product_f32", M, K, J, P, In(x), In(w), In(bias), InOut(out))
        assert hip.last_return == 0, (M, K, J, P)
        assert (o == -3.0).all()


def test_conv2d_cols_matmul_rejects_what_it_cannot_index(hip):
    x = np.zeros(16, np.float32)
    md = meta_conv(1, 1, 4, 4, 3, 3, 4, 4, 1, 1, 1, 1)
    with pytest.raises(hip.L.HipError, match="unit stride"):
        hip.call("conv2d_cols_matmul_f32", md, 0, In(x), In(np.zeros(64, np.float32)), 2, u64(4, 2), Out(32, "f32"))
    big = meta_conv(1 << 12, 64, 64, 64, 3, 3, 64, 64, 1, 1, 1, 1)       # a column matrix of 2^31 entries and more
    with pytest.raises(hip.L.HipError, match="2\\^31"):
        hip.call("conv2d_cols_matmul_f32", big, 0, In(x), In(np.zeros(64, np.float32)), 2, u64(2, 1), Out(32, "f32"))


@pytest.mark.parametrize("dt", DTS + ["f64"])
@pytest.mark.parametrize("k", [3, 4])
def test_col2im_row_stride_two_column_stride_one(oracle, hip, k, dt):
    B, Cc, H, W, p, sh, sw = 2, 3, 15, 16, 1, 2, 1
    oh, ow = (H + 2 * p - k) // sh + 1, (W + 2 * p - k) // sw + 1
    n_col = B * Cc * k * k * oh * ow
    md = meta_conv(B, Cc, H, W, k, k, oh, ow, p, p, sh, sw)
    y = to_storage(rng(68).standard_normal(n_col).astype(np.float32), dt)
    for num_els in (n_col, n_col // 2 + 3):
        (o,), (h,) = both(oracle, hip, f"conv2d_col2im_{dt}", lambda: (num_els, md, In(y), Out(B * Cc * H * W, dt)))
        assert same_bits(o, h), num_els


@pytest.mark.parametrize("B,Cc,H,W,k,p,sh,sw", [(2, 3, 16, 16, 3, 1, 1, 1), (2, 3, 15, 16, 3, 1, 2, 1), (1, 2, 9, 7, 3, 1, 1, 1), (3, 4, 12, 12, 5, 2, 1, 1),
                                                 (2, 5, 8, 8, 1, 1, 1, 1), (2, 2, 10, 12, 4, 1, 2, 3)])
def test_col2im_add_is_col2im_then_add_inplace(oracle, hip, B, Cc, H, W, k, p, sh, sw):
    """hip_conv2d_col2im_add_f32 against the two calls it stands for - col2im into a fresh buffer, then add_inplace into
    the gradient (lib.rs:221-241) - on the GPU and on the oracle: the same bits, for whole and truncated num_els (planes
    beyond num_els add +0: a -0 in the gradient becomes +0 there), vector and scalar kernels."""
    oh, ow = (H + 2 * p - k) // sh + 1, (W + 2 * p - k) // sw + 1
    n_col, n_in = B * Cc * k * k * oh * ow, B * Cc * H * W
    md = meta_conv(B, Cc, H, W, k, k, oh, ow, p, p, sh, sw)
    r = rng(70 + k + H)
    y = r.standard_normal(n_col).astype(np.float32)
    grad0 = r.standard_normal(n_in).astype(np.float32)
    grad0[::7] = -0.0
    grad0[3::11] = 0.0
    for num_els in (n_col, n_in, n_col // 2 + 3):
        (got,) = hip.call("conv2d_col2im_add_f32", num_els, md, In(y), InOut(grad0.copy()))
        for be in (hip, oracle):
            (gi,) = be.call("conv2d_col2im_f32", num_els, md, In(y), Out(n_in, "f32"))
            (want,) = be.call("add_inplace_f32", n_in, 1, meta_binary([n_in], [1], [1]), InOut(grad0.copy()), In(gi))
            assert same_bits(got, want), (num_els, be.kind)


# ---------------------------------------------------------------------------------------------------
# reflection / replication padding, fold, softmax
# ---------------------------------------------------------------------------------------------------
EDGE_CASES = [([7], [(3, 2)]), ([5, 6], [(1, 2), (0, 3)]), ([2, 3, 4], [(1, 0), (2, 2), (3, 1)]), ([4, 9], [(0, 0), (4, 8)]),
              ([3], [(7, 5)]), ([2, 3, 20, 24], [(0, 0), (0, 0), (3, 3), (2, 5)]), ([1, 6], [(0, 0), (2, 2)])]


@pytest.mark.parametrize("dt", DTS + ["f64"])
@pytest.mark.parametrize("mode", ["reflection", "replication"])
@pytest.mark.parametrize("shape,pads", EDGE_CASES)
def test_pad_edge_forward_backward(oracle, hip, shape, pads, mode, dt):
    r = rng(103)
    out_shape = [s + p[0] + p[1] for s, p in zip(shape, pads)]
    n_in, n_out = int(np.prod(shape)), int(np.prod(out_shape))
    st = to_storage(np.concatenate([[9.0], r.standard_normal(n_in)]).astype(np.float32), dt)
    md = meta_pad(shape, contiguous_strides(shape), 1, out_shape, pads)
    (o,), (h,) = both(oracle, hip, f"pad_with_{mode}_{dt}", lambda: (n_in, n_out, len(shape), md, In(st), Out(n_out, dt)))
    assert same_bits(o, h)
    go = to_storage(r.standard_normal(n_out).astype(np.float32), dt)
    (o,), (h,) = both(oracle, hip, f"pad_with_{mode}_backward_{dt}",
                      lambda: (n_in, n_out, len(shape), md, In(go), InOut(to_storage(np.full(n_in + 2, 7.0, np.float32), dt))))
    if dt == "f32":
        assert same_bits(o, h)          # same terms in the same (ascending output) order
    else:
        # the reference rounds after every add, the kernel once: compare with the exact sums
        assert same_bits(o[:1], h[:1]) and same_bits(o[n_in + 1:], h[n_in + 1:])
        g64 = to_float(go, dt).astype(np.float64).reshape(out_shape)
        np_mode = "reflect" if mode == "reflection" else "edge"
        idx = np.pad(np.arange(n_in).reshape(shape), pads, mode=np_mode).ravel()
        truth = np.bincount(idx, weights=g64.ravel(), minlength=n_in)
        scale = np.bincount(idx, weights=np.abs(g64).ravel(), minlength=n_in)
        assert np.max(np.abs(to_float(h, dt)[1:n_in + 1] - truth) / np.maximum(scale, 1e-30)) <= 1e-2


@pytest.mark.parametrize("mode", ["reflection", "replication"])
def test_pad_edge_transposed_input(oracle, hip, mode):
    lay = LY.permuted([6, 9], [1, 0])
    r = rng(107)
    st = r.standard_normal(54).astype(np.float32)
    pads = [(2, 1), (3, 4)]
    md = meta_pad([6, 9], lay["strides"], 0, [9, 16], pads)
    (o,), (h,) = both(oracle, hip, f"pad_with_{mode}_f32", lambda: (54, 144, 2, md, In(st), Out(144, "f32")))
    assert same_bits(o, h)
    go = r.standard_normal(144).astype(np.float32)
    (o,), (h,) = both(oracle, hip, f"pad_with_{mode}_backward_f32", lambda: (54, 144, 2, md, In(go), InOut(np.full(54, 7.0, np.float32))))
    assert same_bits(o, h)


def test_pad_reflection_of_a_size_one_dim_is_refused(hip):
    md = meta_pad([1, 4], [4, 1], 0, [3, 4], [(1, 1), (0, 0)])
    with pytest.raises(Exception):
        hip.call("pad_with_reflection_f32", 4, 12, 2, md, In(np.ones(4, np.float32)), Out(12, "f32"))


FOLD_CASES = [([4, 2], [1, 1], 0, 1, 5, 1), ([2, 2, 2], [3, 1, 1], 1, 2, 3, 1), ([30, 7], [3, 1], 0, 1, 94, 3), ([5, 40, 6, 3], None, 1, 2, 84, 2),
              ([6, 5, 9], None, 1, 0, 20, 3), ([50, 4], None, 0, 1, 4, 0)]


@pytest.mark.parametrize("dt", DTS)
@pytest.mark.parametrize("dims,strides,fd,wd,fold_size,step", FOLD_CASES)
def test_fold(oracle, hip, dims, strides, fd, wd, fold_size, step, dt):
    r = rng(109)
    n = int(np.prod(dims))
    strides = strides or contiguous_strides(dims)
    x = to_storage(r.standard_normal(n + 1).astype(np.float32), dt)
    md = u64(dims, strides, fd, wd, fold_size, step, dims[wd], 1)
    out_n = int(np.prod([fold_size if d == fd else v for d, v in enumerate(dims) if d != wd]))
    (o,), (h,) = both(oracle, hip, f"fold_{dt}", lambda: (n, len(dims), md, In(x), Out(out_n, dt)))
    if dt == "f32" and fd < wd:
        assert same_bits(o, h)          # windows are added in ascending order by both
    else:
        a, b = to_float(o, dt).astype(np.float64), to_float(h, dt).astype(np.float64)
        assert np.max(np.abs(a - b)) <= (1e-5 if dt == "f32" else 6e-2) * max(1.0, np.max(np.abs(a)))


@pytest.mark.parametrize("dt", ["f64"] + INT_DTS)
@pytest.mark.parametrize("dims,strides,fd,wd,fold_size,step", FOLD_CASES)
def test_fold_f64_and_integers(oracle, hip, dims, strides, fd, wd, fold_size, step, dt):
    """Integers add with wrap-around (order-free, so bit-exact); f64 adds its windows in ascending order, which is the
    sequential reference's order when the window dim follows the fold dim (as the tensor layer builds it)."""
    r = rng(113)
    n = int(np.prod(dims))
    strides = strides or contiguous_strides(dims)
    x = r.standard_normal(n + 1) if dt == "f64" else int_values(r, n + 1, dt)
    md = u64(dims, strides, fd, wd, fold_size, step, dims[wd], 1)
    out_n = int(np.prod([fold_size if d == fd else v for d, v in enumerate(dims) if d != wd]))
    (o,), (h,) = both(oracle, hip, f"fold_{dt}", lambda: (n, len(dims), md, In(x), Out(out_n, dt)))
    if dt != "f64" or fd < wd:
        assert same_bits(o, h)
    else:
        assert np.max(np.abs(o - h)) <= 1e-13 * max(1.0, np.max(np.abs(o)))


SOFTMAX_CASES = [([2, 3], 1), ([2, 2, 3], 2), ([2, 3], 0), ([64, 5], 1), ([33, 2048], 1), ([9, 2052], 1), ([3, 40000], 1), ([7, 300], 1),
                 ([6, 50, 130], 1), ([4, 3, 5, 6], 0), ([5, 6], 7), ([10000], 0),
                 # long inner columns: the block-split kernel with narrow and with 16-byte column vectors
                 ([3, 200, 132], 1), ([300, 64, 128], 1), ([1000, 70], 0),
                 # few slabs of long columns: the rows in groups, three launches (a ragged last group, dead lanes, pre > 1)
                 ([2048, 264], 0), ([1100, 520], 0), ([3, 1500, 136], 1), ([4096, 1024], 0),
                 # short rows: 8, 16 or 32 lanes each (a ragged last block, rows that fill a group exactly or in part)
                 ([3001, 32], 1), ([70, 9, 64], 2), ([333, 128], 1), ([101, 256], 1), ([1000, 16], 1), ([517, 8], 1), ([259, 200], 1)]


@pytest.mark.parametrize("dt", DTS)
@pytest.mark.parametrize("shape,dim", SOFTMAX_CASES)
def test_softmax(oracle, hip, shape, dim, dt):
    from scipy.special import softmax as sp_softmax
    r = rng(113)
    n = int(np.prod(shape))
    x = to_storage((r.standard_normal(n) * 3).astype(np.float32), dt)
    md = meta_unary(shape, contiguous_strides(shape), 0)
    (o,), (h,) = both(oracle, hip, f"softmax_{dt}", lambda: (n, len(shape), dim, md, In(x), Out(n, dt)))
    axis = dim if dim < len(shape) else len(shape) - 1
    truth = sp_softmax(to_float(x, dt).astype(np.float64).reshape(shape), axis=axis).ravel()
    got = to_float(h, dt).astype(np.float64)
    if dt == "f32":
        assert np.all(np.abs(got - truth) <= 1e-5 * truth + 1e-30)
        # the reference's own sequential f32 sum drifts from the exact value by about sqrt(D) roundings
        ref_tol = max(1e-5, 4 * np.sqrt(shape[axis]) * 2.0 ** -24)
        assert np.all(np.abs(got - to_float(o, dt)) <= ref_tol * truth + 1e-30)
    else:
        # bf16 rounds x - max and exp like the reference; only the sum differs: the reference's bf16 running sum
        # stalls on long slices, the kernel sums in f32.  Compare with the exact sum of the same rounded terms.
        xf = to_float(x, dt).reshape(shape)
        rnd = lambda v: to_float(to_storage(v, dt), dt)
        t = rnd(xf - xf.max(axis=axis, keepdims=True))
        e = rnd(np.exp(t)).astype(np.float64)
        truth = (e / e.sum(axis=axis, keepdims=True)).ravel()
        assert np.all(np.abs(got - truth) <= 1e-2 * truth + (2.0 ** -24 if dt == "f16" else 1e-30))      # f16 subnormal spacing
        if shape[axis] <= 8:
            # the reference's running sum of D terms in the 16-bit type: at most D - 1 roundings of half a unit in its last place
            ref = to_float(o, dt).astype(np.float64)
            assert np.all(np.abs(got - ref) <= shape[axis] * 2.0 ** -8 * np.maximum(got, ref) + 2.0 ** -24)


@pytest.mark.parametrize("dt", ["bf16", "f16"])
@pytest.mark.parametrize("rows,D", [(2100, 2048), (8100, 520), (520, 8192), (515, 8200), (1030, 4096), (1400, 3000),
                                    (131101, 32), (65603, 64), (32801, 128), (16401, 256), (262201, 16), (524301, 8)])
def test_softmax_16bit_rows_by_table_are_the_arithmetic_kernels_bits(hip, rows, D, dt):
    """A large 16-bit softmax along the last dim takes exp(x - m) from the dtype's table of exp; a call of fewer than 2^22
    elements computes it.  Same rows, same bits - and the known sum of every row."""
    r = rng(127)
    x = to_storage((r.standard_normal(rows * D) * 3).astype(np.float32), dt)
    x[:7] = to_storage(np.array([-np.inf, np.inf, np.nan, 0.0, -0.0, 88.0, -104.0], np.float32), dt)    # row 0: special values
    md = meta_unary([rows, D], [D, 1], 0)
    (big,) = hip.call(f"softmax_{dt}", rows * D, 2, 1, md, In(x), Out(rows * D, dt))
    assert rows * D >= 1 << 22
    part = max(1, ((1 << 22) - 1) // D)
    for r0 in list(range(0, rows, part))[:3] + [rows - min(part, rows)]:
        n = min(part, rows - r0)
        mdp = meta_unary([n, D], [D, 1], 0)
        (small,) = hip.call(f"softmax_{dt}", n * D, 2, 1, mdp, In(x[r0 * D:(r0 + n) * D]), Out(n * D, dt))
        assert same_bits(small, big[r0 * D:(r0 + n) * D]), r0
    sums = to_float(big, dt).reshape(rows, D)[1:].astype(np.float64).sum(1)
    assert np.all(np.abs(sums - 1.0) <= 2e-2)


@pytest.mark.parametrize("dt", ["bf16", "f16"])
@pytest.mark.parametrize("pre,D,post,sub", [(1, 4096, 2048, 512), (2, 1500, 2048, 512), (1, 8190, 1024, 256)])
def test_softmax_16bit_columns_by_table_are_the_arithmetic_kernels_bits(hip, pre, D, post, sub, dt):
    """Long columns in groups of rows: a 16-bit call of 2^22 elements or more takes exp(x - m) from the table.  The same
    columns as a call of fewer elements (same D and as many groups, so the same order of additions) are computed: same bits."""
    r = rng(139)
    n = pre * D * post
    x = to_storage((r.standard_normal(n) * 3).astype(np.float32), dt).reshape(pre, D, post)
    x[0, :7, 3] = to_storage(np.array([-np.inf, np.inf, np.nan, 0.0, -0.0, 88.0, -104.0], np.float32), dt)
    x[0, :, 5] = to_storage(np.full(D, -np.inf, np.float32), dt)
    assert n >= 1 << 22 and pre * D * sub < 1 << 22
    (big,) = hip.call(f"softmax_{dt}", n, 3, 1, meta_unary([pre, D, post], contiguous_strides([pre, D, post]), 0), In(x.ravel()), Out(n, dt))
    big = big.reshape(pre, D, post)
    for c0 in (0, post - sub):
        part = np.ascontiguousarray(x[:, :, c0:c0 + sub])
        (small,) = hip.call(f"softmax_{dt}", part.size, 3, 1, meta_unary([pre, D, sub], contiguous_strides([pre, D, sub]), 0), In(part.ravel()), Out(part.size, dt))
        assert same_bits(small, np.ascontiguousarray(big[:, :, c0:c0 + sub]).ravel()), c0
    sums = to_float(big.ravel(), dt).reshape(pre, D, post).astype(np.float64).sum(1)[:, 8:]
    assert np.all(np.abs(sums - 1.0) <= 2e-2)


@pytest.mark.parametrize("dt", ["f32", "bf16"])
@pytest.mark.parametrize("dims,perm", [([520, 640], [1, 0]), ([300, 6, 200], [0, 2, 1]), ([1, 40, 72, 128], [0, 3, 1, 2])])
def test_softmax_large_strided_input_is_the_softmax_of_its_logical_copy(oracle, hip, dims, perm, dt):
    """From 2^18 elements, a strided input with at most one leading dim of more than one element is copied into logical
    order and takes the contiguous kernels; with more leading dims it keeps the reference's own walk.  Against the
    oracle, which restates that walk."""
    lay = LY.permuted(dims, perm)
    r = rng(193)
    st = to_storage((r.standard_normal(lay["size"]) * 2).astype(np.float32), dt)
    n = int(np.prod(dims))
    assert n >= 1 << 18
    md = meta_unary(lay["dims"], lay["strides"], 0)
    logical = np.ascontiguousarray(LY.gather(st, lay)).ravel()
    mdc = meta_unary(dims, contiguous_strides(dims), 0)
    for dim in range(len(dims)):
        (h,) = hip.call(f"softmax_{dt}", n, len(dims), dim, md, In(st), Out(n, dt))
        if sum(d > 1 for d in dims[:dim]) <= 1:
            (hc,) = hip.call(f"softmax_{dt}", n, len(dims), dim, mdc, In(logical), Out(n, dt))
            assert same_bits(h, hc), dim
        if dt == "f32":         # (the reference's bf16 running sum stalls on slices this long: no bar to hold bf16 to)
            (o,) = oracle.call(f"softmax_{dt}", n, len(dims), dim, md, In(st), Out(n, dt))
            of, hf = o.astype(np.float64), h.astype(np.float64)
            assert np.all(np.abs(of - hf) <= 2e-5 * of + 1e-30), dim
        sums = to_float(h, dt).astype(np.float64).reshape(dims).sum(axis=dim)
        assert np.all(np.abs(sums - 1.0) <= 3e-2), dim


def test_softmax_strided_and_special_values(oracle, hip):
    r = rng(127)
    lay = LY.permuted([6, 9], [1, 0], off=2)
    st = np.concatenate([np.zeros(2), r.standard_normal(54)]).astype(np.float32)
    for dim in (0, 1):
        md = meta_unary([6, 9], lay["strides"], lay["off"])
        (o,), (h,) = both(oracle, hip, "softmax_f32", lambda: (54, 2, dim, md, In(st), Out(54, "f32")))
        assert np.allclose(o, h, rtol=1e-5, atol=0)
    # three leading dims, permuted: the reference's own (dim 0 fastest) walk of the leading dims
    lay = LY.permuted([3, 4, 5, 6], [2, 0, 3, 1])
    st = r.standard_normal(360).astype(np.float32)
    md = meta_unary([3, 4, 5, 6], lay["strides"], 0)
    for dim in (1, 2, 3):
        (o,), (h,) = both(oracle, hip, "softmax_f32", lambda: (360, 4, dim, md, In(st), Out(360, "f32")))
        assert np.allclose(o, h, rtol=1e-5, atol=0)
    v = np.array([[0.0, -np.inf, 1.0], [-np.inf, -np.inf, -np.inf], [np.nan, 1.0, 2.0], [np.inf, 1.0, 2.0]], dtype=np.float32)
    (o,), (h,) = both(oracle, hip, "softmax_f32", lambda: (12, 2, 1, meta_unary([4, 3], [3, 1], 0), In(v.ravel()), Out(12, "f32")))
    assert np.array_equal(np.isnan(o), np.isnan(h))
    assert np.allclose(o[~np.isnan(o)], h[~np.isnan(o)], rtol=1e-6)


@pytest.mark.parametrize("shape,dim", SOFTMAX_CASES)
def test_softmax_f64(oracle, hip, shape, dim):
    """f64 (softmax.rs:26-31 of the CUDA crate lists it): against scipy's softmax in float64 and against the oracle;
    the only differences are the device library's exp (within 1 ulp of the host's) and the tree order of a long row's sum."""
    from scipy.special import softmax as sp_softmax
    r = rng(131)
    n = int(np.prod(shape))
    x = r.standard_normal(n) * 3
    md = meta_unary(shape, contiguous_strides(shape), 0)
    (o,), (h,) = both(oracle, hip, "softmax_f64", lambda: (n, len(shape), dim, md, In(x), Out(n, "f64")))
    axis = dim if dim < len(shape) else len(shape) - 1
    truth = sp_softmax(x.reshape(shape), axis=axis).ravel()
    assert np.all(np.abs(h - truth) <= 1e-13 * truth + 1e-300)
    assert np.all(np.abs(h - o) <= 1e-13 * truth + 1e-300)


def test_softmax_f64_large_strided_input(oracle, hip):
    """f64 as f32: a large strided input goes through its logical-order copy; against the oracle's walk."""
    r = rng(197)
    for dims, perm in (([520, 640], [1, 0]), ([300, 6, 200], [0, 2, 1])):
        lay = LY.permuted(dims, perm)
        st = r.standard_normal(lay["size"]) * 2
        n = int(np.prod(dims))
        md = meta_unary(lay["dims"], lay["strides"], 0)
        for dim in range(len(dims)):
            (o,), (h,) = both(oracle, hip, "softmax_f64", lambda: (n, len(dims), dim, md, In(st), Out(n, "f64")))
            assert np.all(np.abs(h - o) <= 1e-13 * o + 1e-300), dim


def test_softmax_f64_strided_and_special_values(oracle, hip):
    r = rng(137)
    lay = LY.permuted([3, 4, 5, 6], [2, 0, 3, 1], off=3)
    st = np.concatenate([np.zeros(3), r.standard_normal(360)])
    md = meta_unary([3, 4, 5, 6], lay["strides"], lay["off"])
    for dim in (0, 1, 2, 3):
        (o,), (h,) = both(oracle, hip, "softmax_f64", lambda: (360, 4, dim, md, In(st), Out(360, "f64")))
        assert np.allclose(o, h, rtol=1e-13, atol=0)
    v = np.array([[0.0, -np.inf, 1.0], [-np.inf, -np.inf, -np.inf], [np.nan, 1.0, 2.0], [np.inf, 1.0, 2.0]])
    (o,), (h,) = both(oracle, hip, "softmax_f64", lambda: (12, 2, 1, meta_unary([4, 3], [3, 1], 0), In(v.ravel()), Out(12, "f64")))
    assert np.array_equal(np.isnan(o), np.isnan(h))
    assert np.allclose(o[~np.isnan(o)], h[~np.isnan(o)], rtol=1e-13)


# ---------------------------------------------------------------------------------------------------
# index ops: bit-exact, same order of the adds as the reference's host loops
# ---------------------------------------------------------------------------------------------------
INDEX_SHAPES = [([5, 7], 0), ([5, 7], 1), ([3, 4, 6], 1), ([2, 3, 4, 5], 2), ([300, 64], 0), ([64, 300], 1), ([17], 0)]


@pytest.mark.parametrize("dt", DTS)
@pytest.mark.parametrize("it", ["i32", "i64"])
@pytest.mark.parametrize("shape,dim", INDEX_SHAPES)
def test_index_select_and_index_add(oracle, hip, shape, dim, it, dt):
    r = rng(149)
    ity = np.int32 if it == "i32" else np.int64
    n = int(np.prod(shape))
    x = to_storage(np.concatenate([[9.0], r.standard_normal(n)]).astype(np.float32), dt)
    n_idx = 2 * shape[dim] + 3                                          # plenty of repeats
    idx = np.concatenate([[0, 0], r.integers(0, shape[dim], n_idx)]).astype(ity)      # offset 2
    out_shape = list(shape)
    out_shape[dim] = n_idx
    n_out = int(np.prod(out_shape))
    (o,), (h,) = both(oracle, hip, f"index_select_{dt}_{it}",
                      lambda: (len(shape), dim, layout(shape, off=1), n_idx, 1, 2, In(idx), In(x), Out(n_out, dt)))
    assert same_bits(o, h)
    src = to_storage(r.standard_normal(n_out + 1).astype(np.float32), dt)
    (o,), (h,) = both(oracle, hip, f"index_add_{dt}_{it}",
                      lambda: (len(shape), dim, layout(shape, off=1), layout(out_shape, off=1), n_idx, 1, 2, In(idx), In(src), InOut(x.copy())))
    assert same_bits(o, h)


@pytest.mark.parametrize("dt", DTS)
@pytest.mark.parametrize("shape,dim,idx_len", [([5, 7], 1, 3), ([5, 7], 0, 8), ([3, 4, 6], 2, 6), ([2, 3, 4], 1, 1), ([128, 1000], 1, 1), ([200, 50], 0, 500)])
def test_gather_and_scatter_add(oracle, hip, shape, dim, idx_len, dt):
    r = rng(151)
    n = int(np.prod(shape))
    x = to_storage(r.standard_normal(n).astype(np.float32), dt)
    ishape = list(shape)
    ishape[dim] = idx_len
    index = r.integers(-shape[dim], shape[dim], ishape).astype(np.int64).ravel()
    m = index.size
    (o,), (h,) = both(oracle, hip, f"gather_{dt}_i64", lambda: (len(shape), dim, layout(shape), layout(ishape), In(index), In(x), Out(m, dt)))
    assert same_bits(o, h)
    src = to_storage(r.standard_normal(m).astype(np.float32), dt)
    (o,), (h,) = both(oracle, hip, f"scatter_add_{dt}_i64",
                      lambda: (len(shape), dim, layout(shape), layout(ishape), layout(ishape), In(index), In(src), InOut(x.copy())))
    assert same_bits(o, h)


@pytest.mark.parametrize("dt", DTS)
@pytest.mark.parametrize("shape,dim,n_idx", [([50, 64], 0, 3000), ([7, 40, 8], 1, 1000), ([33, 500], 1, 2048), ([3, 40, 2048], 1, 700), ([6, 50, 6], 1, 900)])
def test_index_add_with_many_indices(oracle, hip, shape, dim, n_idx, dt):
    # enough indices for the sorted path; some out of range, which both sides skip or stop at — so keep them valid here
    r = rng(167)
    n = int(np.prod(shape))
    x = to_storage(r.standard_normal(n).astype(np.float32), dt)
    idx = r.integers(0, shape[dim], n_idx).astype(np.int32)
    src_shape = list(shape)
    src_shape[dim] = n_idx
    src = to_storage(r.standard_normal(int(np.prod(src_shape))).astype(np.float32), dt)
    (o,), (h,) = both(oracle, hip, f"index_add_{dt}_i32",
                      lambda: (len(shape), dim, layout(shape), layout(src_shape), n_idx, 1, 0, In(idx), In(src), InOut(x.copy())))
    assert same_bits(o, h)


@pytest.mark.parametrize("shape,dim,n_idx,spread", [([70000, 2], 0, 200000, 70000), ([300000], 0, 50000, 300000), ([2, 66000, 1], 1, 9000, 17),
                                                    ([5000, 4], 0, 131072, 5000), ([1 << 17, 1], 0, 4097, 1 << 17)])
def test_index_add_sorts_many_indices_over_many_destinations(oracle, hip, shape, dim, n_idx, spread):
    """Destinations of up to 19 bits (three passes of the radix sort), index counts that make several blocks of it and
    one that ends a block with a single element, many equal destinations (`spread` 17): the f32 sums are added in the
    reference's order, so the bits are the oracle's."""
    r = rng(171 + n_idx)
    n = int(np.prod(shape))
    x = r.standard_normal(n).astype(np.float32)
    idx = r.integers(0, spread, n_idx).astype(np.int32)
    src_shape = list(shape)
    src_shape[dim] = n_idx
    src = r.standard_normal(int(np.prod(src_shape))).astype(np.float32)
    (o,), (h,) = both(oracle, hip, "index_add_f32_i32",
                      lambda: (len(shape), dim, layout(shape), layout(src_shape), n_idx, 1, 0, In(idx), In(src), InOut(x.copy())))
    assert same_bits(o, h)


@pytest.mark.parametrize("dt", ["f64", "bool"] + INT_DTS)
@pytest.mark.parametrize("it", ["i32", "i64"])
def test_index_ops_wide_dtypes(oracle, hip, dt, it):
    """Every storage dtype has the index ops (the reference moves Scalars).  Copies are bit-exact; the in-place adds are
    add_at_index's: f64 in order, `||` for bool, wrap-around for the integers (full-range values, so they do wrap)."""
    r = rng(179)
    IT = NP[it]
    shape, dim = [6, 40, 9], 1
    n = int(np.prod(shape))
    x = wide_values(r, n + 2, dt)
    L = layout(shape, off=2)
    # index_select with few and with many indices; gather with negative indices
    for n_idx in (5, 700):
        idx = r.integers(0, shape[dim], n_idx).astype(IT)
        out_shape = [6, n_idx, 9]
        (o,), (h,) = both(oracle, hip, f"index_select_{dt}_{it}", lambda: (3, dim, L, n_idx, 1, 0, In(idx), In(x), Out(int(np.prod(out_shape)), dt)))
        assert same_bits(o, h)
        assert same_bits(h.reshape(out_shape), np.take(x[2:].reshape(shape), idx, axis=dim))
        src = wide_values(r, int(np.prod(out_shape)), dt)
        (o,), (h,) = both(oracle, hip, f"index_add_{dt}_{it}", lambda: (3, dim, L, layout(out_shape), n_idx, 1, 0, In(idx), In(src), InOut(x.copy())))
        assert same_bits(o, h), ("index_add", n_idx)
    ishape = [6, 17, 9]
    index = r.integers(-shape[dim], shape[dim], ishape).astype(IT).ravel()
    (o,), (h,) = both(oracle, hip, f"gather_{dt}_{it}", lambda: (3, dim, L, layout(ishape), In(index), In(x), Out(index.size, dt)))
    assert same_bits(o, h)
    assert same_bits(h.reshape(ishape), np.take_along_axis(x[2:].reshape(shape), index.reshape(ishape).astype(np.int64) % shape[dim], axis=dim))
    src = wide_values(r, index.size, dt)
    (o,), (h,) = both(oracle, hip, f"scatter_add_{dt}_{it}", lambda: (3, dim, L, layout(ishape), layout(ishape), In(index), In(src), InOut(x.copy())))
    assert same_bits(o, h)
    # index_put_: a [40, 9] source into self[4]
    srcp = wide_values(r, 40 * 9, dt)
    (o,), (h,) = both(oracle, hip, f"index_put_{dt}", lambda: (3, L, 1, u64(4), 2, layout([40, 9]), In(srcp), InOut(x.copy())))
    assert same_bits(o, h)
    want = x.copy()
    want[2:].reshape(shape)[4] = srcp.reshape(40, 9)
    assert same_bits(h, want)


def test_index_ops_on_permuted_tensors(oracle, hip):
    r = rng(157)
    lay = LY.permuted([6, 9, 4], [2, 0, 1], off=3)
    st = np.concatenate([np.zeros(3), r.standard_normal(216)]).astype(np.float32)
    idx = r.integers(0, 9, 5).astype(np.int32)
    L = layout([6, 9, 4], lay["strides"], lay["off"])
    (o,), (h,) = both(oracle, hip, "index_select_f32_i32", lambda: (3, 1, L, 5, 1, 0, In(idx), In(st), Out(6 * 5 * 4, "f32")))
    assert same_bits(o, h)
    src = r.standard_normal(6 * 5 * 4).astype(np.float32)
    (o,), (h,) = both(oracle, hip, "index_add_f32_i32", lambda: (3, 1, L, layout([6, 5, 4]), 5, 1, 0, In(idx), In(src), InOut(st.copy())))
    assert same_bits(o, h)
    index = r.integers(0, 4, (6, 9, 2)).astype(np.int32).ravel()
    (o,), (h,) = both(oracle, hip, "gather_f32_i32", lambda: (3, 2, L, layout([6, 9, 2]), In(index), In(st), Out(index.size, "f32")))
    assert same_bits(o, h)


def test_bincount(oracle, hip):
    r = rng(163)
    for it, ity in (("i32", np.int32), ("i64", np.int64)):
        v = r.integers(0, 1000, 200000).astype(ity)
        (o,), (h,) = both(oracle, hip, f"bincount_{it}", lambda: (v.size, 1, 0, In(v), 1024, Out(1024, it)))
        assert np.array_equal(o, h) and int(h.sum()) == v.size
        for dt in DTS:
            w = to_storage(r.standard_normal(5000).astype(np.float32), dt)
            (o,), (h,) = both(oracle, hip, f"bincount_weighted_{dt}_{it}", lambda: (5000, 1, 0, In(v[:5000]), 1, 0, In(w), 1024, Out(1024, dt)))
            assert same_bits(o, h)


@pytest.mark.parametrize("dt", DTS)
@pytest.mark.parametrize("shape,n_fixed", [([6], 0), ([40, 50], 1), ([3, 40, 50], 1), ([3, 4, 5], 2), ([2, 3, 4, 5], 3), ([64, 1024], 1), ([8, 256, 256], 1)])
def test_index_put(oracle, hip, shape, n_fixed, dt):
    """Sub-tensor assignment, contiguous and through permuted views of both tensors, and the single-element and flat-copy
    forms; every byte of self equals the oracle's, written or not."""
    r = rng(163)
    n = int(np.prod(shape))
    x = to_storage(r.standard_normal(n + 2).astype(np.float32), dt)
    fixed = [int(r.integers(0, shape[d])) for d in range(n_fixed)]
    rest = shape[n_fixed:]
    m = int(np.prod(rest))
    src = to_storage(r.standard_normal(m + 3).astype(np.float32), dt)
    idx = np.array(fixed + [0], dtype=np.uint64)
    (o,), (h,) = both(oracle, hip, f"index_put_{dt}", lambda: (len(shape), layout(shape, off=2), n_fixed, idx, len(rest), layout(rest, off=3), In(src), InOut(x.copy())))
    assert same_bits(o, h) and not same_bits(h, x)
    if len(rest) >= 2:
        st = contiguous_strides(shape[:-2] + [shape[-1], shape[-2]])
        st[-1], st[-2] = st[-2], st[-1]
        sst = contiguous_strides(rest[:-2] + [rest[-1], rest[-2]])
        sst[-1], sst[-2] = sst[-2], sst[-1]
        (o,), (h,) = both(oracle, hip, f"index_put_{dt}", lambda: (len(shape), layout(shape, st, off=2), n_fixed, idx, len(rest), layout(rest, sst, off=3), In(src), InOut(x.copy())))
        assert same_bits(o, h) and not same_bits(h, x)
    full = np.array([int(r.integers(0, s)) for s in shape], dtype=np.uint64)
    (o,), (h,) = both(oracle, hip, f"index_put_{dt}", lambda: (len(shape), layout(shape, off=2), len(shape), full, 0, np.array([1], dtype=np.uint64), In(src), InOut(x.copy())))
    assert same_bits(o, h)
    if len(shape) == 1:
        (o,), (h,) = both(oracle, hip, f"index_put_{dt}", lambda: (1, layout(shape, off=2), 1, np.array([2], dtype=np.uint64), 1, layout([2], [2], off=1), In(src), InOut(x.copy())))
        assert same_bits(o, h) and not same_bits(h, x)


def test_index_put_errors_write_nothing(hip):
    import maidenx_amd.lib as L
    L.check()
    x = np.arange(10, dtype=np.float32)
    cases = [
        ("does not fit", (1, layout([10]), 1, np.array([8], dtype=np.uint64), 1, layout([3]))),
        ("more indices than dims", (1, layout([10]), 2, np.array([1, 1], dtype=np.uint64), 0, layout([]))),
        ("out of bounds", (2, layout([2, 5]), 1, np.array([2], dtype=np.uint64), 1, layout([5]))),
        ("shape differs", (2, layout([2, 5]), 1, np.array([1], dtype=np.uint64), 1, layout([4]))),
        ("1-d destination", (2, layout([2, 5]), 2, np.array([1, 1], dtype=np.uint64), 1, layout([2]))),
    ]
    for what, args in cases:
        buf = InOut(x.copy())
        with pytest.raises(L.HipError, match=what):
            hip.call("index_put_f32", *args, In(np.ones(5, np.float32)), buf)
    (h,) = hip.call("index_put_f32", 1, layout([10]), 1, np.array([7], dtype=np.uint64), 1, layout([3]), In(np.ones(5, np.float32)), InOut(x.copy()))
    assert h.tolist() == [0, 1, 2, 3, 4, 5, 6, 1, 1, 1]


def test_index_out_of_bounds_is_reported(hip):
    import maidenx_amd.lib as L
    L.check()
    bad = np.array([0, 3, 1], dtype=np.int32)
    with pytest.raises(L.HipError, match="index out of bounds"):
        hip.call("index_select_f32_i32", 1, 0, layout([3]), 3, 1, 0, In(bad), In(np.arange(3, dtype=np.float32)), Out(3, "f32"))
    # the flag was cleared with the report: a valid call afterwards is clean
    (h,) = hip.call("index_select_f32_i32", 1, 0, layout([3]), 3, 1, 0, In(np.array([2, 1, 0], dtype=np.int32)),
                    In(np.arange(3, dtype=np.float32)), Out(3, "f32"))
    assert h.tolist() == [2.0, 1.0, 0.0]
    with pytest.raises(L.HipError, match="index out of bounds"):
        hip.call("gather_f32_i32", 1, 0, layout([3]), layout([2]), In(np.array([-4, 0], dtype=np.int32)), In(np.arange(3, dtype=np.float32)), Out(2, "f32"))


def test_gather_refuses_an_index_larger_than_the_input_off_dim(hip):
    """indexing.rs:331-340: the index tensor must have the input's extent in every dim but `dim`.  The host refuses the
    call before anything is queued, so nothing is launched and the output keeps its poison."""
    import maidenx_amd.lib as L
    L.check()
    x = np.arange(12, dtype=np.float32)
    index = np.zeros(5 * 2, dtype=np.int32)
    out = Out(10, "f32")
    with pytest.raises(L.HipError, match="index and input shapes differ"):
        hip.call("gather_f32_i32", 2, 1, layout([3, 4]), layout([5, 2]), In(index), In(x), out)
    assert (out.arr.view(np.uint8) == 0xCD).all()
    # the same extent off `dim` is accepted, whatever the extent along `dim`
    (h,) = hip.call("gather_f32_i32", 2, 1, layout([3, 4]), layout([3, 6]), In(np.tile(np.array([3, 0, 1, 2, 3, 0], np.int32), 3)), In(x), Out(18, "f32"))
    assert h.reshape(3, 6)[1].tolist() == [7.0, 4.0, 5.0, 6.0, 7.0, 4.0]


@pytest.mark.parametrize("dt", DTS)
@pytest.mark.parametrize("n", [1, 7, 1000, 4099, 1 << 16])
def test_fused_adam_step_equals_the_fourteen_ops(oracle, hip, n, dt):
    """adam.rs:46-86 as the op sequence it is, on the oracle and on the GPU, against one hip_adam_step call: the same
    bits in param, m and v, over several steps with the reference's beta^(t+1) bias terms."""
    r = rng(173)
    st = lambda a: to_storage(np.asarray(a, dtype=np.float32), dt)
    p0 = st(r.standard_normal(n))
    m0, v0 = st(np.zeros(n)), st(np.zeros(n))
    lr, b1, b2, eps = 0.001, 0.9, 0.999, 1e-8
    md1 = meta_unary([n], [1])
    md2 = meta_binary([n], [1], [1])

    def chain(be, p, g, m, v, sc):
        un = lambda op, x: be.call(f"{op}_{dt}", n, 1, md1, In(x), Out(n, dt))[0]
        unc = lambda op, x, c: be.call(f"{op}_{dt}", n, 1, md1, In(x), const_arg(c, dt), Out(n, dt))[0]
        bi = lambda op, a, b: be.call(f"{op}_{dt}", n, 1, md2, In(a), In(b), Out(n, dt))[0]
        m = bi("add", unc("mul_scalar", m, sc[0]), unc("mul_scalar", g, sc[1]))
        v = bi("add", unc("mul_scalar", v, sc[2]), unc("mul_scalar", un("square", g), sc[3]))
        step = bi("div", unc("div_scalar", m, sc[4]), unc("add_scalar", un("sqrt", unc("div_scalar", v, sc[5])), sc[6]))
        (p,) = be.call(f"sub_inplace_{dt}", n, 1, md2, InOut(p), In(unc("mul_scalar", step, sc[7])))
        return p, m, v

    po, mo, vo = p0.copy(), m0.copy(), v0.copy()
    ph, mh, vh = p0.copy(), m0.copy(), v0.copy()
    pf, mf, vf = p0.copy(), m0.copy(), v0.copy()
    for t in range(1, 4):
        g = st(r.standard_normal(n) * (0.0 if t == 2 and n == 7 else 1.0))          # a zero gradient: 0 / (0 + eps)
        b1t, b2t = b1 ** (t + 1), b2 ** (t + 1)                                        # adam.rs:56-61 multiplies t times from beta
        sc = [b1, 1 - b1, b2, 1 - b2, 1 - b1t, 1 - b2t, eps, lr * np.sqrt(1 - b2t) / (1 - b1t)]
        po, mo, vo = chain(oracle, po, g, mo, vo, sc)
        ph, mh, vh = chain(hip, ph, g, mh, vh, sc)
        pf, mf, vf = hip.call(f"adam_step_{dt}", n, InOut(pf), In(g), InOut(mf), InOut(vf), *[const_arg(c, dt) for c in sc])
        for a, b, c, what in ((po, ph, pf, "param"), (mo, mh, mf, "m"), (vo, vh, vf, "v")):
            assert same_bits(a, b), (what, t, "op by op: oracle vs GPU")
            assert same_bits(b, c), (what, t, "fused vs op by op")
    assert not same_bits(mf, m0) and not same_bits(vf, v0)
    if dt == "f32":
        assert not same_bits(pf, p0)          # (a 16-bit parameter near 1 does not move by 0.001)


@pytest.mark.parametrize("n", [1, 3, 7, 1000, 10000, 65536, 65540, (1 << 20) + 5, 32 * 64 * 56 * 56])
def test_fused_mse_loss_equals_the_op_sequence(oracle, hip, n):
    """losses/mse.rs:21-29 as the ops it is - sub, pow(2), a sum of everything, div_scalar - and their backward
    (div_scalar, the broadcast, mul_scalar(2), mul, sub's `0 + g` and neg) against hip_mse_loss_f32 and
    hip_mse_loss_backward_f32: both gradients bit for bit (on the GPU's ops and, where it finishes in a moment, the
    oracle's), the loss within 1e-5 of the sum of the terms' magnitudes divided by n (f64)."""
    r = rng(181)
    pred = r.standard_normal(n).astype(np.float32)
    target = r.standard_normal(n).astype(np.float32)
    target[::5] = pred[::5]                                   # exact zeros among the differences (+0 and, negated, -0)
    g = np.array([0.37], np.float32)                          # the loss's incoming gradient (backward() seeds it with 1)
    md1, md2 = meta_unary([n], [1]), meta_binary([n], [1], [1])
    mdb = meta_binary([n], [0], [1])                          # the scalar broadcast over [n]

    def chain(be):
        diff = be.call("sub_f32", n, 1, md2, In(pred), In(target), Out(n, "f32"))[0]
        g1 = be.call("div_scalar_f32", 1, 1, meta_unary([1], [1]), In(g), const_arg(float(n), "f32"), Out(1, "f32"))[0]
        g2 = be.call("mul_scalar_f32", n, 1, meta_unary([n], [0]), In(g1), const_arg(2.0, "f32"), Out(n, "f32"))[0]
        g3 = be.call("mul_f32", n, 1, md2, In(g2), In(diff), Out(n, "f32"))[0]
        gp = be.call("sum_to_shape_f32", n, 1, meta_sum_to_shape([n], [1], [n]), In(g3), Out(n, "f32"))[0]
        neg = be.call("neg_f32", n, 1, md1, In(g3), Out(n, "f32"))[0]
        gt = be.call("sum_to_shape_f32", n, 1, meta_sum_to_shape([n], [1], [n]), In(neg), Out(n, "f32"))[0]
        return diff, gp, gt
    diff, gp, gt = chain(hip)
    (loss,) = hip.call("mse_loss_f32", n, In(pred), In(target), Out(1, "f32"))
    fp, ft = hip.call("mse_loss_backward_f32", n, In(pred), In(target), In(g), Out(n, "f32"), Out(n, "f32"))
    assert same_bits(fp, gp) and same_bits(ft, gt)
    (fp2,) = hip.call("mse_loss_backward_f32", n, In(pred), In(target), In(g), Out(n, "f32"), None)
    (ft2,) = hip.call("mse_loss_backward_f32", n, In(pred), In(target), In(g), None, Out(n, "f32"))
    assert same_bits(fp2, gp) and same_bits(ft2, gt)
    # no grad_loss: the seed of backward(), a gradient of exactly 1
    (fp1,) = hip.call("mse_loss_backward_f32", n, In(pred), In(target), None, Out(n, "f32"), None)
    (fpo,) = hip.call("mse_loss_backward_f32", n, In(pred), In(target), In(np.array([1.0], np.float32)), Out(n, "f32"), None)
    assert same_bits(fp1, fpo)
    if n <= (1 << 20) + 5:
        _, op, ot = chain(oracle)
        assert same_bits(fp, op) and same_bits(ft, ot)
    d64 = pred.astype(np.float64) - target.astype(np.float64)
    want = float((d64 * d64).sum() / n)
    assert abs(float(loss[0]) - want) <= 1e-5 * want + 1e-30
    # the unfused loss of the GPU's own ops, for comparison (another order of the same sum)
    sq = hip.call("square_f32", n, 1, md1, In(diff), Out(n, "f32"))[0]
    (s,) = hip.call("sum_f32", n, 1, 1, meta_reduce([n], [1], 0), In(sq), Out(1, "f32"))
    assert abs(float(loss[0]) - float(s[0]) / n) <= 2e-5 * want + 1e-30


@pytest.mark.parametrize("n", [1, 3, 1000, 4099, 1 << 16, 64 * 64 * 9])
def test_fused_sgd_step_equals_mul_scalar_and_sub_inplace(oracle, hip, n):
    """optimizers/sgd.rs:17-27: param.sub_(grad.mul_scalar(lr)), against one hip_sgd_step_f32 call."""
    r = rng(182)
    p0 = r.standard_normal(n).astype(np.float32)
    g = (r.standard_normal(n) * 10).astype(np.float32)
    md1, md2 = meta_unary([n], [1]), meta_binary([n], [1], [1])
    outs = []
    for be in (oracle, hip):
        step = be.call("mul_scalar_f32", n, 1, md1, In(g), const_arg(0.01, "f32"), Out(n, "f32"))[0]
        outs.append(be.call("sub_inplace_f32", n, 1, md2, InOut(p0.copy()), In(step))[0])
    (fused,) = hip.call("sgd_step_f32", n, InOut(p0.copy()), In(g), const_arg(0.01, "f32"))
    assert same_bits(outs[0], outs[1]) and same_bits(fused, outs[1]) and not same_bits(fused, p0)


@pytest.mark.parametrize("dt", DTS)
def test_empty_inputs_are_no_ops(hip, dt):
    """Zero elements anywhere: nothing is launched, nothing is written, no error is recorded."""
    import maidenx_amd.lib as L
    L.check()
    e = np.zeros(0, dtype=np.float32 if dt == "f32" else np.uint16)
    poison = lambda n=4: Out(n, dt)
    keep = poison().arr.copy()
    for call in (
        lambda: hip.call(f"add_{dt}", 0, 2, meta_binary([0, 5], [5, 1], [5, 1]), In(e), In(e), poison()),
        lambda: hip.call(f"add_inplace_{dt}", 0, 1, meta_binary([0], [1], [1]), InOut(poison().arr), In(e)),
        lambda: hip.call(f"exp_{dt}", 0, 1, meta_unary([0], [1]), In(e), poison()),
        lambda: hip.call(f"mul_scalar_{dt}", 0, 1, meta_unary([0], [1]), In(e), const_arg(2.0, dt), poison()),
        lambda: hip.call(f"sum_{dt}", 0, 2, 1, meta_reduce([0, 4], [4, 1], 1), In(e), poison()),
        lambda: hip.call(f"sum_to_shape_{dt}", 0, 2, meta_sum_to_shape([0, 4], [4, 1], [0, 1]), In(e), poison()),
        lambda: hip.call(f"matmul_{dt}", 0, meta_matmul([0, 3], [0, 2], [2, 3], [2, 1], [3, 1]), In(e), In(to_storage(np.ones(6, np.float32), dt)), poison()),
        lambda: hip.call(f"pad_with_constant_{dt}", 0, 0, 2, meta_pad([0, 3], [3, 1], 0, [0, 5], [(0, 0), (1, 1)]), In(e), poison(), const_arg(1.0, dt)),
        lambda: hip.call(f"pad_with_replication_{dt}", 0, 0, 2, meta_pad([0, 3], [3, 1], 0, [0, 5], [(0, 0), (1, 1)]), In(e), poison()),
        lambda: hip.call(f"conv2d_im2col_{dt}", 0, meta_conv(0, 3, 4, 4, 3, 3, 4, 4, 1, 1, 1, 1), In(e), poison()),
        lambda: hip.call(f"conv2d_col2im_{dt}", 0, meta_conv(0, 3, 4, 4, 3, 3, 4, 4, 1, 1, 1, 1), In(e), poison()),
        lambda: hip.call(f"softmax_{dt}", 0, 2, 1, meta_unary([0, 4], [4, 1]), In(e), poison()),
        lambda: hip.call(f"index_select_{dt}_i32", 2, 0, layout([3, 0]), 2, 1, 0, In(np.array([0, 1], dtype=np.int32)), In(e), poison()),
        lambda: hip.call(f"gather_{dt}_i32", 1, 0, layout([3]), layout([0]), In(np.zeros(0, np.int32)), In(to_storage(np.ones(3, np.float32), dt)), poison()),
        lambda: hip.call(f"fill_{dt}", 0, poison(), const_arg(1.0, dt)),
        lambda: hip.call(f"copy_strided_{dt}", 0, 1, meta_unary([0], [1]), In(e), poison()),
    ):
        (out,) = call()[-1:]
        assert same_bits(out[:4], keep), "an empty call wrote to its output"
    L.check()


# ---------------------------------------------------------------------------------------------------
# fill / cast / strided copy (device-side helpers without a reference symbol)
# ---------------------------------------------------------------------------------------------------
def test_fill_cast_copy(hip):
    (f,) = hip.call("fill_f32", 1001, Out(1001, "f32"), 2.5)
    assert np.all(f == 2.5)
    (f,) = hip.call("fill_bf16", 77, Out(77, "bf16"), const_arg(1.0, "bf16"))
    assert np.all(f == 0x3F80)
    r = rng(71)
    x = r.standard_normal(5000).astype(np.float32)
    (b,) = hip.call("cast_f32_bf16", 5000, In(x), Out(5000, "bf16"))
    assert np.array_equal(b, f32_to_bf16(x))
    (back,) = hip.call("cast_bf16_f32", 5000, In(b), Out(5000, "f32"))
    assert np.array_equal(back, bf16_to_f32(b))
    # bf16 from every kind of f32 (random bit patterns: all exponents, subnormals, infinities, NaNs) against the closed form
    pat = r.integers(0, 1 << 32, 1 << 22, dtype=np.uint64).astype(np.uint32).view(np.float32)
    (pb,) = hip.call("cast_f32_bf16", pat.size, In(pat), Out(pat.size, "bf16"))
    want_b = f32_to_bf16(pat)
    isn = np.isnan(pat)
    assert np.array_equal(pb[~isn], want_b[~isn])
    assert np.all(np.isnan(bf16_to_f32(pb[isn])))
    # f16: every bit pattern to f32 and back, and f32 values across the f16 range (subnormals, overflow, ties) against numpy
    hb = np.arange(1 << 16, dtype=np.uint16)
    (hf,) = hip.call("cast_f16_f32", hb.size, In(hb), Out(hb.size, "f32"))
    want = hb.view(np.float16).astype(np.float32)
    assert np.array_equal(np.isnan(hf), np.isnan(want)) and np.array_equal(hf[~np.isnan(want)], want[~np.isnan(want)])
    wide = (r.standard_normal(200000) * np.exp(r.uniform(-20, 12, 200000))).astype(np.float32)
    (hh,) = hip.call("cast_f32_f16", wide.size, In(wide), Out(wide.size, "f16"))
    with np.errstate(over="ignore"):
        assert np.array_equal(hh, wide.astype(np.float16).view(np.uint16))
    (f,) = hip.call("fill_f16", 77, Out(77, "f16"), const_arg(1.0, "f16"))
    assert np.all(f == 0x3C00)
    m = (x > 0).astype(np.uint8)
    (mh,) = hip.call("cast_bool_f16", 5000, In(m), Out(5000, "f16"))
    assert np.array_equal(mh, np.where(m, 0x3C00, 0).astype(np.uint16))
    (mb,) = hip.call("cast_f16_bool", hb.size, In(hb), Out(hb.size, "bool"))
    assert np.array_equal(mb, (np.nan_to_num(want, nan=1.0) != 0).astype(np.uint8))
    (mf,) = hip.call("cast_bool_f32", 5000, In(m), Out(5000, "f32"))
    assert np.array_equal(mf, m.astype(np.float32))
    lay = LY.permuted([70, 90], [1, 0], off=1)
    st = r.standard_normal(lay["size"]).astype(np.float32)
    (c,) = hip.call("copy_strided_f32", 6300, 2, meta_unary(lay["dims"], lay["strides"], 1), In(st), Out(6300, "f32"))
    assert np.array_equal(c.reshape(70, 90), LY.gather(st, lay))


def test_error_reporting(hip):
    import maidenx_amd.lib as L
    x = np.zeros(16, np.float32)
    md2 = np.array([4, 4, 4, 1, 4, 4, 4, 1, 0], dtype=np.uint64)     # dims | strides | red_len[2] | red_stride[2] | offset
    buf = L.DeviceBuffer.from_numpy(x)
    out = L.DeviceBuffer(64)
    L.call("sum_f32", 16, 2, 2, md2, buf, out)          # two reduced dims: not supported, must say so
    with pytest.raises(L.HipError):
        L.check()
    L.check()                                            # reading the status cleared it


# ---- the binary families for f64, bool and the integers ---------------------------------------------------------
WIDE_DTS = ["f64", "bool", "u8", "u16", "u32", "u64", "i8", "i16", "i32", "i64"]


def wide_values(r, n, dt):
    if dt == "f64":
        x = r.standard_normal(n)
        k = min(n, 8)
        x[:k] = np.array([0.0, -0.0, np.inf, -np.inf, np.nan, 1.0, -1.0, 1e308])[:k]
        return x
    if dt == "bool":
        return r.integers(0, 2, n, dtype=np.uint8)
    info = np.iinfo(NP[dt])
    x = r.integers(info.min, info.max, n, dtype=NP[dt], endpoint=True)
    sel = r.random(n)
    x[sel < 0.35] = r.integers(max(info.min, -9), 9, int((sel < 0.35).sum()), dtype=NP[dt])      # zeros, small factors and divisors
    x[(sel > 0.9)] = info.max
    x[(sel > 0.95)] = info.min
    if info.min < 0:
        x[(sel > 0.85) & (sel <= 0.9)] = -1
    return x


@pytest.mark.parametrize("dt", WIDE_DTS)
@pytest.mark.parametrize("lname", list(BIN_LAYOUTS))
def test_binary_ops_wide_dtypes_bit_exact(oracle, hip, lname, dt):
    ll, rl = BIN_LAYOUTS[lname]()
    r = rng(hash(lname) % 1000 + 7)
    ls, rs = wide_values(r, ll["size"], dt), wide_values(r, rl["size"], dt)
    n = int(np.prod(ll["dims"]))
    md = meta_binary(ll["dims"], ll["strides"], rl["strides"], ll["off"], rl["off"])
    for op in ["add", "sub", "mul", "div", "maximum", "minimum"]:
        (o,), (h,) = both(oracle, hip, f"{op}_{dt}", lambda: (n, len(ll["dims"]), md, In(ls), In(rs), Out(n, dt)))
        if dt == "f64":
            assert np.array_equal(np.isnan(o), np.isnan(h)), op
            if op in ("maximum", "minimum"):
                assert np.array_equal(o, h, equal_nan=True), op                  # (either zero may come back for (+0, -0))
            else:
                assert same_bits(np.where(np.isnan(o), 0, o), np.where(np.isnan(h), 0, h)), op
        else:
            assert same_bits(o, h), op
    for op in ["eq", "ne", "lt", "le", "gt", "ge", "logical_and", "logical_or", "logical_xor"]:
        (o,), (h,) = both(oracle, hip, f"{op}_{dt}", lambda: (n, len(ll["dims"]), md, In(ls), In(rs), Out(n, "bool")))
        assert np.array_equal(o, h), op


@pytest.mark.parametrize("dt", WIDE_DTS)
@pytest.mark.parametrize("lname", ["contig", "offset_misaligned", "rhs_row_bcast", "scalar_bcast", "nhwc_view_plus_bias"])
def test_inplace_ops_wide_dtypes_bit_exact(oracle, hip, lname, dt):
    ll, rl = BIN_LAYOUTS[lname]()
    lc = LY.contiguous(ll["dims"], off=ll["off"])
    r = rng(11)
    ls, rs = wide_values(r, lc["size"], dt), wide_values(r, rl["size"], dt)
    if dt == "f64":
        ls[:8], rs[:8] = r.standard_normal(min(8, ls.size)), r.standard_normal(min(8, rs.size))      # (NaN payloads are not compared here)
    n = int(np.prod(lc["dims"]))
    md = meta_binary(lc["dims"], lc["strides"], rl["strides"], lc["off"], rl["off"])
    for op in ["add_inplace", "sub_inplace", "mul_inplace", "div_inplace"]:
        (o,), (h,) = both(oracle, hip, f"{op}_{dt}", lambda: (n, len(lc["dims"]), md, InOut(ls.copy()), In(rs)))
        assert same_bits(o, h), op


# ---- conversions between the plain-number dtypes; fill and strided copy for the wide dtypes -------------------------
@pytest.mark.parametrize("src", PLAIN)
def test_casts_bit_exact(oracle, hip, src):
    x = cast_inputs(src, n=70001)
    for dst in PLAIN:
        if dst == src:
            continue
        (o,), (h,) = both(oracle, hip, f"cast_{src}_{dst}", lambda: (x.size, In(x), Out(x.size, dst)))
        if dst in ("f32", "f64"):
            assert np.array_equal(np.isnan(o), np.isnan(h)), (src, dst)
            assert same_bits(np.where(np.isnan(o), 0, o), np.where(np.isnan(h), 0, h)), (src, dst)
        else:
            assert same_bits(o, h), (src, dst)


@pytest.mark.parametrize("dt", WIDE_DTS)
def test_fill_and_strided_copy_wide_dtypes(hip, dt):
    r = rng(31)
    if dt != "bool":
        value = {"f64": -2.5}.get(dt, 7)
        (f,) = hip.call(f"fill_{dt}", 5001, Out(5001, dt), const_arg(value, dt))
        assert np.array_equal(f, np.full(5001, value, dtype=NP[dt]))
    for lay in (LY.permuted([150, 200], [1, 0]), LY.broadcast([40, 50], [1, 50]), LY.contiguous([77, 13], off=1), LY.permuted([2, 5, 6, 7], [3, 1, 0, 2])):
        src = wide_values(r, lay["size"], dt)
        n = int(np.prod(lay["dims"]))
        (c,) = hip.call(f"copy_strided_{dt}", n, len(lay["dims"]), meta_unary(lay["dims"], lay["strides"], lay["off"]), In(src), Out(n, dt))
        want = np.lib.stride_tricks.as_strided(src[lay["off"]:], lay["dims"], [st * src.itemsize for st in lay["strides"]]).ravel()
        assert same_bits(c, want), dt


# ---- unary forms for f64, bool and the integers ------------------------------------------------------------------------
@pytest.mark.parametrize("dt", WIDE_DTS)
@pytest.mark.parametrize("lname", list(UN_LAYOUTS))
def test_unary_wide_dtypes_bit_exact(oracle, hip, lname, dt):
    import maidenx_amd._signatures as S
    lay = UN_LAYOUTS[lname]()
    r = rng(hash(lname) % 1000 + 13)
    x = wide_values(r, lay["size"], dt)
    n = int(np.prod(lay["dims"]))
    md = meta_unary(lay["dims"], lay["strides"], lay["off"])
    plain, const = S.wide_unary_ops(dt)

    transcendental = {"sigmoid", "tanh", "gelu", "sin", "cos", "tan", "ln", "log10", "log2", "exp", "exp10", "exp2", "softplus", "pow", "elu"}

    def ulp_diff_f64(a, b):
        ia, ib = a.view(np.int64), b.view(np.int64)
        with np.errstate(over="ignore"):
            ia = np.where(ia < 0, np.int64(-2 ** 63) - ia, ia)        # order-preserving map of the bit patterns
            ib = np.where(ib < 0, np.int64(-2 ** 63) - ib, ib)
            return np.abs(ia - ib)                                    # (the two results are close: no overflow)

    def check(o, h, what):
        op_name = what if isinstance(what, str) else what[0]
        if dt == "f64" and op_name in transcendental:
            # the device math library against the host libm: 2 ulp (the bar stated for these f64 forms), NaN and infinities alike
            assert np.array_equal(np.isnan(o), np.isnan(h)), what
            fin = np.isfinite(o) & np.isfinite(h)
            assert np.array_equal(o[~fin & ~np.isnan(o)], h[~fin & ~np.isnan(h)]), what
            d = ulp_diff_f64(o[fin], h[fin])
            tiny = np.abs(o[fin]) < 1e-300                                        # results in or next to the subnormal range: absolute
            ok = (d <= 2) | tiny
            if op_name in ("gelu", "sigmoid", "softplus", "elu"):
                # composed forms: `1 + tanh(..)` and `exp(x) - 1` cancel, so one ulp of the inner routine is many ulp of a
                # small result; there the bar is absolute, 8 units of 2^-53 on the scale of max(1, |result|)
                ok |= np.abs(o[fin] - h[fin]) <= 8 * 2.0 ** -53 * np.maximum(1.0, np.abs(h[fin]))
            assert np.all(ok), (what, float(d[~ok].max()))
        elif dt == "f64" and o.dtype == np.float64:
            assert np.array_equal(np.isnan(o), np.isnan(h)), what
            assert same_bits(np.where(np.isnan(o), 0, o), np.where(np.isnan(h), 0, h)), what
        else:
            assert same_bits(o, h), what
    for op in plain:
        odt = "bool" if op == "logical_not" else dt
        (o,), (h,) = both(oracle, hip, f"{op}_{dt}", lambda: (n, len(lay["dims"]), md, In(x), Out(n, odt)))
        check(o, h, op)
    if dt == "f64":
        consts = [0.0, -1.5, 3.25]
    elif dt == "bool":
        consts = [0, 1]
    else:
        info = np.iinfo(NP[dt])
        consts = [0, 3, info.max, info.min] + ([-1] if info.min < 0 else [])
    for c in consts:
        for op in const:
            odt = "bool" if op in S.BOOL_OUT else dt
            (o,), (h,) = both(oracle, hip, f"{op}_{dt}", lambda: (n, len(lay["dims"]), md, In(x), const_arg(c, dt), Out(n, odt)))
            if dt == "f64" and op in ("maximum_scalar", "minimum_scalar"):
                assert np.array_equal(o, h, equal_nan=True), (op, c)
            else:
                check(o, h, (op, c))


# ---- reductions for f64 and the integers ---------------------------------------------------------------------------------
RED_WIDE = ["f64", "u8", "u16", "u32", "u64", "i8", "i16", "i32", "i64"]


@pytest.mark.parametrize("dt", RED_WIDE)
@pytest.mark.parametrize("shape,dim", RED_CASES)
def test_reductions_wide_dtypes(oracle, hip, shape, dim, dt):
    r = rng(43)
    n = int(np.prod(shape))
    off = 1 if n % 2 else 0
    if dt == "f64":
        x = np.concatenate([np.full(off, 5.0), r.uniform(-1, 1, n)])
    else:
        info = np.iinfo(NP[dt])
        x = r.integers(info.min, info.max, n + off, dtype=NP[dt], endpoint=True)          # sums wrap many times over
    md = meta_reduce(shape, contiguous_strides(shape), dim, off)
    for op in ["sum", "max", "min"] + (["mean"] if dt == "f64" else []):
        (o,), (h,) = both(oracle, hip, f"{op}_{dt}", lambda: (n, len(shape), 1, md, In(x), Out(n // shape[dim], dt)))
        if dt != "f64" or op in ("max", "min"):
            assert same_bits(o, h), op
            continue
        xs = x[off:].reshape(shape)
        scale = np.abs(xs).sum(dim).ravel() / (shape[dim] if op == "mean" else 1)
        assert np.max(np.abs(h - o) / np.maximum(scale, 1e-300)) <= 1e-13, op         # f64: the two summation orders agree to rounding


@pytest.mark.parametrize("dt", RED_WIDE)
@pytest.mark.parametrize("shape,out_shape", STS_CASES)
def test_sum_to_shape_wide_dtypes(oracle, hip, shape, out_shape, dt):
    r = rng(47)
    n = int(np.prod(shape))
    x = r.uniform(-1, 1, n) if dt == "f64" else r.integers(np.iinfo(NP[dt]).min, np.iinfo(NP[dt]).max, n, dtype=NP[dt], endpoint=True)
    md = meta_sum_to_shape(shape, contiguous_strides(shape), out_shape, 0)
    n_out = int(np.prod(out_shape))
    (o,), (h,) = both(oracle, hip, f"sum_to_shape_{dt}", lambda: (n, len(shape), md, In(x), Out(n_out, dt)))
    if dt != "f64":
        assert same_bits(o, h)
        return
    axes = tuple(i for i, (a, b) in enumerate(zip(shape, out_shape)) if a != b)
    scale = np.abs(x.reshape(shape)).sum(axis=axes).ravel() if axes else np.abs(x)
    assert np.max(np.abs(h - o) / np.maximum(scale, 1e-300)) <= 1e-13


@pytest.mark.parametrize("dt", ["i32", "u8", "i64", "f64"])
def test_reduce_wide_large_strided_input_is_the_reduction_of_its_logical_copy(oracle, hip, dt):
    """As for f32: from 2^18 elements a strided input is reduced through its logical-order copy.  Integer sums wrap, so
    any order gives the reference's bits; f64 sums agree to rounding; max / min bit for bit."""
    r = rng(191)
    for dims, perm in (([520, 640], [1, 0]), ([6, 300, 200], [0, 2, 1])):
        lay = LY.permuted(dims, perm)
        n = int(np.prod(dims))
        st = r.standard_normal(lay["size"]) if dt == "f64" else r.integers(0 if dt == "u8" else -100, 100, lay["size"]).astype(NP[dt])
        for dim in range(len(dims)):
            md = meta_reduce(lay["dims"], lay["strides"], dim, 0)
            out_n = n // lay["dims"][dim]
            for op in ("sum", "max", "min"):
                (o,), (h,) = both(oracle, hip, f"{op}_{dt}", lambda: (n, len(dims), 1, md, In(st), Out(out_n, dt)))
                if dt == "f64" and op == "sum":
                    assert np.allclose(o, h, rtol=1e-12, atol=1e-11), (op, dim)
                else:
                    assert same_bits(o, h), (op, dim)


def test_reduce_wide_strided_input_and_nan_rule(oracle, hip):
    lay = LY.permuted([30, 50], [1, 0])
    x = rng(53).integers(-1000, 1000, lay["size"], dtype=np.int64)
    md = meta_reduce(lay["dims"], lay["strides"], 1, lay["off"])
    (o,), (h,) = both(oracle, hip, "sum_i64", lambda: (30 * 50, 2, 1, md, In(x), Out(30, "i64")))
    assert same_bits(o, h)
    for data in ([-np.inf, np.nan, -np.inf, np.nan], [np.nan, 2.0, np.nan, -1.0]):
        v = np.array(data, dtype=np.float64)
        for op in ("max", "min"):
            (o,), (h,) = both(oracle, hip, f"{op}_f64", lambda: (4, 1, 1, meta_reduce([4], [1], 0), In(v), Out(1, "f64")))
            assert same_bits(o, h), (op, data)


# ---- matmul for f64 and the integers: the reference's accumulation order, so identical bits -----------------------------
MM_WIDE_SHAPES = [(1, 128, 128, 128), (2, 130, 70, 97), (3, 64, 600, 64), (1, 1000, 3, 1), (1, 3, 1000, 1), (2, 37, 19, 53), (1, 100, 576, 64),
                  (4, 16, 16, 16), (1, 1, 257, 1)]


def wide_matrix(r, shape, dt):
    if dt == "f64":
        return r.standard_normal(shape)
    info = np.iinfo(NP[dt])
    return r.integers(info.min, info.max, shape, dtype=NP[dt], endpoint=True)      # products and sums wrap


@pytest.mark.parametrize("dt", ["f64", "i32", "i64", "u8", "u64", "i16"])
@pytest.mark.parametrize("a_perm,b_perm", [(False, False), (True, False), (False, True), (True, True)])
@pytest.mark.parametrize("shape", MM_WIDE_SHAPES, ids=lambda s: "x".join(map(str, s)))
def test_matmul_forward_wide_dtypes(oracle, hip, shape, a_perm, b_perm, dt):
    batch, m, k, n = shape
    r = rng(59)
    a, b = wide_matrix(r, (batch, m, k), dt), wide_matrix(r, (batch, k, n), dt)
    a_shape, b_shape = [batch, m, k], [batch, k, n]
    a_st, b_st = contiguous_strides(a_shape), contiguous_strides(b_shape)
    if a_perm:
        a, a_st = np.ascontiguousarray(a.transpose(0, 2, 1)), [m * k, 1, m]
    if b_perm:
        b, b_st = np.ascontiguousarray(b.transpose(0, 2, 1)), [k * n, 1, k]
    md = meta_matmul([batch, m, n], a_shape, b_shape, a_st, b_st)
    (o,), (h,) = both(oracle, hip, f"matmul_{dt}", lambda: (batch * m * n, md, In(a.ravel()), In(b.ravel()), Out(batch * m * n, dt)))
    assert same_bits(o, h)


@pytest.mark.parametrize("dt", ["f64", "i32", "i64", "u16"])
@pytest.mark.parametrize("shape", [(1, 128, 128, 128), (2, 130, 70, 97), (1, 10000, 3, 1), (3, 33, 65, 17)], ids=lambda s: "x".join(map(str, s)))
def test_matmul_backward_wide_dtypes(oracle, hip, shape, dt):
    batch, m, k, n = shape
    r = rng(61)
    a, b, go = wide_matrix(r, (batch, m, k), dt), wide_matrix(r, (batch, k, n), dt), wide_matrix(r, (batch, m, n), dt)
    md = meta_matmul([batch, m, n], [batch, m, k], [batch, k, n], contiguous_strides([batch, m, k]), contiguous_strides([batch, k, n]))
    build = lambda: (batch * m * k, batch * k * n, md, In(go.ravel()), In(a.ravel()), In(b.ravel()), Out(batch * m * k, dt), Out(batch * k * n, dt))
    (oa, ob), (ha, hb) = both(oracle, hip, f"matmul_backward_{dt}", build)
    assert same_bits(oa, ha) and same_bits(ob, hb)
