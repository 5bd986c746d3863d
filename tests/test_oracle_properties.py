"""CPU: pin the parts of the oracle the reference's own vectors leave open, with checks a
plausible mistake (wrong stride, dropped offset, transposed operand, wrong rounding) would fail:
numpy N-d indexing for the strided walks, closed forms in f64, the bf16 rounding rule over all
2^16 bit patterns, textbook matmul, adjoint identities for pad and im2col/col2im."""
import numpy as np
import pytest

import layouts as LY
from helpers import (NP, PLAIN, cast_inputs, In, InOut, Out, bf16_to_f32, const_arg, contiguous_strides, f32_to_bf16, meta_binary, meta_conv,
                     meta_matmul, meta_pad, meta_reduce, meta_sum_to_shape, meta_unary, rng, ulp_diff_f32)


def test_bf16_rounding_rule_exhaustive():
    # every bf16 bit pattern survives f32 -> bf16 unchanged (NaNs stay NaN, quiet bit forced)
    bits = np.arange(1 << 16, dtype=np.uint16)
    f = bf16_to_f32(bits)
    back = f32_to_bf16(f)
    nan = np.isnan(f)
    assert np.array_equal(back[~nan], bits[~nan])
    assert np.all(np.isnan(bf16_to_f32(back[nan])))
    # ties go to even, everything else to nearest: check around every representable value
    lo = (bits[:-1].astype(np.uint32) << 16)
    finite = np.isfinite(f[:-1]) & np.isfinite(f[1:]) & (bits[:-1] & 0x7FFF != 0x7F7F)
    mid = (lo + 0x8000).view(np.float32)          # exactly half way to the next bf16
    up = (lo + 0x8001).view(np.float32)
    down = (lo + 0x7FFF).view(np.float32)
    even = np.where(bits[:-1] & 1 == 0, bits[:-1], bits[:-1] + 1)
    assert np.array_equal(f32_to_bf16(mid)[finite], even[finite])
    assert np.array_equal(f32_to_bf16(up)[finite], (bits[:-1] + 1)[finite])
    assert np.array_equal(f32_to_bf16(down)[finite], bits[:-1][finite])


def test_oracle_bf16_add_matches_host_rounding(oracle):
    r = rng(1)
    a = f32_to_bf16(r.standard_normal(4096).astype(np.float32))
    b = f32_to_bf16(r.standard_normal(4096).astype(np.float32))
    (out,) = oracle.call("add_bf16", 4096, 1, meta_binary([4096], [1], [1]), In(a), In(b), Out(4096, "bf16"))
    assert np.array_equal(out, f32_to_bf16(bf16_to_f32(a) + bf16_to_f32(b)))


LAYOUT_CASES = [
    ("contig", lambda: (LY.contiguous([5, 7]), LY.contiguous([5, 7]))),
    ("offset", lambda: (LY.contiguous([5, 7], off=1), LY.contiguous([5, 7], off=3))),
    ("rhs_row_bcast", lambda: (LY.contiguous([5, 7]), LY.broadcast([5, 7], [1, 7]))),
    ("lhs_col_bcast", lambda: (LY.broadcast([5, 7], [5, 1]), LY.contiguous([5, 7]))),
    ("lhs_transposed", lambda: (LY.permuted([5, 7], [1, 0]), LY.contiguous([5, 7]))),
    ("both_transposed", lambda: (LY.permuted([5, 7], [1, 0], off=2), LY.permuted([5, 7], [1, 0]))),
    ("nchw_view_plus_bias", lambda: (LY.permuted([2, 3, 4, 5], [0, 3, 1, 2]), LY.broadcast([2, 3, 4, 5], [1, 3, 1, 1]))),
    ("scalar_bcast", lambda: (LY.contiguous([6]), LY.broadcast([6], [1]))),
]


@pytest.mark.parametrize("name,mk", LAYOUT_CASES, ids=[c[0] for c in LAYOUT_CASES])
def test_oracle_binary_index_math_vs_numpy(oracle, name, mk):
    ll, rl = mk()
    r = rng(7)
    ls = r.standard_normal(ll["size"]).astype(np.float32)
    rs = r.standard_normal(rl["size"]).astype(np.float32)
    n = int(np.prod(ll["dims"]))
    md = meta_binary(ll["dims"], ll["strides"], rl["strides"], ll["off"], rl["off"])
    (out,) = oracle.call("sub_f32", n, len(ll["dims"]), md, In(ls), In(rs), Out(n, "f32"))
    assert np.array_equal(out.reshape(ll["dims"]), LY.gather(ls, ll) - LY.gather(rs, rl))
    # in place on a contiguous lhs with the same rhs view
    lc = LY.contiguous(ll["dims"], off=1)
    acc = r.standard_normal(lc["size"]).astype(np.float32)
    want = acc.copy()
    want[1:1 + n] = (LY.gather(acc, lc) + LY.gather(rs, rl)).ravel()
    md = meta_binary(lc["dims"], lc["strides"], rl["strides"], 1, rl["off"])
    (got,) = oracle.call("add_inplace_f32", n, len(lc["dims"]), md, InOut(acc), In(rs))
    assert np.array_equal(got, want)


def test_oracle_div_by_zero_rule(oracle):
    a = np.array([0.0, 1.0, -1.0, np.nan, -0.0, 5.0], dtype=np.float32)
    b = np.array([0.0, 0.0, 0.0, 0.0, -0.0, -0.0], dtype=np.float32)
    (out,) = oracle.call("div_f32", 6, 1, meta_binary([6], [1], [1]), In(a), In(b), Out(6, "f32"))
    assert np.array_equal(out, np.array([0.0, np.inf, np.inf, np.inf, 0.0, np.inf], dtype=np.float32))


def test_oracle_unary_closed_forms(oracle):
    r = rng(3)
    x = (r.standard_normal(20000) * 3).astype(np.float32)
    md = meta_unary([x.size], [1], 0)
    x64 = x.astype(np.float64)
    truth = {
        "exp": np.exp(x64), "tanh": np.tanh(x64), "sigmoid": 1 / (1 + np.exp(-x64)),
        "gelu": 0.5 * x64 * (1 + np.tanh(0.7978845608028654 * (x64 + 0.044715 * x64 ** 3))),
        "softplus": np.log1p(np.exp(x64)), "square": x64 * x64, "neg": -x64, "relu": np.maximum(x64, 0),
    }
    for op, t in truth.items():
        (out,) = oracle.call(f"{op}_f32", x.size, 1, md, In(x), Out(x.size, "f32"))
        err = np.abs(out.astype(np.float64) - t)
        scale = np.maximum(np.abs(t), 1e-30)
        # gelu/softplus lose relative accuracy where 1+tanh / 1+exp cancel; bound them absolutely
        if op in ("gelu", "softplus"):
            assert np.max(err) < 2e-6, op
        else:
            assert np.max(err / scale) < 3e-7, op
    (out,) = oracle.call("pow_f32", x.size, 1, md, In(x), 2.0, Out(x.size, "f32"))
    assert np.max(ulp_diff_f32(out, (x64 * x64).astype(np.float32))) <= 1


@pytest.mark.parametrize("shape,dim", [([6, 5], 0), ([6, 5], 1), ([3, 4, 5], 0), ([3, 4, 5], 1), ([3, 4, 5], 2), ([7], 0)])
def test_oracle_reductions_vs_numpy(oracle, shape, dim):
    r = rng(11)
    x = r.uniform(-1, 1, int(np.prod(shape))).astype(np.float32)
    st = np.concatenate([[9.0], x]).astype(np.float32)      # offset 1
    md = meta_reduce(shape, contiguous_strides(shape), dim, 1)
    xs = x.reshape(shape).astype(np.float64)
    n = x.size
    for op, ref in (("sum", xs.sum(dim)), ("mean", xs.mean(dim)), ("max", xs.max(dim)), ("min", xs.min(dim))):
        (out,) = oracle.call(f"{op}_f32", n, len(shape), 1, md, In(st), Out(n // shape[dim], "f32"))
        if op in ("max", "min"):
            assert np.array_equal(out, ref.ravel().astype(np.float32))
        else:
            assert np.allclose(out, ref.ravel(), rtol=0, atol=1e-5)


def test_oracle_max_seed_and_nan_rule(oracle):
    # every element below the seed f32::MIN or NaN: the seed survives (reduction.rs:433,603)
    x = np.array([-np.inf, np.nan, -np.inf, np.nan], dtype=np.float32)
    (out,) = oracle.call("max_f32", 4, 1, 1, meta_reduce([4], [1], 0), In(x), Out(1, "f32"))
    assert out[0] == np.finfo(np.float32).min
    x = np.array([np.nan, 2.0, np.nan, -1.0], dtype=np.float32)
    (out,) = oracle.call("max_f32", 4, 1, 1, meta_reduce([4], [1], 0), In(x), Out(1, "f32"))
    assert out[0] == 2.0


@pytest.mark.parametrize("shape,out_shape", [([4, 6], [4, 6]), ([4, 6], [1, 6]), ([4, 6], [4, 1]), ([3, 4, 5], [1, 4, 1]),
                                             ([3, 4, 5], [3, 1, 5]), ([2, 3, 4, 5], [1, 3, 1, 5]), ([5], [1])])
def test_oracle_sum_to_shape_vs_numpy(oracle, shape, out_shape):
    r = rng(5)
    x = r.uniform(-1, 1, int(np.prod(shape))).astype(np.float32)
    md = meta_sum_to_shape(shape, contiguous_strides(shape), out_shape, 0)
    (out,) = oracle.call("sum_to_shape_f32", x.size, len(shape), md, In(x), Out(int(np.prod(out_shape)), "f32"))
    axes = tuple(i for i, (a, b) in enumerate(zip(shape, out_shape)) if a != b)
    ref = x.reshape(shape).astype(np.float64).sum(axis=axes, keepdims=True)
    assert np.allclose(out.reshape(out_shape), ref, atol=1e-5)


def test_oracle_sum_to_shape_identity_turns_negative_zero_positive(oracle):
    x = np.array([-0.0, 1.0, -2.0], dtype=np.float32)
    (out,) = oracle.call("sum_to_shape_f32", 3, 1, meta_sum_to_shape([3], [1], [3]), In(x), Out(3, "f32"))
    assert np.array_equal(out, x) and not np.signbit(out[0])


def matmul_case(r, batch, m, k, n, a_perm=False, b_perm=False):
    a = r.standard_normal((batch, m, k)).astype(np.float32)
    b = (r.standard_normal((batch, k, n)) * 0.02).astype(np.float32)
    a_shape, b_shape = [batch, m, k], [batch, k, n]
    a_st, b_st = contiguous_strides(a_shape), contiguous_strides(b_shape)
    a_store, b_store = a, b
    if a_perm:      # a is a transposed view of storage [batch, k, m]
        a_store = np.ascontiguousarray(a.transpose(0, 2, 1))
        a_st = [m * k, 1, m]
    if b_perm:
        b_store = np.ascontiguousarray(b.transpose(0, 2, 1))
        b_st = [k * n, 1, k]
    md = meta_matmul([batch, m, n], a_shape, b_shape, a_st, b_st)
    return a, b, a_store.ravel(), b_store.ravel(), md


@pytest.mark.parametrize("a_perm,b_perm", [(False, False), (True, False), (False, True), (True, True)])
def test_oracle_matmul_vs_textbook(oracle, a_perm, b_perm):
    r = rng(2)
    batch, m, k, n = 3, 5, 7, 4
    a, b, a_st, b_st, md = matmul_case(r, batch, m, k, n, a_perm, b_perm)
    (c,) = oracle.call("matmul_f32", batch * m * n, md, In(a_st), In(b_st), Out(batch * m * n, "f32"))
    ref = np.einsum("bmk,bkn->bmn", a.astype(np.float64), b.astype(np.float64))
    assert np.allclose(c.reshape(batch, m, n), ref, rtol=1e-5, atol=1e-6)


def test_oracle_matmul_backward_vs_textbook(oracle):
    r = rng(4)
    batch, m, k, n = 2, 5, 6, 3
    a, b, a_st, b_st, md = matmul_case(r, batch, m, k, n)
    go = r.standard_normal((batch, m, n)).astype(np.float32)
    ga, gb = oracle.call("matmul_backward_f32", a.size, b.size, md, In(go.ravel()), In(a_st), In(b_st), Out(a.size, "f32"),
                         Out(b.size, "f32"))
    ref_a = np.einsum("bmn,bkn->bmk", go.astype(np.float64), b.astype(np.float64))
    ref_b = np.einsum("bmk,bmn->bkn", a.astype(np.float64), go.astype(np.float64))
    assert np.allclose(ga.reshape(a.shape), ref_a, rtol=1e-5, atol=1e-6)
    assert np.allclose(gb.reshape(b.shape), ref_b, rtol=1e-5, atol=1e-6)


def test_oracle_bf16_matmul_rounds_every_step(oracle):
    # 1 + 2^-9 * 256 terms: an f32 accumulator reaches 1.5, a bf16 accumulator stays at 1
    k = 257
    a = f32_to_bf16(np.ones(k, dtype=np.float32))
    b = f32_to_bf16(np.concatenate([[1.0], np.full(k - 1, 2.0 ** -9)]).astype(np.float32))
    md = meta_matmul([1, 1], [1, k], [k, 1], [k, 1], [1, 1])
    (c,) = oracle.call("matmul_bf16", 1, md, In(a), In(b), Out(1, "bf16"))
    assert bf16_to_f32(c)[0] == 1.0


def test_oracle_pad_is_adjoint_of_its_backward(oracle):
    r = rng(9)
    shape, pads = [2, 3, 4], [(1, 0), (0, 2), (2, 1)]
    out_shape = [s + p[0] + p[1] for s, p in zip(shape, pads)]
    n_in, n_out = int(np.prod(shape)), int(np.prod(out_shape))
    md = meta_pad(shape, contiguous_strides(shape), 0, out_shape, pads)
    x = r.standard_normal(n_in).astype(np.float32)
    y = r.standard_normal(n_out).astype(np.float32)
    (px,) = oracle.call("pad_with_constant_f32", n_in, n_out, 3, md, In(x), Out(n_out, "f32"), 0.0)
    (by,) = oracle.call("pad_with_constant_backward_f32", n_in, n_out, 3, md, In(y), InOut(np.zeros(n_in, np.float32)))
    ref = np.pad(x.reshape(shape), pads)
    assert np.array_equal(px.reshape(out_shape), ref)
    assert np.isclose(np.dot(px.astype(np.float64), y), np.dot(x.astype(np.float64), by))


def im2col_numpy(x, kh, kw, ph, pw, sh, sw):
    B, Cc, H, W = x.shape
    oh, ow = (H + 2 * ph - kh) // sh + 1, (W + 2 * pw - kw) // sw + 1
    xp = np.pad(x, [(0, 0), (0, 0), (ph, ph), (pw, pw)])
    col = np.zeros((B, Cc * kh * kw, oh * ow), dtype=x.dtype)
    for c in range(Cc):
        for i in range(kh):
            for j in range(kw):
                patch = xp[:, c, i:i + sh * oh:sh, j:j + sw * ow:sw]
                col[:, (c * kh + i) * kw + j, :] = patch.reshape(B, -1)
    return col, oh, ow


@pytest.mark.parametrize("kh,kw,p,s", [(3, 3, 1, 1), (3, 3, 0, 1), (2, 3, 1, 2), (1, 1, 0, 1), (5, 5, 2, 2)])
def test_oracle_im2col_col2im_vs_bruteforce_and_adjoint(oracle, kh, kw, p, s):
    r = rng(13)
    B, Cc, H, W = 2, 3, 7, 8
    x = r.standard_normal((B, Cc, H, W)).astype(np.float32)
    col_ref, oh, ow = im2col_numpy(x, kh, kw, p, p, s, s)
    md = meta_conv(B, Cc, H, W, kh, kw, oh, ow, p, p, s, s)
    (col,) = oracle.call("conv2d_im2col_f32", col_ref.size, md, In(x.ravel()), Out(col_ref.size, "f32"))
    assert np.array_equal(col.reshape(col_ref.shape), col_ref)
    # adjoint identity <im2col(x), y> == <x, col2im(y)> when no column index is cut off
    y = r.standard_normal(col_ref.size).astype(np.float32)
    (back,) = oracle.call("conv2d_col2im_f32", y.size, md, In(y), Out(x.size, "f32"))
    lhs = np.dot(col_ref.ravel().astype(np.float64), y.astype(np.float64))
    rhs = np.dot(x.ravel().astype(np.float64), back.astype(np.float64))
    assert np.isclose(lhs, rhs, rtol=1e-5)
    # the reference's caller passes num_els = B*C*H*W: column indices at or beyond it contribute nothing
    cut = x.size
    y_cut = y.copy()
    y_cut[cut:] = 0
    (a,) = oracle.call("conv2d_col2im_f32", cut, md, In(y), Out(x.size, "f32"))
    (b,) = oracle.call("conv2d_col2im_f32", y.size, md, In(y_cut), Out(x.size, "f32"))
    assert np.array_equal(a, b)


def test_oracle_threaded_mode_agrees_with_sequential(oracle):
    r = rng(21)
    x = r.uniform(-1, 1, 64 * 33).astype(np.float32)
    md = meta_reduce([64, 33], [33, 1], 0)
    (seq,) = oracle.call("max_f32", x.size, 2, 1, md, In(x), Out(33, "f32"))
    (s1,) = oracle.call("sum_f32", x.size, 2, 1, md, In(x), Out(33, "f32"))
    oracle.set_threads(4)
    try:
        (par,) = oracle.call("max_f32", x.size, 2, 1, md, In(x), Out(33, "f32"))
        (s4,) = oracle.call("sum_f32", x.size, 2, 1, md, In(x), Out(33, "f32"))
    finally:
        oracle.set_threads(1)
    assert np.array_equal(seq, par)
    assert np.allclose(s1, s4, atol=1e-5)


# ---- reflection / replication padding, fold, softmax -------------------------------------------------
EDGE_CASES = [([7], [(3, 2)]), ([5, 6], [(1, 2), (0, 3)]), ([2, 3, 4], [(1, 0), (2, 2), (3, 1)]), ([4, 9], [(0, 0), (4, 8)])]


@pytest.mark.parametrize("mode,np_mode", [("reflection", "reflect"), ("replication", "edge")])
@pytest.mark.parametrize("shape,pads", EDGE_CASES)
def test_oracle_edge_pad_vs_numpy_pad_and_adjoint(oracle, shape, pads, mode, np_mode):
    r = rng(83)
    x = r.standard_normal(shape)
    out_shape = [s + p[0] + p[1] for s, p in zip(shape, pads)]
    n_in, n_out = x.size, int(np.prod(out_shape))
    md = meta_pad(shape, contiguous_strides(shape), 0, out_shape, pads)
    (y,) = oracle.call(f"pad_with_{mode}_f64", n_in, n_out, len(shape), md, In(x.ravel()), Out(n_out, "f64"))
    assert np.array_equal(y.reshape(out_shape), np.pad(x, pads, mode=np_mode))      # numpy's own pad
    # a transposed (strided) input reads the same logical tensor
    if len(shape) == 2:
        lay = LY.permuted(shape, [1, 0])
        st = np.ascontiguousarray(x.T).ravel()
        assert np.array_equal(LY.gather(st, lay), x)
        mds = meta_pad(shape, lay["strides"], 0, out_shape, pads)
        (ys,) = oracle.call(f"pad_with_{mode}_f64", n_in, n_out, 2, mds, In(st), Out(n_out, "f64"))
        assert np.array_equal(ys, y)
    # backward is the adjoint: <pad(x), g> = <x, pad_backward(g)>
    g = r.standard_normal(n_out)
    (gx,) = oracle.call(f"pad_with_{mode}_backward_f64", n_in, n_out, len(shape), md, In(g), InOut(np.full(n_in, 9.0)))
    assert abs(np.dot(y, g) - np.dot(x.ravel(), gx)) <= 1e-9 * (np.abs(y * g).sum() + 1)


@pytest.mark.parametrize("dt", ["u8", "i16", "u32", "i64"])
def test_oracle_integer_pads_vs_numpy_and_wrapping_sums(oracle, dt):
    """The integer instantiations (padding.rs:670-743): forward against numpy.pad, backward against numpy's wrapping
    add.at over the index map that numpy.pad of an index tensor gives (an independent statement of which output reads
    which input)."""
    from helpers import NP
    r = rng(89)
    info = np.iinfo(NP[dt])
    shape, pads = [4, 9], [(2, 1), (4, 8)]
    out_shape = [s + p[0] + p[1] for s, p in zip(shape, pads)]
    n_in, n_out = int(np.prod(shape)), int(np.prod(out_shape))
    x = r.integers(info.min, info.max, shape, dtype=NP[dt], endpoint=True)
    g = r.integers(info.min, info.max, n_out, dtype=NP[dt], endpoint=True)
    md = meta_pad(shape, contiguous_strides(shape), 0, out_shape, pads)
    (y,) = oracle.call(f"pad_with_constant_{dt}", n_in, n_out, 2, md, In(x.ravel()), Out(n_out, dt), 3)
    assert np.array_equal(y.reshape(out_shape), np.pad(x, pads, constant_values=3))
    (gx,) = oracle.call(f"pad_with_constant_backward_{dt}", n_in, n_out, 2, md, In(g), InOut(np.full(n_in, 9, NP[dt])))
    assert np.array_equal(gx.reshape(shape), g.reshape(out_shape)[2:2 + 4, 4:4 + 9])
    for mode, np_mode in (("reflection", "reflect"), ("replication", "edge")):
        (y,) = oracle.call(f"pad_with_{mode}_{dt}", n_in, n_out, 2, md, In(x.ravel()), Out(n_out, dt))
        assert np.array_equal(y.reshape(out_shape), np.pad(x, pads, mode=np_mode))
        (gx,) = oracle.call(f"pad_with_{mode}_backward_{dt}", n_in, n_out, 2, md, In(g), InOut(np.full(n_in, 9, NP[dt])))
        idx = np.pad(np.arange(n_in).reshape(shape), pads, mode=np_mode).ravel()
        want = np.zeros(n_in, dtype=NP[dt])
        with np.errstate(over="ignore"):
            np.add.at(want, idx, g)
        assert np.array_equal(gx, want)


def test_oracle_reflection_wraps_more_than_once(oracle):
    # pads wider than the dim: the mirror loop of padding.rs:186-193 runs several times; numpy's reflect does the same
    x = np.arange(1.0, 4.0)
    md = meta_pad([3], [1], 0, [3 + 7 + 5], [(7, 5)])
    (y,) = oracle.call("pad_with_reflection_f64", 3, 15, 1, md, In(x), Out(15, "f64"))
    assert np.array_equal(y, np.pad(x, (7, 5), mode="reflect"))


@pytest.mark.parametrize("shape,dim,size,step", [([9], 0, 3, 2), ([4, 10], 1, 4, 3), ([3, 8, 2], 1, 2, 1), ([6, 5], 0, 3, 3)])
def test_oracle_fold_is_adjoint_of_unfold(oracle, shape, dim, size, step):
    from numpy.lib.stride_tricks import sliding_window_view
    r = rng(89)
    x = r.standard_normal(shape)
    # unfold as Layout::unfold builds it (layout.rs:193-250): windows at `dim`, the window dim right after
    win = np.moveaxis(sliding_window_view(x, size, axis=dim), -1, dim + 1)
    win = np.take(win, np.arange(0, win.shape[dim], step), axis=dim)
    y = r.standard_normal(win.shape)
    n_windows = win.shape[dim]
    fold_size = (n_windows - 1) * step + size                  # tensor/ops/reduction.rs:257
    md = u64_(list(win.shape), contiguous_strides(list(win.shape)), dim, dim + 1, fold_size, step, size, 0)
    out_shape = list(shape)
    out_shape[dim] = fold_size
    (f,) = oracle.call("fold_f64", y.size, y.ndim, md, In(y.ravel()), Out(int(np.prod(out_shape)), "f64"))
    xs = np.take(x, np.arange(fold_size), axis=dim)            # the part of x the windows cover
    assert abs(np.sum(win * y) - np.sum(xs * f.reshape(out_shape))) <= 1e-9 * (np.abs(win * y).sum() + 1)
    # and fold(unfold(x)) multiplies every position by the number of windows that contain it
    (fx,) = oracle.call("fold_f64", win.size, win.ndim, md, In(np.ascontiguousarray(win).ravel()), Out(int(np.prod(out_shape)), "f64"))
    (cnt,) = oracle.call("fold_f64", win.size, win.ndim, md, In(np.ones(win.size)), Out(int(np.prod(out_shape)), "f64"))
    assert np.allclose(fx.reshape(out_shape), xs * cnt.reshape(out_shape), rtol=1e-12)


def u64_(*parts):
    from helpers import u64
    return u64(*parts)


@pytest.mark.parametrize("dt", ["u8", "i32", "u64"])
def test_oracle_integer_fold_counts_windows_and_wraps(oracle, dt):
    """fold of all-ones windows counts the windows that cover each position (a closed form); fold of full-range values
    is numpy's wrapping add.at over the positions c[fold]*step + c[window]."""
    from helpers import NP
    n_windows, size, step, inner = 7, 4, 3, 5
    fold_size = (n_windows - 1) * step + size
    dims = [n_windows, size, inner]
    md = u64_(dims, contiguous_strides(dims), 0, 1, fold_size, step, size, 0)
    (cnt,) = oracle.call(f"fold_{dt}", n_windows * size * inner, 3, md, In(np.ones(n_windows * size * inner, NP[dt])), Out(fold_size * inner, dt))
    pos = np.arange(fold_size)
    want = np.array([sum(1 for w in range(n_windows) if 0 <= p - w * step < size) for p in pos])
    assert np.array_equal(cnt.reshape(fold_size, inner), np.repeat(want[:, None], inner, 1).astype(NP[dt]))
    r = rng(91)
    info = np.iinfo(NP[dt])
    y = r.integers(info.min, info.max, dims, dtype=NP[dt], endpoint=True)
    (f,) = oracle.call(f"fold_{dt}", y.size, 3, md, In(y.ravel()), Out(fold_size * inner, dt))
    acc = np.zeros((fold_size, inner), NP[dt])
    w, k = np.meshgrid(np.arange(n_windows), np.arange(size), indexing="ij")
    with np.errstate(over="ignore"):
        np.add.at(acc, (w * step + k).ravel(), y.reshape(-1, inner))
    assert np.array_equal(f.reshape(fold_size, inner), acc)


@pytest.mark.parametrize("shape,dim", [([5, 7], 1), ([5, 7], 0), ([3, 4, 6], 1), ([2, 3, 4, 5], 3), ([2, 3, 4, 5], 0), ([6], 0), ([4, 3], 9)])
def test_oracle_softmax_vs_scipy(oracle, shape, dim):
    from scipy.special import softmax as sp_softmax
    r = rng(97)
    x = r.standard_normal(shape) * 3
    n = x.size
    md = meta_unary(shape, contiguous_strides(shape), 0)
    (y,) = oracle.call("softmax_f64", n, len(shape), dim, md, In(x.ravel()), Out(n, "f64"))
    axis = dim if dim < len(shape) else len(shape) - 1          # out of range means the last dim (softmax.rs:74)
    assert np.allclose(y.reshape(shape), sp_softmax(x, axis=axis), rtol=1e-12, atol=0)
    (y32,) = oracle.call("softmax_f32", n, len(shape), dim, md, In(x.astype(np.float32).ravel()), Out(n, "f32"))
    assert np.allclose(y32.reshape(shape), sp_softmax(x.astype(np.float32).astype(np.float64), axis=axis), rtol=2e-6)


def test_oracle_softmax_strided_two_dims_and_special_values(oracle):
    from scipy.special import softmax as sp_softmax
    r = rng(101)
    x = r.standard_normal((6, 9))
    lay = LY.permuted([6, 9], [1, 0], off=2)
    st = np.concatenate([np.zeros(2), np.ascontiguousarray(x.T).ravel()])
    assert np.array_equal(LY.gather(st, lay), x)
    for dim in (0, 1):
        md = meta_unary([6, 9], lay["strides"], lay["off"])
        (y,) = oracle.call("softmax_f64", 54, 2, dim, md, In(st), Out(54, "f64"))
        assert np.allclose(y.reshape(6, 9), sp_softmax(x, axis=dim), rtol=1e-12)
    # -inf entries vanish, an all -inf slice is NaN (the sum starts from exp(-inf - -inf)), NaNs never become the maximum
    v = np.array([[0.0, -np.inf, 1.0], [-np.inf, -np.inf, -np.inf], [np.nan, 1.0, 2.0]], dtype=np.float32)
    (y,) = oracle.call("softmax_f32", 9, 2, 1, meta_unary([3, 3], [3, 1], 0), In(v.ravel()), Out(9, "f32"))
    y = y.reshape(3, 3)
    assert y[0, 1] == 0 and abs(y[0, 0] + y[0, 2] - 1) < 1e-6
    assert np.all(np.isnan(y[1]))
    assert np.isnan(y[2, 0]) and np.all(np.isnan(y[2]))        # exp(NaN - max) poisons the sum


@pytest.mark.parametrize("shape,perm,dim", [([3, 4, 5], (0, 2, 1), 2), ([2, 3, 4, 5], (3, 1, 0, 2), 2), ([2, 3, 4, 5], (1, 0, 3, 2), 3),
                                            ([4, 3, 5], (2, 1, 0), 2), ([2, 5, 3, 2], (0, 1, 3, 2), 2)])
def test_oracle_softmax_strided_with_several_leading_dims(oracle, shape, perm, dim):
    """The non-contiguous branch with two or more dims in front of `dim` (softmax.rs:120-126) decomposes the slice number
    with dim 0 FASTEST, and writes slice number `pre_idx` to the pre_idx-th block of the contiguous output
    (softmax.rs:176-178).  So the output, read as [prod(leading), D, post], holds at block p the softmax of the logical
    slice whose leading coordinates are the Fortran-order decomposition of p: scipy's softmax of the logical tensor with
    its leading dims reversed (transpose, then flatten in C order).  A C-order decomposition gives another tensor whenever
    two leading dims differ in size, as they do in every case here."""
    from scipy.special import softmax as sp_softmax
    r = rng(103)
    base = r.standard_normal([shape[p] for p in np.argsort(perm)]) * 2          # storage, contiguous
    x = base.transpose(perm)                                                      # the logical tensor, a permuted view
    assert list(x.shape) == shape and not x.flags["C_CONTIGUOUS"]
    strides = [st // 8 for st in x.strides]
    n = x.size
    (y,) = oracle.call("softmax_f64", n, len(shape), dim, meta_unary(shape, strides, 0), In(base.ravel()), Out(n, "f64"))
    sm = sp_softmax(x, axis=dim)
    lead = list(range(dim))
    want = sm.transpose(lead[::-1] + list(range(dim, len(shape))))               # leading dims reversed: C flatten = F decomposition
    assert np.allclose(y, want.ravel(), rtol=1e-12, atol=0)
    c_order = sm.ravel()
    assert not np.allclose(y, c_order, rtol=1e-6), "the case cannot tell the two decompositions apart"
    (y32,) = oracle.call("softmax_f32", n, len(shape), dim, meta_unary(shape, strides, 0), In(base.astype(np.float32).ravel()), Out(n, "f32"))
    assert np.allclose(y32, sp_softmax(x.astype(np.float32).astype(np.float64), axis=dim).transpose(lead[::-1] + list(range(dim, len(shape)))).ravel(), rtol=2e-6)


def test_oracle_softmax_bf16_rounds_every_step(oracle):
    x = f32_to_bf16(np.array([0.1, 1.3, -0.7, 2.2], dtype=np.float32))
    (y,) = oracle.call("softmax_bf16", 4, 1, 0, meta_unary([4], [1], 0), In(x), Out(4, "bf16"))
    b = lambda v: bf16_to_f32(f32_to_bf16(np.float32(v)))
    xf = bf16_to_f32(x)
    m = xf.max()
    e = [b(np.exp(np.float32(b(v - m)))) for v in xf]
    s = np.float32(0)
    for t in e:
        s = b(s + t)
    want = f32_to_bf16(np.array([t / s for t in e], dtype=np.float32)).ravel()
    assert np.array_equal(y, want)


# ---- index_put_: numpy's sub-tensor assignment ------------------------------------------------------------------
@pytest.mark.parametrize("shape,n_fixed", [([6], 0), ([4, 5], 1), ([3, 4, 5], 1), ([3, 4, 5], 2), ([2, 3, 4, 5], 3)])
def test_oracle_index_put_vs_numpy(oracle, shape, n_fixed):
    r = rng(401)
    x = r.standard_normal(shape)
    fixed = [int(r.integers(0, shape[d])) for d in range(n_fixed)]
    rest = shape[n_fixed:]
    src = r.standard_normal(rest)
    # contiguous
    (y,) = oracle.call("index_put_f64", len(shape), layout(shape), n_fixed, np.array(fixed + [0], dtype=np.uint64), len(rest), layout(rest),
                       In(src.ravel()), InOut(x.ravel().copy()))
    want = x.copy()
    want[tuple(fixed)] = src
    assert np.array_equal(y.reshape(shape), want) and oracle.lib.oracle_index_error() == 0
    # permuted self and source, offsets
    if len(shape) >= 2 and len(rest) >= 2:
        xt = np.ascontiguousarray(np.moveaxis(x, -1, -2))                 # memory of a tensor whose last two dims are swapped
        st = contiguous_strides(list(xt.shape))
        st[-1], st[-2] = st[-2], st[-1]
        srct = np.ascontiguousarray(np.moveaxis(src, -1, -2))
        sst = contiguous_strides(list(srct.shape))
        sst[-1], sst[-2] = sst[-2], sst[-1]
        (y2,) = oracle.call("index_put_f64", len(shape), layout(shape, st, off=2), n_fixed, np.array(fixed + [0], dtype=np.uint64), len(rest),
                            layout(rest, sst, off=3), In(np.concatenate([[7.0] * 3, srct.ravel()])), InOut(np.concatenate([[5.0] * 2, xt.ravel()])))
        assert np.array_equal(np.moveaxis(y2[2:].reshape(xt.shape), -1, -2), want) and y2[0] == 5.0
    # every dim fixed: one element from a 0-d source
    full = [int(r.integers(0, s)) for s in shape]
    (y3,) = oracle.call("index_put_f64", len(shape), layout(shape), len(shape), np.array(full, dtype=np.uint64), 0, np.array([4], dtype=np.uint64),
                        In(np.arange(6.0)), InOut(x.ravel().copy()))
    want3 = x.copy()
    want3[tuple(full)] = 4.0
    assert np.array_equal(y3.reshape(shape), want3)


def test_oracle_index_put_flat_copy_and_errors(oracle):
    x = np.arange(10.0)
    # 1-d self, every dim fixed, 1-d source: copied behind the index, the source read with its stride
    (y,) = oracle.call("index_put_f64", 1, layout([10], [1]), 1, np.array([4], dtype=np.uint64), 1, layout([3], [2]), In(np.arange(100.0, 106.0)),
                       InOut(x.copy()))
    assert y.tolist() == [0, 1, 2, 3, 100, 102, 104, 7, 8, 9]
    def err(*args):
        (out,) = oracle.call("index_put_f64", *args)
        e = oracle.lib.oracle_index_error()
        return e, out
    same = lambda out: np.array_equal(out, x)
    e, out = err(1, layout([10]), 1, np.array([8], dtype=np.uint64), 1, layout([3]), In(np.ones(3)), InOut(x.copy()))       # does not fit
    assert e == 1 and same(out)
    e, out = err(1, layout([10]), 2, np.array([1, 1], dtype=np.uint64), 0, layout([]), In(np.ones(1)), InOut(x.copy()))     # more indices than dims
    assert e == 1 and same(out)
    e, out = err(2, layout([2, 5]), 1, np.array([2], dtype=np.uint64), 1, layout([5]), In(np.ones(5)), InOut(x.copy()))     # index out of bounds
    assert e == 1 and same(out)
    e, out = err(2, layout([2, 5]), 1, np.array([1], dtype=np.uint64), 1, layout([4]), In(np.ones(4)), InOut(x.copy()))     # shape mismatch
    assert e == 1 and same(out)
    e, out = err(2, layout([2, 5]), 2, np.array([1, 1], dtype=np.uint64), 1, layout([2]), In(np.ones(2)), InOut(x.copy()))  # flat copy into a 2-d self
    assert e == 1 and same(out)


# ---- index ops: numpy's own take / take_along_axis / add.at / bincount -------------------------------------
from helpers import layout  # noqa: E402


@pytest.mark.parametrize("shape,dim", [([5, 7], 0), ([5, 7], 1), ([3, 4, 6], 1), ([2, 3, 4, 5], 2)])
@pytest.mark.parametrize("it", ["i32", "i64"])
def test_oracle_index_select_and_index_add_vs_numpy(oracle, shape, dim, it):
    r = rng(131)
    ity = np.int32 if it == "i32" else np.int64
    x = r.standard_normal(shape)
    n_idx = 9
    idx = r.integers(0, shape[dim], n_idx).astype(ity)            # with repeats
    out_shape = list(shape)
    out_shape[dim] = n_idx
    (y,) = oracle.call(f"index_select_f64_{it}", len(shape), dim, layout(shape), n_idx, 1, 0, In(idx), In(x.ravel()),
                       Out(int(np.prod(out_shape)), "f64"))
    assert np.array_equal(y.reshape(out_shape), np.take(x, idx, axis=dim))
    # a permuted input reads the same logical tensor
    perm = list(range(len(shape)))[::-1]
    lay = LY.permuted(shape, perm)
    st = np.ascontiguousarray(np.transpose(x, np.argsort(perm))).ravel()
    assert np.array_equal(LY.gather(st, lay), x)
    (y2,) = oracle.call(f"index_select_f64_{it}", len(shape), dim, layout(shape, lay["strides"]), n_idx, 1, 0, In(idx), In(st),
                        Out(int(np.prod(out_shape)), "f64"))
    assert np.array_equal(y2, y)
    # index_add_ is the scatter that numpy's add.at does (unbuffered, in index order)
    src = r.standard_normal(out_shape)
    want = x.copy()
    sl = [slice(None)] * len(shape)
    for i, t in enumerate(idx):
        a, b = list(sl), list(sl)
        a[dim], b[dim] = int(t), i
        want[tuple(a)] = want[tuple(a)] + src[tuple(b)]
    (z,) = oracle.call(f"index_add_f64_{it}", len(shape), dim, layout(shape), layout(out_shape), n_idx, 1, 0, In(idx), In(src.ravel()),
                       InOut(x.ravel().copy()))
    assert np.array_equal(z.reshape(shape), want)
    ref = x.copy()
    index = [slice(None)] * len(shape)
    index[dim] = idx
    np.add.at(ref, tuple(index), src)
    assert np.allclose(z.reshape(shape), ref, rtol=1e-12, atol=1e-12)


@pytest.mark.parametrize("shape,dim,idx_len", [([5, 7], 1, 3), ([5, 7], 0, 8), ([3, 4, 6], 2, 6), ([2, 3, 4], 1, 1)])
def test_oracle_gather_and_scatter_add_vs_numpy(oracle, shape, dim, idx_len):
    r = rng(137)
    x = r.standard_normal(shape)
    ishape = list(shape)
    ishape[dim] = idx_len
    index = r.integers(-shape[dim], shape[dim], ishape).astype(np.int64)       # negative values wrap
    (y,) = oracle.call("gather_f64_i64", len(shape), dim, layout(shape), layout(ishape), In(index.ravel()), In(x.ravel()),
                       Out(index.size, "f64"))
    assert np.array_equal(y.reshape(ishape), np.take_along_axis(x, np.where(index < 0, index + shape[dim], index), axis=dim))
    src = r.standard_normal(ishape)
    ref = x.copy()
    pos = np.where(index < 0, index + shape[dim], index)
    grids = list(np.meshgrid(*[np.arange(s) for s in ishape], indexing="ij"))
    grids[dim] = pos
    np.add.at(ref, tuple(grids), src)
    (z,) = oracle.call("scatter_add_f64_i64", len(shape), dim, layout(shape), layout(ishape), layout(ishape), In(index.ravel()),
                       In(src.ravel()), InOut(x.ravel().copy()))
    assert np.allclose(z.reshape(shape), ref, rtol=1e-12, atol=1e-12)
    # gather and scatter_add_ are adjoint: <gather(x), g> = <x, scatter_add(0, g)>
    (s0,) = oracle.call("scatter_add_f64_i64", len(shape), dim, layout(shape), layout(ishape), layout(ishape), In(index.ravel()),
                        In(src.ravel()), InOut(np.zeros(x.size)))
    assert abs(np.dot(y, src.ravel()) - np.dot(x.ravel(), s0)) < 1e-9


def test_oracle_bincount_vs_numpy_and_errors(oracle):
    r = rng(139)
    v = r.integers(0, 50, 1000).astype(np.int32)
    (c,) = oracle.call("bincount_i32", 1000, 1, 0, In(v), 64, Out(64, "i32"))
    assert np.array_equal(c, np.bincount(v, minlength=64))
    w = r.standard_normal(1000)
    (s,) = oracle.call("bincount_weighted_f64_i32", 1000, 1, 0, In(v), 1, 0, In(w), 64, Out(64, "f64"))
    assert np.allclose(s, np.bincount(v, weights=w, minlength=64), rtol=1e-12, atol=1e-12)
    assert oracle.lib.oracle_index_error() == 0
    bad = np.array([0, 3, 1], dtype=np.int32)
    oracle.call("index_select_f64_i32", 1, 0, layout([3]), 3, 1, 0, In(bad), In(np.arange(3.0)), Out(3, "f64"))
    assert oracle.lib.oracle_index_error() == 1          # IndexOutOfBounds in the reference
    oracle.call("gather_f64_i32", 1, 0, layout([3]), layout([2]), In(np.array([-4, 0], dtype=np.int32)), In(np.arange(3.0)), Out(2, "f64"))
    assert oracle.lib.oracle_index_error() == 1


# ---- f16: the oracle's software codec against numpy's IEEE binary16 ---------------------------------------
def test_oracle_f16_codec_matches_numpy_float16(oracle):
    # decode: every bit pattern through a cast to f32 (cast_f16... is a HIP-only helper, so use neg twice + add 0 paths):
    # add_f16(x, +0) returns encode(decode(x) + 0) — exact for every finite pattern and a NaN for NaNs
    bits = np.arange(1 << 16, dtype=np.uint16)
    zero = np.zeros(1 << 16, dtype=np.uint16)
    (out,) = oracle.call("add_f16", 1 << 16, 1, meta_binary([1 << 16], [1], [1]), In(bits), In(zero), Out(1 << 16, "f16"))
    f = bits.view(np.float16)
    nan = np.isnan(f)
    keep = ~nan & (bits != 0x8000)                       # -0 + +0 = +0
    assert np.array_equal(out[keep], bits[keep])
    assert np.all(np.isnan(out[nan].view(np.float16)))
    assert out[0x8000] == 0
    # encode: products of random f16 pairs are exact in f32, so mul_f16 = encode(exact product); numpy rounds the same product
    r = rng(171)
    a = r.integers(0, 1 << 16, 1 << 20).astype(np.uint16)
    b = r.integers(0, 1 << 16, 1 << 20).astype(np.uint16)
    (m,) = oracle.call("mul_f16", a.size, 1, meta_binary([a.size], [1], [1]), In(a), In(b), Out(a.size, "f16"))
    with np.errstate(all="ignore"):
        want = (a.view(np.float16).astype(np.float32) * b.view(np.float16).astype(np.float32)).astype(np.float16)
    ok = ~np.isnan(want)
    assert np.array_equal(m[ok], want.view(np.uint16)[ok])           # overflow to inf, subnormals, ties to even
    assert np.all(np.isnan(m[~ok].view(np.float16)))


# ---- integers and bool: the oracle against exact (unbounded) integer arithmetic -------------------------------
def int_operands(dt, n=4096, seed=3):
    """Values that make every saturation and division case meet: the extremes, 0, +-1 and random fill."""
    info = np.iinfo(NP[dt])
    r = rng(seed)
    edge = [info.min, info.max, 0, 1, info.max - 1, info.min + 1, 2, 3] + ([-1, -2] if info.min < 0 else [])
    a = r.integers(info.min, info.max, n, dtype=NP[dt], endpoint=True)
    b = r.integers(info.min, info.max, n, dtype=NP[dt], endpoint=True)
    small = r.integers(max(info.min, -12), 12, n // 2, dtype=NP[dt])          # products and quotients that do not saturate
    a[: n // 2: 2] = small[: n // 4]
    b[1: n // 2: 2] = small[n // 4: n // 2]
    k = len(edge)
    grid_a, grid_b = np.repeat(np.array(edge, dtype=object), k), np.tile(np.array(edge, dtype=object), k)                     # every edge value against every edge value
    a[-k * k:], b[-k * k:] = grid_a.astype(NP[dt]), grid_b.astype(NP[dt])
    return a, b


@pytest.mark.parametrize("dt", ["u8", "u16", "u32", "u64", "i8", "i16", "i32", "i64"])
def test_oracle_integer_binary_ops_vs_exact_arithmetic(oracle, dt):
    info = np.iinfo(NP[dt])
    a, b = int_operands(dt)
    n = a.size
    A, B = [int(v) for v in a], [int(v) for v in b]                           # Python integers: exact
    clip = lambda v: min(max(v, info.min), info.max)

    def quotient(x, y):                                                      # truncation toward zero, then the clamp
        if y == 0:
            return 0 if x == 0 else (info.min if x < 0 else info.max)
        q = abs(x) // abs(y)
        return clip(q if (x < 0) == (y < 0) else -q)
    want = {"add": [clip(x + y) for x, y in zip(A, B)], "sub": [clip(x - y) for x, y in zip(A, B)],
            "mul": [clip(x * y) for x, y in zip(A, B)], "div": [quotient(x, y) for x, y in zip(A, B)],
            "maximum": [max(x, y) for x, y in zip(A, B)], "minimum": [min(x, y) for x, y in zip(A, B)]}
    md = meta_binary([n], [1], [1])
    for op, exp in want.items():
        (out,) = oracle.call(f"{op}_{dt}", n, 1, md, In(a), In(b), Out(n, dt))
        assert [int(v) for v in out] == exp, op
        if op in ("add", "sub", "mul", "div"):
            (acc,) = oracle.call(f"{op}_inplace_{dt}", n, 1, md, InOut(a.copy()), In(b))
            assert np.array_equal(acc, out), op
    cmp = {"eq": a == b, "ne": a != b, "lt": a < b, "le": a <= b, "gt": a > b, "ge": a >= b,
           "logical_and": (a != 0) & (b != 0), "logical_or": (a != 0) | (b != 0), "logical_xor": (a != 0) ^ (b != 0)}
    for op, exp in cmp.items():
        (out,) = oracle.call(f"{op}_{dt}", n, 1, md, In(a), In(b), Out(n, "bool"))
        assert np.array_equal(out.astype(bool), exp), op


def test_oracle_bool_binary_ops_truth_tables(oracle):
    a = np.array([0, 0, 1, 1], dtype=np.uint8)
    b = np.array([0, 1, 0, 1], dtype=np.uint8)
    md = meta_binary([4], [1], [1])
    # binary.rs:374 (add = or), :388 (sub = and), :402 (mul = xor), :457 (div = and), :584 (maximum = or), :598 (minimum = and)
    tables = {"add": a | b, "sub": a & b, "mul": a ^ b, "div": a & b, "maximum": a | b, "minimum": a & b,
              "eq": a == b, "ne": a != b, "lt": a < b, "le": a <= b, "gt": a > b, "ge": a >= b,
              "logical_and": a & b, "logical_or": a | b, "logical_xor": a ^ b}
    for op, exp in tables.items():
        (out,) = oracle.call(f"{op}_bool", 4, 1, md, In(a), In(b), Out(4, "bool"))
        assert out.tolist() == exp.astype(np.uint8).tolist(), op


def test_oracle_f64_binary_vs_numpy(oracle):
    r = rng(9)
    a, b = r.standard_normal(1000), r.standard_normal(1000)
    a[:6] = [0.0, 1.0, -2.0, np.nan, 0.0, 1e308]
    b[:6] = [0.0, 0.0, 0.0, 0.0, 3.0, 1e308]
    md = meta_binary([1000], [1], [1])
    with np.errstate(all="ignore"):
        want = {"add": a + b, "sub": a - b, "mul": a * b, "maximum": np.fmax(a, b), "minimum": np.fmin(a, b),
                "div": np.where(b == 0, np.where(a == 0, 0.0, np.inf), a / np.where(b == 0, 1.0, b))}
    for op, exp in want.items():
        (out,) = oracle.call(f"{op}_f64", 1000, 1, md, In(a), In(b), Out(1000, "f64"))
        assert np.array_equal(out, exp, equal_nan=True), op


# ---- dtype conversions: the oracle against exact arithmetic on Python numbers ----------------------------------------
def exact_cast(values, src, dst):
    """What Rust's `as` (towards bool: `!= 0`) gives, worked out with Python integers and numpy's IEEE conversions."""
    if dst == "bool":
        return [int(v != 0) for v in values.tolist()] if src not in ("f32", "f64") else [int(not (v == 0)) for v in values.tolist()]
    if dst in ("f32", "f64"):
        if src in ("f32", "f64"):
            with np.errstate(over="ignore"):
                return values.astype(NP[dst])                              # IEEE narrowing / widening
        # integer -> float: round to nearest even, from the exact integer (via the fractions module, independent of any C cast)
        from fractions import Fraction
        out = []
        for v in values.tolist():
            f = float(Fraction(int(v)))                                   # correctly rounded to binary64
            out.append(np.float32(f) if dst == "f32" else f)
        # (binary64 -> binary32 of an integer below 2^64 cannot double-round wrongly only if the first step was exact;
        #  integers above 2^53 are checked against the single rounding below instead)
        if dst == "f32":
            out = [np.float32(nearest_f32(int(v))) for v in values.tolist()]
        return np.array(out, dtype=NP[dst])
    info = np.iinfo(NP[dst])
    out = []
    for v in values.tolist():
        if src in ("f32", "f64"):
            if v != v:
                out.append(0)
            elif v in (float("inf"), float("-inf")):
                out.append(info.max if v > 0 else info.min)
            else:
                out.append(min(max(int(v), info.min), info.max))          # int() drops the fraction; then saturate
        else:
            out.append((int(v) - info.min) % (info.max - info.min + 1) + info.min)      # keep the low bits (two's complement)
    return out


def nearest_f32(i):
    """The binary32 nearest to the integer i, ties to even, by integer arithmetic alone."""
    if i == 0:
        return 0.0
    sign, m = (-1.0 if i < 0 else 1.0), abs(i)
    shift = max(m.bit_length() - 24, 0)
    q, rem = m >> shift, m & ((1 << shift) - 1)
    half = 1 << (shift - 1) if shift else 0
    if shift and (rem > half or (rem == half and (q & 1))):
        q += 1
    return sign * float(q) * 2.0 ** shift


@pytest.mark.parametrize("src", PLAIN)
def test_oracle_casts_vs_exact_arithmetic(oracle, src):
    x = cast_inputs(src)
    for dst in PLAIN:
        if dst == src:
            continue
        (out,) = oracle.call(f"cast_{src}_{dst}", x.size, In(x), Out(x.size, dst))
        want = exact_cast(x, src, dst)
        if dst in ("f32", "f64"):
            assert np.array_equal(out, np.asarray(want, dtype=NP[dst]), equal_nan=True), (src, dst)
        else:
            assert [int(v) for v in out] == list(want), (src, dst)


# ---- unary forms of the integers and bool: the oracle against exact arithmetic / numpy ------------------------------
@pytest.mark.parametrize("dt", ["u8", "u16", "u32", "u64", "i8", "i16", "i32", "i64"])
def test_oracle_integer_unary_vs_exact_arithmetic(oracle, dt):
    info = np.iinfo(NP[dt])
    x, _ = int_operands(dt)
    n, md = x.size, meta_unary([x.size], [1], 0)
    X = [int(v) for v in x]
    span = info.max - info.min + 1
    wrap = lambda v: (v - info.min) % span + info.min
    clip = lambda v: min(max(v, info.min), info.max)
    plain = {"sign": [(v > 0) - (v < 0) for v in X], "square": [wrap(v * v) for v in X]}
    if info.min < 0:
        plain["neg"] = [wrap(-v) for v in X]
        plain["abs"] = [wrap(abs(v)) for v in X]
    for op, exp in plain.items():
        (out,) = oracle.call(f"{op}_{dt}", n, 1, md, In(x), Out(n, dt))
        assert [int(v) for v in out] == exp, op
    # sqrt: numpy's correctly rounded float32 (int64: float64) square root of |x| (wrapped, so MIN stays negative -> NaN -> 0), then truncation
    ft = np.float64 if dt == "i64" else np.float32
    a = np.array([wrap(abs(v)) for v in X], dtype=object).astype(NP[dt])
    with np.errstate(invalid="ignore"):
        r = np.sqrt(a.astype(ft))
    want = [0 if v != v else min(int(v), info.max) for v in r.tolist()]
    (out,) = oracle.call(f"sqrt_{dt}", n, 1, md, In(x), Out(n, dt))
    assert [int(v) for v in out] == want
    (out,) = oracle.call(f"logical_not_{dt}", n, 1, md, In(x), Out(n, "bool"))
    assert np.array_equal(out.astype(bool), x == 0)
    for c in [0, 1, 3, info.max, info.min, info.max // 3] + ([-1, -7] if info.min < 0 else []):

        def quotient(v):
            if c == 0:
                return 0 if v == 0 else (info.min if v < 0 else info.max)
            q = abs(v) // abs(c)
            return clip(q if (v < 0) == (c < 0) else -q)
        const = {"add_scalar": [clip(v + c) for v in X], "sub_scalar": [clip(v - c) for v in X], "mul_scalar": [clip(v * c) for v in X],
                 "div_scalar": [quotient(v) for v in X], "maximum_scalar": [max(v, c) for v in X], "minimum_scalar": [min(v, c) for v in X]}
        for op, exp in const.items():
            (out,) = oracle.call(f"{op}_{dt}", n, 1, md, In(x), const_arg(c, dt), Out(n, dt))
            assert [int(v) for v in out] == exp, (op, c)
        cv = NP[dt](c)
        cmp = {"eq_scalar": x == cv, "ne_scalar": x != cv, "lt_scalar": x < cv, "le_scalar": x <= cv, "gt_scalar": x > cv, "ge_scalar": x >= cv}
        for op, exp in cmp.items():
            (out,) = oracle.call(f"{op}_{dt}", n, 1, md, In(x), const_arg(c, dt), Out(n, "bool"))
            assert np.array_equal(out.astype(bool), exp), (op, c)


def test_oracle_bool_unary_truth_tables(oracle):
    x = np.array([1, 0, 0, 1], dtype=np.uint8)                    # the reference's TEST_DATA_BOOL (ops_unary.rs)
    md = meta_unary([4], [1], 0)
    for op in ["abs", "sign", "square", "sqrt", "relu", "sigmoid", "tanh"]:
        (out,) = oracle.call(f"{op}_bool", 4, 1, md, In(x), Out(4, "bool"))
        assert out.tolist() == x.tolist(), op
    (out,) = oracle.call("neg_bool", 4, 1, md, In(x), Out(4, "bool"))
    assert out.tolist() == [0, 1, 1, 0]
    (out,) = oracle.call("logical_not_bool", 4, 1, md, In(x), Out(4, "bool"))
    assert out.tolist() == [0, 1, 1, 0]                           # ops_unary.rs:1036-1040
    for c in (0, 1):
        tables = {"add_scalar": x | c, "sub_scalar": x ^ c, "mul_scalar": x & c, "div_scalar": x & c, "maximum_scalar": x | c,
                  "minimum_scalar": x & c, "pow": x, "eq_scalar": x == c, "ne_scalar": x != c, "lt_scalar": x < c, "le_scalar": x <= c,
                  "gt_scalar": x > c, "ge_scalar": x >= c}
        for op, exp in tables.items():
            (out,) = oracle.call(f"{op}_bool", 4, 1, md, In(x), const_arg(c, "bool"), Out(4, "bool"))
            assert out.tolist() == np.asarray(exp).astype(np.uint8).tolist(), (op, c)


def test_oracle_integer_scalar_comparisons_match_reference_vectors(oracle):
    # ops_unary.rs: TEST_DATA_U32 = [1, 0, 2, 3]; eq/ne/lt/le_scalar(2), gt_scalar(1), logical_not (:1041-1046, 1472-1560)
    for dt in ["u8", "u16", "u32", "u64", "i8", "i16", "i32", "i64"]:
        x = np.array([1, 0, 2, 3], dtype=NP[dt])
        md = meta_unary([4], [1], 0)
        for op, c, exp in (("eq_scalar", 2, [0, 0, 1, 0]), ("ne_scalar", 2, [1, 1, 0, 1]), ("lt_scalar", 2, [1, 1, 0, 0]),
                           ("le_scalar", 2, [1, 1, 1, 0]), ("gt_scalar", 1, [0, 0, 1, 1])):
            (out,) = oracle.call(f"{op}_{dt}", 4, 1, md, In(x), const_arg(c, dt), Out(4, "bool"))
            assert out.tolist() == exp, (op, dt)
        (out,) = oracle.call(f"logical_not_{dt}", 4, 1, md, In(x), Out(4, "bool"))
        assert out.tolist() == [0, 1, 0, 0]


# ---- integer reductions: the oracle against numpy's wrapping sums and exact extrema -----------------------------------
@pytest.mark.parametrize("dt", ["u8", "u16", "u32", "u64", "i8", "i16", "i32", "i64"])
@pytest.mark.parametrize("shape,dim", [([7, 9], 0), ([7, 9], 1), ([4, 5, 6], 1), ([300], 0)])
def test_oracle_integer_reductions_vs_numpy(oracle, shape, dim, dt):
    info = np.iinfo(NP[dt])
    n = int(np.prod(shape))
    x = rng(5).integers(info.min, info.max, n, dtype=NP[dt], endpoint=True)         # sums overflow: they must wrap
    md = meta_reduce(shape, contiguous_strides(shape), dim, 0)
    xs = x.reshape(shape)
    with np.errstate(over="ignore"):
        want = {"sum": xs.sum(axis=dim, dtype=NP[dt]), "max": xs.max(axis=dim), "min": xs.min(axis=dim)}      # numpy integer sums wrap
    exact = np.asarray(np.array([int(v) for v in x], dtype=object).reshape(shape).sum(axis=dim), dtype=object).ravel()
    span = info.max - info.min + 1
    want = {k: np.asarray(v) for k, v in want.items()}
    assert [int(v) for v in want["sum"].ravel()] == [(int(v) - info.min) % span + info.min for v in exact]      # ... and equal the exact sum modulo 2^bits
    for op, exp in want.items():
        (out,) = oracle.call(f"{op}_{dt}", n, len(shape), 1, md, In(x), Out(n // shape[dim], dt))
        assert np.array_equal(out, exp.ravel()), op
    out_shape = [1 if d == dim else v for d, v in enumerate(shape)]
    (out,) = oracle.call(f"sum_to_shape_{dt}", n, len(shape), meta_sum_to_shape(shape, contiguous_strides(shape), out_shape, 0), In(x), Out(n // shape[dim], dt))
    assert np.array_equal(out, want["sum"].ravel())


# ---- matmul for the integers and f64: the oracle against exact integer products and a plain ascending loop ------------------
@pytest.mark.parametrize("dt", ["u8", "u16", "u32", "u64", "i8", "i16", "i32", "i64", "f64"])
@pytest.mark.parametrize("a_perm,b_perm", [(False, False), (True, True)])
def test_oracle_wide_matmul_vs_exact_products(oracle, dt, a_perm, b_perm):
    from helpers import meta_matmul
    batch, m, k, n = 2, 5, 7, 4
    r = rng(71)
    if dt == "f64":
        a, b = r.standard_normal((batch, m, k)), r.standard_normal((batch, k, n))
    else:
        info = np.iinfo(NP[dt])
        a = r.integers(info.min, info.max, (batch, m, k), dtype=NP[dt], endpoint=True)
        b = r.integers(info.min, info.max, (batch, k, n), dtype=NP[dt], endpoint=True)
    a_st, b_st = contiguous_strides([batch, m, k]), contiguous_strides([batch, k, n])
    sa, sb = a, b
    if a_perm:
        sa, a_st = np.ascontiguousarray(a.transpose(0, 2, 1)), [m * k, 1, m]
    if b_perm:
        sb, b_st = np.ascontiguousarray(b.transpose(0, 2, 1)), [k * n, 1, k]
    md = meta_matmul([batch, m, n], [batch, m, k], [batch, k, n], a_st, b_st)
    (out,) = oracle.call(f"matmul_{dt}", batch * m * n, md, In(sa.ravel()), In(sb.ravel()), Out(batch * m * n, dt))
    if dt == "f64":
        want = np.zeros((batch, m, n))
        for bi in range(batch):
            for i in range(m):
                for j in range(n):
                    acc = 0.0
                    for t in range(k):                       # ascending, multiply and add as two roundings
                        acc = acc + float(a[bi, i, t]) * float(b[bi, t, j])
                    want[bi, i, j] = acc
        assert np.array_equal(out.reshape(want.shape), want)
        return
    exact = np.einsum("bik,bkj->bij", a.astype(object), b.astype(object))           # Python integers: no overflow
    span = info.max - info.min + 1
    want = [(int(v) - info.min) % span + info.min for v in exact.ravel()]            # ... reduced modulo 2^bits
    assert [int(v) for v in out] == want
    # the two gradients are products of the same kind: dA = dC.B^T, dB = A^T.dC
    go = r.integers(info.min, info.max, (batch, m, n), dtype=NP[dt], endpoint=True)
    mdc = meta_matmul([batch, m, n], [batch, m, k], [batch, k, n], contiguous_strides([batch, m, k]), contiguous_strides([batch, k, n]))
    ga, gb = oracle.call(f"matmul_backward_{dt}", batch * m * k, batch * k * n, mdc, In(go.ravel()), In(a.ravel()), In(b.ravel()),
                         Out(batch * m * k, dt), Out(batch * k * n, dt))
    ea = np.einsum("bij,bkj->bik", go.astype(object), b.astype(object))
    eb = np.einsum("bik,bij->bkj", a.astype(object), go.astype(object))
    assert [int(v) for v in ga] == [(int(v) - info.min) % span + info.min for v in ea.ravel()]
    assert [int(v) for v in gb] == [(int(v) - info.min) % span + info.min for v in eb.ravel()]


# ---- integer pow -------------------------------------------------------------------------------------
def int_pow_model(x, c, dt):
    """`(x as f64).powf(c as f64) as T` from first principles, in Python's unbounded integers: the exact power (a
    fraction for c < 0), rounded to f64 as a correctly rounded pow returns it, truncated toward zero and clamped to the
    type like Rust's `as`.  64-bit operands are first rounded to f64 like the reference's own conversion."""
    from fractions import Fraction
    from helpers import NP
    info = np.iinfo(NP[dt])
    x, c = int(x), int(c)
    if info.bits == 64:
        x, c = int(float(x)), int(float(c))
    if c == 0:
        v = 1.0
    elif x == 0:
        v = float("inf") if c < 0 else 0.0
    elif abs(x) == 1:
        v = float(x) if c % 2 else 1.0
    elif c < 0:
        v = 0.0                                              # |x| >= 2: a fraction below 1 in magnitude
    elif c * (abs(x).bit_length() - 1) > 70:
        v = float("inf") if x > 0 or c % 2 == 0 else float("-inf")      # beyond 2^70: saturates whatever it is exactly
    else:
        v = float(Fraction(x) ** c)                          # Python rounds int -> float to nearest even
    if v != v:
        return 0
    if v >= float(info.max):
        return info.max
    if v <= float(info.min):
        return info.min
    return int(v)


@pytest.mark.parametrize("dt", ["u8", "i8"])
def test_oracle_integer_pow_exhaustive_8bit(oracle, dt):
    from helpers import NP
    info = np.iinfo(NP[dt])
    xs = np.arange(info.min, info.max + 1).astype(NP[dt])
    for c in range(info.min, info.max + 1):
        (o,) = oracle.call(f"pow_{dt}", xs.size, 1, meta_unary([xs.size], [1]), In(xs), int(c), Out(xs.size, dt))
        want = np.array([int_pow_model(x, c, dt) for x in xs], dtype=NP[dt])
        assert np.array_equal(o, want), c


def int_pow_cases(dt, r, n=400):
    """Bases and exponents around every place the result changes character: 0, +-1, +-2, the square, cube and higher
    roots of the type's bounds (one below, at, one above), powers of two, the bounds themselves, and random fill."""
    from helpers import NP
    info = np.iinfo(NP[dt])
    xs = {0, 1, 2, 3, info.max, info.max - 1, info.min, info.min + 1 if info.min < 0 else 1}
    for k in range(2, 64):
        root = int(round(info.max ** (1.0 / k)))
        for d in (-2, -1, 0, 1, 2):
            xs.add(max(0, root + d))
        xs.add(1 << min(k, info.bits - 2))
    if info.min < 0:
        xs |= {-v for v in xs if -v >= info.min}
    if info.bits == 64:
        xs |= {2 ** 53 - 1, 2 ** 53, 2 ** 53 + 1, 2 ** 53 + 3, 3037000499, 3037000500, 2642245, 2642246, 2 ** 32 - 1, 2 ** 32 + 1}
    xs = sorted(v for v in xs if info.min <= v <= info.max)
    xs = np.array(xs + list(r.integers(info.min, info.max, n, endpoint=True, dtype=NP[dt])), dtype=NP[dt])
    cs = sorted({0, 1, 2, 3, 4, 5, 7, 8, 15, 16, 31, 32, 33, 52, 53, 62, 63, 64, 65, 100, info.max} | ({-1, -2, -3, info.min} if info.min < 0 else set()))
    return xs, [c for c in cs if info.min <= c <= info.max]


@pytest.mark.parametrize("dt", ["u16", "i16", "u32", "i32", "u64", "i64"])
def test_oracle_integer_pow_on_boundary_sets(oracle, dt):
    from helpers import NP
    xs, cs = int_pow_cases(dt, rng(95))
    for c in cs:
        (o,) = oracle.call(f"pow_{dt}", xs.size, 1, meta_unary([xs.size], [1]), In(xs), int(c), Out(xs.size, dt))
        want = np.array([int_pow_model(x, c, dt) for x in xs], dtype=NP[dt])
        assert np.array_equal(o, want), c


@pytest.mark.parametrize("dt", ["u8", "i32", "u64", "bool"])
def test_oracle_integer_index_adds_wrap_and_bool_ors(oracle, dt):
    """index_add_ / scatter_add_ on the integer dtypes against numpy's wrapping add.at, on bool against logical_or.at
    (add_at_index, utils/indexing.rs:121-135)."""
    from helpers import NP, layout
    r = rng(99)
    vals = (lambda n: r.integers(0, 2, n).astype(np.uint8)) if dt == "bool" else (lambda n: r.integers(np.iinfo(NP[dt]).min, np.iinfo(NP[dt]).max, n, dtype=NP[dt], endpoint=True))
    shape, dim, n_idx = [5, 12, 4], 1, 30
    x = vals(int(np.prod(shape)))
    idx = r.integers(0, shape[dim], n_idx).astype(np.int32)
    src_shape = [5, n_idx, 4]
    src = vals(int(np.prod(src_shape)))
    (got,) = oracle.call(f"index_add_{dt}_i32", 3, dim, layout(shape), layout(src_shape), n_idx, 1, 0, In(idx), In(src), InOut(x.copy()))
    want = x.reshape(shape).copy()
    moved = np.moveaxis(want, dim, 0)
    with np.errstate(over="ignore"):
        (np.logical_or if dt == "bool" else np.add).at(moved, idx, np.moveaxis(src.reshape(src_shape), dim, 0))
    assert np.array_equal(got.reshape(shape), want)
    index = r.integers(0, shape[dim], src_shape).astype(np.int32)
    (got,) = oracle.call(f"scatter_add_{dt}_i32", 3, dim, layout(shape), layout(src_shape), layout(src_shape), In(index.ravel()), In(src), InOut(x.copy()))
    want = x.reshape(shape).copy()
    i0, _, i2 = np.meshgrid(np.arange(5), np.arange(n_idx), np.arange(4), indexing="ij")
    with np.errstate(over="ignore"):
        (np.logical_or if dt == "bool" else np.add).at(want, (i0.ravel(), index.ravel(), i2.ravel()), src)
    assert np.array_equal(got.reshape(shape), want)
