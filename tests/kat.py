"""Known-answer cases from the reference's own tests (tests/golden/reference_kat.json), runnable
against any Runner (CPU oracle or HIP backend).  Inputs are laid out as the reference's test
utilities lay them out: one pad element each side, offset 1 (tests/utils/mod.rs:12-21)."""
import json
import os

import numpy as np

from helpers import (In, InOut, Out, const_arg, contiguous_strides, layout, meta_binary, meta_matmul, meta_pad, meta_reduce,
                     meta_sum_to_shape, meta_unary, to_float, to_storage, u64, NP)

KAT = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "reference_kat.json")))


def padded(values, dt):
    """[0, values..., 0] storage; the logical tensor starts at offset 1."""
    v = np.concatenate([[0.0], np.asarray(values, dtype=np.float64).ravel(), [0.0]])
    return to_storage(v.astype(np.float32), dt)


def tol_for(dt, tol):
    # the reference asserts |Δ| < 0.1 for bf16/f16 (e.g. ops_binary.rs:28); these cases are exact
    # or nearly so in bf16 as well, so a bf16 rounding step of the expected value is allowed.
    return tol if dt not in ("bf16", "f16") else None


def check(actual_storage, expect, dt, tol):
    got = to_float(actual_storage, dt).astype(np.float64)
    exp = np.asarray(expect, dtype=np.float64)
    if dt in ("bf16", "f16"):
        # value must be the bf16 rounding of something within 1 bf16 ulp of the expectation
        # (the reference itself only asserts |Δ| < 0.1 for bf16, e.g. ops_binary.rs:28)
        lim = np.abs(exp) * 2.0 ** -7 + tol
        assert np.all(np.abs(got - exp) <= lim), (got, exp)
    elif tol == 0:
        assert np.array_equal(got.astype(np.float32), exp.astype(np.float32)), (got, exp)
    else:
        assert np.all(np.abs(got - exp) < tol), (got, exp)


def run_binary(be, dt):
    for c in KAT["binary"]:
        n = len(c["lhs"])
        md = meta_binary([n], [1], [1], 1, 1)
        (out,) = be.call(f"{c['op']}_{dt}", n, 1, md, In(padded(c["lhs"], dt)), In(padded(c["rhs"], dt)), Out(n, dt))
        check(out, c["expect"], dt, 0)


def run_compare(be, dt):
    for c in KAT["compare"]:
        n = len(c["lhs"])
        md = meta_binary([n], [1], [1], 1, 1)
        (out,) = be.call(f"{c['op']}_{dt}", n, 1, md, In(padded(c["lhs"], dt)), In(padded(c["rhs"], dt)), Out(n, "bool"))
        assert out.tolist() == c["expect"], (c["op"], out)


def run_inplace(be, dt):
    for c in KAT["inplace"]:
        n = len(c["lhs"])
        md = meta_binary([n], [1], [1], 1, 1)
        (lhs,) = be.call(f"{c['op']}_{dt}", n, 1, md, InOut(padded(c["lhs"], dt)), In(padded(c["rhs"], dt)))
        check(lhs[1:-1], c["expect"], dt, 0)
        assert to_float(lhs, dt)[0] == 0 and to_float(lhs, dt)[-1] == 0     # neighbours untouched


INT_DTYPES = ["u8", "u16", "u32", "u64", "i8", "i16", "i32", "i64"]


def padded_int(values, dt):
    return np.concatenate([[0], np.asarray(values), [0]]).astype(NP[dt])


def run_binary_wide(be, dt):
    """The integer and bool branches of the reference's binary tests (sections *_int, compare_bool)."""
    md_of = lambda n: meta_binary([n], [1], [1], 1, 1)
    if dt == "bool":
        for c in KAT["compare_bool"]:
            n = len(c["lhs"])
            (out,) = be.call(f"{c['op']}_bool", n, 1, md_of(n), In(padded_int(c["lhs"], dt)), In(padded_int(c["rhs"], dt)), Out(n, "bool"))
            assert out.tolist() == c["expect"], (c["op"], out)
        return
    for c in KAT["binary_int"]:
        n = len(c["lhs"])
        (out,) = be.call(f"{c['op']}_{dt}", n, 1, md_of(n), In(padded_int(c["lhs"], dt)), In(padded_int(c["rhs"], dt)), Out(n, dt))
        assert out.tolist() == c["expect"], (c["op"], dt, out)
    for c in KAT["compare_int"]:
        n = len(c["lhs"])
        (out,) = be.call(f"{c['op']}_{dt}", n, 1, md_of(n), In(padded_int(c["lhs"], dt)), In(padded_int(c["rhs"], dt)), Out(n, "bool"))
        assert out.tolist() == c["expect"], (c["op"], dt, out)
    for c in KAT["inplace_int"]:
        n = len(c["lhs"])
        (lhs,) = be.call(f"{c['op']}_{dt}", n, 1, md_of(n), InOut(padded_int(c["lhs"], dt)), In(padded_int(c["rhs"], dt)))
        assert lhs.tolist() == [0] + c["expect"] + [0], (c["op"], dt, lhs)


def run_unary(be, dt):
    for c in KAT["unary"]:
        n = len(c["x"])
        md = meta_unary([n], [1], 1)
        (out,) = be.call(f"{c['op']}_{dt}", n, 1, md, In(padded(c["x"], dt)), Out(n, dt))
        check(out, c["expect"], dt, c["tol"])
    for c in KAT["unary_bool"]:
        n = len(c["x"])
        (out,) = be.call(f"{c['op']}_{dt}", n, 1, meta_unary([n], [1], 1), In(padded(c["x"], dt)), Out(n, "bool"))
        assert out.tolist() == c["expect"]


def run_unary_const(be, dt):
    for c in KAT["unary_const"]:
        n = len(c["x"])
        md = meta_unary([n], [1], 1)
        (out,) = be.call(f"{c['op']}_{dt}", n, 1, md, In(padded(c["x"], dt)), const_arg(c["c"], dt), Out(n, dt))
        check(out, c["expect"], dt, c["tol"])
    for c in KAT["unary_const_bool"]:
        n = len(c["x"])
        (out,) = be.call(f"{c['op']}_{dt}", n, 1, meta_unary([n], [1], 1), In(padded(c["x"], dt)), const_arg(c["c"], dt),
                         Out(n, "bool"))
        assert out.tolist() == c["expect"], c["op"]


def reduce_once(be, op, dt, storage, shape, strides, dim, off):
    n = int(np.prod(shape))
    md = meta_reduce(shape, strides, dim, off)
    (out,) = be.call(f"{op}_{dt}", n, len(shape), 1, md, In(storage), Out(n // shape[dim], dt))
    return out


def run_reduce(be, dt):
    for c in KAT["reduce"]:
        shape = c["shape"]
        out = reduce_once(be, c["op"], dt, padded(c["data"], dt), shape, contiguous_strides(shape), c["dim"], 1)
        check(out, c["expect"], dt, 0)
    # *_all = chain over dims from the last to the first (tensor/ops/reduction.rs:76-83)
    for c in KAT["reduce_all"]:
        shape = list(c["shape"])
        cur, off = padded(c["data"], dt), 1
        for dim in reversed(range(len(shape))):
            cur = reduce_once(be, c["op"], dt, cur, shape, contiguous_strides(shape), dim, off)
            off = 0
            shape.pop(dim)
            if not shape:
                break
        check(cur, [c["expect"]], dt, 0)


def run_sum_to_shape(be, dt):
    for c in KAT["sum_to_shape"]:
        shape = c["shape"]
        n = int(np.prod(shape))
        md = meta_sum_to_shape(shape, contiguous_strides(shape), c["out_shape"], 1)
        (out,) = be.call(f"sum_to_shape_{dt}", n, len(shape), md, In(padded(c["data"], dt)), Out(int(np.prod(c["out_shape"])), dt))
        check(out, c["expect"], dt, 0)


def prepare_matmul_metadata(a_shape, a_strides, a_off, b_shape, b_strides, b_off):
    """crates/maidenx_tensor/src/ops/matmul.rs:227-264."""
    a_shape, b_shape, a_strides, b_strides = list(a_shape), list(b_shape), list(a_strides), list(b_strides)
    if len(a_shape) == 1:
        a_shape.insert(0, 1)
        a_strides.insert(0, a_strides[0] * a_shape[1])
    if len(b_shape) == 1:
        b_shape.append(1)
        b_strides.append(1)
    out_ndim = len(a_shape)
    out_shape = a_shape[:out_ndim - 2] + [a_shape[out_ndim - 2], b_shape[out_ndim - 1]]
    return meta_matmul(out_shape, a_shape, b_shape, a_strides, b_strides, a_off, b_off), out_shape


def run_matmul(be, dt):
    for c in KAT["matmul"]:
        a_shape, b_shape = c["a_shape"], c["b_shape"]
        md, out_shape = prepare_matmul_metadata(a_shape, contiguous_strides(a_shape), 1, b_shape, contiguous_strides(b_shape), 1)
        n_out = int(np.prod(out_shape))
        a, b = padded(c["a"], dt), padded(c["b"], dt)
        (out,) = be.call(f"matmul_{dt}", n_out, md, In(a), In(b), Out(n_out, dt))
        check(out, c["c"], dt, 0)
        go = to_storage(np.ones(n_out, dtype=np.float32), dt)          # backward() seeds ones_like
        na, nb = len(c["a"]), len(c["b"])
        ga, gb = be.call(f"matmul_backward_{dt}", na, nb, md, In(go), In(a), In(b), Out(na, dt), Out(nb, dt))
        check(ga, c["grad_a"], dt, 0)
        check(gb, c["grad_b"], dt, 0)


def run_pad(be, dt):
    for c in KAT["pad"]:
        shape, pads = c["shape"], c["pads"]
        out_shape = [s + p[0] + p[1] for s, p in zip(shape, pads)]
        n_in, n_out = int(np.prod(shape)), int(np.prod(out_shape))
        md = meta_pad(shape, contiguous_strides(shape), 1, out_shape, pads)
        (out,) = be.call(f"pad_with_constant_{dt}", n_in, n_out, len(shape), md, In(padded(c["data"], dt)), Out(n_out, dt),
                         const_arg(c["value"], dt))
        exp = to_float(to_storage(np.array(c["expect"], dtype=np.float64), dt), dt)
        assert np.array_equal(to_float(out, dt), exp)
        go = to_storage(np.ones(n_out, dtype=np.float32), dt)
        gi = padded(np.full(n_in, 7.0), dt)                              # stale contents must be overwritten
        (gi,) = be.call(f"pad_with_constant_backward_{dt}", n_in, n_out, len(shape), md, In(go), InOut(gi))
        check(gi[1:-1], c["grad"], dt, 0)


def run_pad_edge(be, dt):
    for c in KAT["pad_edge"]:
        shape, pads = c["shape"], c["pads"]
        out_shape = [s + p[0] + p[1] for s, p in zip(shape, pads)]
        n_in, n_out = int(np.prod(shape)), int(np.prod(out_shape))
        md = meta_pad(shape, contiguous_strides(shape), 1, out_shape, pads)
        (out,) = be.call(f"pad_with_{c['mode']}_{dt}", n_in, n_out, len(shape), md, In(padded(c["data"], dt)), Out(n_out, dt))
        assert np.array_equal(to_float(out, dt), np.array(c["expect"], dtype=np.float32))
        if "grad" in c:
            go = to_storage(np.ones(n_out, dtype=np.float32), dt)
            gi = padded(np.full(n_in, 7.0), dt)
            (gi,) = be.call(f"pad_with_{c['mode']}_backward_{dt}", n_in, n_out, len(shape), md, In(go), InOut(gi))
            check(gi[1:-1], c["grad"], dt, 0)


def run_fold(be, dt):
    for c in KAT["fold"]:
        dims = c["dims"]
        n = int(np.prod(dims))
        md = u64(dims, c["strides"], c["fold_dim"], c["window_dim"], c["fold_size"], c["step"], dims[c["window_dim"]], 1)
        # the unfolded view shares the 5- or 6-element buffer; the kernel may index up to num_els of it
        data = np.concatenate([padded(c["data"], dt), to_storage(np.zeros(n, np.float32), dt)])
        (out,) = be.call(f"fold_{dt}", n, len(dims), md, In(data), Out(len(c["expect"]), dt))
        check(out, c["expect"], dt, 0)


def run_softmax(be, dt):
    for c in KAT["softmax"]:
        shape = c["shape"]
        n = int(np.prod(shape))
        md = meta_unary(shape, contiguous_strides(shape), 1)
        (out,) = be.call(f"softmax_{dt}", n, len(shape), c["dim"], md, In(padded(c["data"], dt)), Out(n, dt))
        y = to_float(out, dt).astype(np.float64).reshape(shape)
        tol = 1e-5 if dt not in ("bf16", "f16") else 2e-2
        assert np.all(np.abs(y.sum(axis=c["dim"]) - 1.0) < tol), y
        assert np.all(np.diff(y, axis=c["dim"]) > 0), y


def run_index(be, dt):
    # the reference's test tensors carry offset 1 (tests/utils/mod.rs:12-21); index tensors are i32
    for it in ("i32", "i64"):
        ity = np.int32 if it == "i32" else np.int64
        for c in KAT["index"]:
            op = c["op"]
            if op == "index_select":
                shape, dim = c["shape"], c["dim"]
                idx = np.array([0] + c["indices"], dtype=ity)
                n_out = len(c["expect"])
                (out,) = be.call(f"index_select_{dt}_{it}", len(shape), dim, layout(shape, off=1), len(c["indices"]), 1, 1, In(idx),
                                 In(padded(c["data"], dt)), Out(n_out, dt))
                check(out, c["expect"], dt, 0)
            elif op == "gather":
                shape, ishape = c["shape"], c["index_shape"]
                idx = np.array([0] + c["index"], dtype=ity)
                (out,) = be.call(f"gather_{dt}_{it}", len(shape), c["dim"], layout(shape, off=1), layout(ishape, off=1), In(idx),
                                 In(padded(c["data"], dt)), Out(len(c["expect"]), dt))
                check(out, c["expect"], dt, 0)
            elif op == "index_add":
                shape, sshape = c["self_shape"], c["src_shape"]
                idx = np.array([0] + c["indices"], dtype=ity)
                (out,) = be.call(f"index_add_{dt}_{it}", len(shape), c["dim"], layout(shape, off=1), layout(sshape, off=1),
                                 len(c["indices"]), 1, 1, In(idx), In(padded(c["src"], dt)), InOut(padded(c["self"], dt)))
                check(out[1:-1], c["expect"], dt, 0)
            elif op == "scatter_add":
                shape, ishape = c["self_shape"], c["index_shape"]
                idx = np.array([0] + c["index"], dtype=ity)
                (out,) = be.call(f"scatter_add_{dt}_{it}", len(shape), c["dim"], layout(shape, off=1), layout(ishape, off=1),
                                 layout(ishape, off=1), In(idx), In(padded(c["src"], dt)), InOut(padded(c["self"], dt)))
                check(out[1:-1], c["expect"], dt, 0)
            elif op == "index_put":
                if it == "i64":
                    continue                      # no index tensor: once is enough
                shape, sshape = c["self_shape"], c["src_shape"]
                (out,) = be.call(f"index_put_{dt}", len(shape), layout(shape, off=1), len(c["indices"]), np.array(c["indices"], dtype=np.uint64),
                                 len(sshape), layout(sshape, off=1), In(padded(c["src"], dt)), InOut(padded(c["self"], dt)))
                check(out[1:-1], c["expect"], dt, 0)
            elif op == "bincount":
                idx = np.array([0] + c["input"], dtype=ity)
                (out,) = be.call(f"bincount_{it}", len(c["input"]), 1, 1, In(idx), c["out_size"], Out(c["out_size"], it))
                assert out.tolist() == c["expect"]
            elif op == "bincount_weighted":
                idx = np.array([0] + c["input"], dtype=ity)
                (out,) = be.call(f"bincount_weighted_{dt}_{it}", len(c["input"]), 1, 1, In(idx), 1, 1, In(padded(c["weights"], dt)),
                                 c["out_size"], Out(c["out_size"], dt))
                check(out, c["expect"], dt, 0)


ALL = [run_index, run_pad_edge, run_fold, run_softmax, run_binary, run_compare, run_inplace, run_unary, run_unary_const, run_reduce, run_sum_to_shape, run_matmul, run_pad]
