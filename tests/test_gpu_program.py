"""Recorded programs: a capture of small kernels replays as one interpreter launch (hip_graph_is_program == 1)
and must leave exactly the bytes the eager calls leave; anything larger or without an interpreter body must
fall back to a HIP graph and still replay correctly."""
import ctypes as C

import numpy as np
import pytest

import maidenx_amd._signatures as S
import maidenx_amd.lib as L

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def lib():
    if L.device_count() < 1:
        pytest.skip("no GPU")
    return L.load()


@pytest.fixture(autouse=True)
def without_resident_programs(lib):
    """These tests pin down whole-capture programs and fused chains; a capture they make would otherwise become a resident
    step program (tests/test_gpu_resident.py runs the same sequences that way)."""
    was = lib.hip_graph_set_resident(0)
    yield
    lib.hip_graph_set_resident(was)


def u64(*parts):
    out = []
    for x in parts:
        out += list(x) if isinstance(x, (list, tuple)) else [x]
    return np.array(out, dtype=np.uint64)


class Seq:
    """A list of backend calls on device buffers that can be run eagerly or inside a capture."""

    def __init__(self, lib):
        self.lib, self.calls, self.outs, self.keep = lib, [], [], []

    def dev(self, a):
        b = L.DeviceBuffer.from_numpy(np.ascontiguousarray(a))
        self.keep.append(b)
        return b

    def out(self, nbytes, dtype):
        b = L.DeviceBuffer(nbytes)
        self.keep.append(b)
        self.outs.append((b, nbytes, dtype))
        return b

    def add(self, name, *args):
        self.keep.append(args)
        self.calls.append((getattr(self.lib, "hip_" + name), args))

    def run(self):
        for fn, args in self.calls:
            fn(*[a.ctypes.data if isinstance(a, np.ndarray) else a for a in args])

    def clear_outputs(self):
        for b, n, dt in self.outs:
            if dt == "f4":
                self.lib.hip_fill_f32(n // 4, b.ptr, C.c_float(-7.0))
            elif dt == "u2":
                self.lib.hip_fill_bf16(n // 2, b.ptr, C.c_uint16(0x7FC0))
            else:
                self.lib.hip_fill_bool(n, b.ptr, C.c_uint8(9))
        assert self.lib.hip_synchronize() == 0

    def read(self):
        assert self.lib.hip_synchronize() == 0
        return [b.to_numpy(np.dtype(dt), n // np.dtype(dt).itemsize).copy() for b, n, dt in self.outs]


def replay_equals_eager(lib, seq, expect_program, replays=3):
    seq.run()
    eager = seq.read()
    assert lib.hip_get_last_status() == 0, lib.hip_status_string()
    seq.clear_outputs()
    assert lib.hip_graph_begin_capture() == 0
    seq.run()
    h = C.c_void_p()
    assert lib.hip_graph_end_capture(C.byref(h)) == 0
    try:
        # one launch of one work-group: a program, or (where those are allowed) the resident step program that replaces it
        one_launch = lib.hip_graph_is_program(h) == 1 or lib.hip_graph_is_resident(h, None, None) > 0
        assert one_launch == bool(expect_program)
        for _ in range(replays):
            seq.clear_outputs()          # eager work and a synchronisation between the replays
            assert lib.hip_graph_launch(h) == 0
            got = seq.read()
            for g, e in zip(got, eager):
                assert g.tobytes() == e.tobytes()
    finally:
        assert lib.hip_graph_destroy(h) == 0
    assert lib.hip_get_last_status() == 0, lib.hip_status_string()


def elementwise_sequence(lib, shape, rhs_strides, seed):
    """Every f32 elementwise entry point once, on the same operands (rhs optionally broadcast)."""
    r = np.random.default_rng(seed)
    n = int(np.prod(shape))
    a = r.standard_normal(n).astype(np.float32)
    a[::7] = 0.0
    b_full = r.standard_normal(n).astype(np.float32)
    b_full[::5] = 0.0
    seq = Seq(lib)
    da = seq.dev(a)
    cont = [int(np.prod(shape[i + 1:])) for i in range(len(shape))]
    if rhs_strides is None:
        rhs_strides, db = cont, seq.dev(b_full)
    else:
        extent = 1 + sum((d - 1) * s for d, s in zip(shape, rhs_strides))
        db = seq.dev(b_full[:extent])
    md2 = u64(list(shape), cont, list(rhs_strides), 0, 0)
    md1 = u64(list(shape), cont, 0)
    nd = len(shape)
    for op in S.BINARY:
        o = seq.out(n * (1 if op in S.BOOL_OUT else 4), "u1" if op in S.BOOL_OUT else "f4")
        seq.add(f"{op}_f32", n, nd, md2, da.ptr, db.ptr, o.ptr)
    for op in S.UNARY:
        o = seq.out(n * (1 if op in S.BOOL_OUT else 4), "u1" if op in S.BOOL_OUT else "f4")
        seq.add(f"{op}_f32", n, nd, md1, da.ptr, o.ptr)
    for op in S.UNARY_CONST:
        o = seq.out(n * (1 if op in S.BOOL_OUT else 4), "u1" if op in S.BOOL_OUT else "f4")
        seq.add(f"{op}_f32", n, nd, md1, da.ptr, C.c_float(0.5 if op != "pow" else 2.0), o.ptr)
    return seq


@pytest.mark.parametrize("shape,rhs_strides", [((1000,), None), ((37, 21), None), ((8, 128), (0, 1)), ((16, 64), (1, 0)), ((5, 3, 7), (0, 7, 1))],
                         ids=["vector", "odd", "row-bcast", "col-bcast", "3d-bcast"])
def test_every_f32_elementwise_op_replays_bit_exact(lib, shape, rhs_strides):
    replay_equals_eager(lib, elementwise_sequence(lib, shape, rhs_strides, 1), expect_program=True)


def test_dependent_chain_with_reductions_and_small_matmul(lib):
    """A training-step-like chain: matmul -> bias add -> loss -> reductions -> in-place update, every call reading what
    an earlier call of the same replay wrote."""
    r = np.random.default_rng(3)
    n, k = 200, 3
    seq = Seq(lib)
    x, w = seq.dev(r.standard_normal((n, k)).astype(np.float32)), seq.dev(r.standard_normal((k, 1)).astype(np.float32))
    bias, y = seq.dev(np.array([0.25], np.float32)), seq.dev(r.standard_normal(n).astype(np.float32))
    pred, pb, diff, sq = (seq.out(n * 4, "f4") for _ in range(4))
    loss, mx, mn, rows = seq.out(4, "f4"), seq.out(4, "f4"), seq.out(4, "f4"), seq.out(10 * 4, "f4")
    gw, wnew = seq.out(k * 4, "f4"), seq.out(k * 4, "f4")
    mm = u64(2, 2, 2, [n, 1], [n, k], [k, 1], [k, 1], [1, 1], 0, 0)
    seq.add("matmul_f32", n, mm, x.ptr, w.ptr, pred.ptr)
    seq.add("add_f32", n, 1, u64([n], [1], [0], 0, 0), pred.ptr, bias.ptr, pb.ptr)
    seq.add("sub_f32", n, 1, u64([n], [1], [1], 0, 0), pb.ptr, y.ptr, diff.ptr)
    seq.add("pow_f32", n, 1, u64([n], [1], 0), diff.ptr, C.c_float(2.0), sq.ptr)
    for name, o in (("mean", loss), ("max", mx), ("min", mn)):
        seq.add(f"{name}_f32", n, 1, 1, u64([n], [1], [n], [1], 0), sq.ptr, o.ptr)
    seq.add("sum_f32", n, 2, 1, u64([10, 20], [20, 1], [20], [1], 0), sq.ptr, rows.ptr)          # 10 rows of 20
    # gw[k,1] = x^T[k,n] . diff[n,1]  (a long reduction for few outputs when n is large; the per-thread kernel here)
    mt = u64(2, 2, 2, [k, 1], [k, n], [n, 1], [1, k], [1, 1], 0, 0)
    seq.add("matmul_f32", k, mt, x.ptr, diff.ptr, gw.ptr)
    seq.add("mul_scalar_f32", k, 1, u64([k], [1], 0), gw.ptr, C.c_float(0.01), wnew.ptr)
    seq.add("sub_inplace_f32", k, 1, u64([k], [1], [1], 0, 0), wnew.ptr, gw.ptr)
    replay_equals_eager(lib, seq, expect_program=True)


def test_block_dot_matmul_in_a_program(lib):
    r = np.random.default_rng(4)
    n = 4096
    seq = Seq(lib)
    x, g = seq.dev(r.standard_normal((n, 1)).astype(np.float32)), seq.dev(r.standard_normal(n).astype(np.float32))
    gw = seq.out(1 * 4, "f4")
    seq.add("matmul_f32", 1, u64(2, 2, 2, [1, 1], [1, n], [n, 1], [1, 1], [1, 1], 0, 0), x.ptr, g.ptr, gw.ptr)
    replay_equals_eager(lib, seq, expect_program=True)


def test_large_or_unsupported_captures_stay_hip_graphs(lib):
    r = np.random.default_rng(5)
    # a tensor beyond one pass of the interpreter's work-group
    n = 1 << 16
    seq = Seq(lib)
    a, o = seq.dev(r.standard_normal(n).astype(np.float32)), seq.out(n * 4, "f4")
    seq.add("neg_f32", n, 1, u64([n], [1], 0), a.ptr, o.ptr)
    replay_equals_eager(lib, seq, expect_program=False)
    # a small one next to a kernel without an interpreter body (column reduction), and a bf16 op
    seq = Seq(lib)
    a = seq.dev(r.standard_normal((32, 48)).astype(np.float32))
    o1, o2 = seq.out(32 * 48 * 4, "f4"), seq.out(48 * 4, "f4")
    seq.add("neg_f32", 32 * 48, 2, u64([32, 48], [48, 1], 0), a.ptr, o1.ptr)
    seq.add("sum_f32", 32 * 48, 2, 1, u64([32, 48], [48, 1], [32], [48], 0), o1.ptr, o2.ptr)
    replay_equals_eager(lib, seq, expect_program=False)
    seq = Seq(lib)
    h = seq.dev((r.standard_normal(512).astype(np.float32).view(np.uint32) >> 16).astype(np.uint16))
    o = seq.out(512 * 2, "u2")
    seq.add("neg_bf16", 512, 1, u64([512], [1], 0), h.ptr, o.ptr)
    replay_equals_eager(lib, seq, expect_program=False)
    # programs switched off
    was = lib.hip_graph_set_programs(0)
    try:
        replay_equals_eager(lib, elementwise_sequence(lib, (1000,), None, 2), expect_program=False, replays=1)
    finally:
        lib.hip_graph_set_programs(was)


def test_scratch_used_by_a_capture_survives_later_growth(lib):
    """A captured call that stages through the library's scratch block has that address in its graph.  A later eager
    call that needs a larger block must not free the old one while the capture is alive: replays still write there."""
    r = np.random.default_rng(7)
    small = r.standard_normal((64, 48)).astype(np.float32)
    seq = Seq(lib)
    a, o = seq.dev(small), seq.out(48 * 4, "f4")
    # sum over dim 0 of the transposed view of a [48, 64] buffer: gathered into scratch first
    seq.add("sum_to_shape_f32", 64 * 48, 2, u64([64, 48], [1, 64], [1, 48], 0), a.ptr, o.ptr)
    seq.run()
    (want,) = seq.read()
    assert lib.hip_graph_begin_capture() == 0
    seq.run()
    h = C.c_void_p()
    assert lib.hip_graph_end_capture(C.byref(h)) == 0
    try:
        # an eager call whose staging copy needs more than the 32 MB block
        n = 12 << 20
        big = L.DeviceBuffer.from_numpy(np.ones(n, np.float32))
        out = L.DeviceBuffer(3 * 4)
        lib.hip_sum_to_shape_f32(n, 2, u64([n // 3, 3], [1, n // 3], [1, 3], 0).ctypes.data, big.ptr, out.ptr)
        assert lib.hip_synchronize() == 0 and lib.hip_get_last_status() == 0
        assert out.to_numpy(np.float32).tolist() == [n // 3] * 3
        # allocations that would land in a freed block, filled with something else
        junk = [L.DeviceBuffer(8 << 20) for _ in range(6)]
        for j in junk:
            lib.hip_fill_f32((8 << 20) // 4, j.ptr, C.c_float(3.0))
        for _ in range(2):
            seq.clear_outputs()
            assert lib.hip_graph_launch(h) == 0
            (got,) = seq.read()
            assert got.tobytes() == want.tobytes()
        for j in junk:
            assert float(j.to_numpy(np.float32, 4)[0]) == 3.0
    finally:
        assert lib.hip_graph_destroy(h) == 0
    seq.clear_outputs()
    seq.run()
    (again,) = seq.read()
    assert again.tobytes() == want.tobytes() and lib.hip_get_last_status() == 0


# ---- fused runs of elementwise launches inside a capture ----------------------------------------------------------
def fused(lib, seq, want_launches=None, want_nodes=None, replays=2):
    """Captures `seq` (after a first launch that cannot be part of a program, so that fusion is active), checks the
    replays against the eager bytes and returns (fused launches, nodes)."""
    seq.run()
    eager = seq.read()
    assert lib.hip_get_last_status() == 0, lib.hip_status_string()
    big = L.DeviceBuffer(1 << 23)
    assert lib.hip_graph_begin_capture() == 0
    lib.hip_fill_f32((1 << 23) // 4, big.ptr, C.c_float(0.0))        # too large for a program command, and for a fused chain
    seq.run()
    h = C.c_void_p()
    assert lib.hip_graph_end_capture(C.byref(h)) == 0
    try:
        nodes = C.c_int()
        launches = lib.hip_graph_fused_launches(h, C.byref(nodes))
        assert lib.hip_graph_is_program(h) == 0
        for _ in range(replays):
            seq.clear_outputs()
            assert lib.hip_graph_launch(h) == 0
            got = seq.read()
            for k, (g, e) in enumerate(zip(got, eager)):
                assert g.tobytes() == e.tobytes(), k
    finally:
        assert lib.hip_graph_destroy(h) == 0
    assert lib.hip_get_last_status() == 0, lib.hip_status_string()
    if want_launches is not None:
        assert launches == want_launches, (launches, nodes.value)
    if want_nodes is not None:
        assert nodes.value == want_nodes, (launches, nodes.value)
    return launches, nodes.value


@pytest.mark.parametrize("n", [1, 3, 1000, 10000, 40004])
def test_fused_chain_of_dependent_ops(lib, n):
    """A chain in which every op reads what the one before wrote, element for element: one node."""
    r = np.random.default_rng(11)
    seq = Seq(lib)
    x, y = seq.dev(r.standard_normal(n).astype(np.float32)), seq.dev(r.standard_normal(n).astype(np.float32))
    outs = [seq.out(n * 4, "f4") for _ in range(7)]
    md1, md2 = u64([n], [1], 0), u64([n], [1], [1], 0, 0)
    seq.add("mul_f32", n, 1, md2, x.ptr, y.ptr, outs[0].ptr)
    seq.add("add_scalar_f32", n, 1, md1, outs[0].ptr, C.c_float(0.5), outs[1].ptr)
    seq.add("tanh_f32", n, 1, md1, outs[1].ptr, outs[2].ptr)
    seq.add("sub_f32", n, 1, md2, outs[2].ptr, x.ptr, outs[3].ptr)
    seq.add("pow_f32", n, 1, md1, outs[3].ptr, C.c_float(2.0), outs[4].ptr)
    seq.add("div_f32", n, 1, md2, outs[4].ptr, outs[1].ptr, outs[5].ptr)          # also reads an older member's output
    seq.add("add_inplace_f32", n, 1, md2, outs[5].ptr, y.ptr)                      # in place on the previous output
    seq.add("neg_f32", n, 1, md1, outs[5].ptr, outs[6].ptr)
    fused(lib, seq, want_launches=8, want_nodes=1)


def test_fused_groups_split_where_threads_would_meet(lib):
    """Overlaps that are not element for element must close the group: a broadcast of something the group wrote, a
    shifted view, a transposed read of a buffer the group then overwrites."""
    r = np.random.default_rng(12)
    n = 4096
    seq = Seq(lib)
    x = seq.dev(r.standard_normal(n).astype(np.float32))
    a, b, c, d, e = seq.out(n * 4, "f4"), seq.out(n * 4, "f4"), seq.out((n - 1) * 4, "f4"), seq.out(n * 4, "f4"), seq.out(n * 4, "f4")
    md1, md2 = u64([n], [1], 0), u64([n], [1], [1], 0, 0)
    seq.add("exp_f32", n, 1, md1, x.ptr, a.ptr)
    # element 0 of `a` broadcast to every element: written by another thread of the same group -> new group
    seq.add("mul_f32", n, 1, u64([n], [1], [0], 0, 0), x.ptr, a.ptr, b.ptr)
    # `b` shifted by one element (read after write across threads) -> new group
    seq.add("add_f32", n - 1, 1, u64([n - 1], [1], [1], 0, 1), x.ptr, b.ptr, c.ptr)
    # [64,64] transposed read of `c`'s buffer, then an overwrite of that buffer (write after read across threads)
    seq.add("mul_scalar_f32", n, 2, u64([64, 64], [64, 1], 0), b.ptr, C.c_float(2.0), d.ptr)        # same space as the next two
    seq.add("add_f32", n, 1, md2, d.ptr, x.ptr, e.ptr)
    seq.add("sub_f32", n, 1, md2, e.ptr, d.ptr, b.ptr)                                                # overwrites b: b was read element for element only
    launches, nodes = fused(lib, seq)
    assert launches == 6 and nodes == 4


def test_fused_two_dim_broadcast_and_a_reduction_in_between(lib):
    r = np.random.default_rng(13)
    rows, cols = 48, 200
    n = rows * cols
    seq = Seq(lib)
    x, row, col = seq.dev(r.standard_normal(n).astype(np.float32)), seq.dev(r.standard_normal(cols).astype(np.float32)), seq.dev(r.standard_normal(rows).astype(np.float32))
    a, b, s, c, d = seq.out(n * 4, "f4"), seq.out(n * 4, "f4"), seq.out(rows * 4, "f4"), seq.out(n * 4, "f4"), seq.out(n * 4, "f4")
    seq.add("add_f32", n, 2, u64([rows, cols], [cols, 1], [0, 1], 0, 0), x.ptr, row.ptr, a.ptr)       # + [1, cols]
    seq.add("mul_f32", n, 2, u64([rows, cols], [cols, 1], [1, 0], 0, 0), a.ptr, col.ptr, b.ptr)       # * [rows, 1]
    seq.add("sum_f32", n, 2, 1, u64([rows, cols], [cols, 1], [cols], [1], 0), b.ptr, s.ptr)            # a kernel node: the group before it runs first
    seq.add("sub_f32", n, 2, u64([rows, cols], [cols, 1], [1, 0], 0, 0), b.ptr, s.ptr, c.ptr)         # reads the reduction's result
    seq.add("relu_f32", n, 2, u64([rows, cols], [cols, 1], 0), c.ptr, d.ptr)
    launches, nodes = fused(lib, seq)
    assert launches == 4 and nodes == 3          # [add, mul], the reduction's kernel node, [sub], [relu: collapses to one dim]


def test_fused_tiny_members_of_any_shape_share_one_block(lib):
    """Members of at most 256 elements are run by one work-group with a barrier between them: different shapes, a
    broadcast of what the member before wrote, a shifted view and an in-place update all stay in one node."""
    r = np.random.default_rng(15)
    seq = Seq(lib)
    w, b = seq.dev(r.standard_normal(3).astype(np.float32)), seq.dev(r.standard_normal(1).astype(np.float32))
    x = seq.dev(r.standard_normal(200).astype(np.float32))
    gw, gb, t1, t2, t3, t4 = seq.out(3 * 4, "f4"), seq.out(4, "f4"), seq.out(200 * 4, "f4"), seq.out(199 * 4, "f4"), seq.out(12 * 16 * 4, "f4"), seq.out(3 * 4, "f4")
    seq.add("mul_scalar_f32", 3, 1, u64([3], [1], 0), w.ptr, C.c_float(0.01), gw.ptr)
    seq.add("mul_scalar_f32", 1, 1, u64([1], [1], 0), b.ptr, C.c_float(0.01), gb.ptr)
    seq.add("add_f32", 200, 1, u64([200], [1], [0], 0, 0), x.ptr, gb.ptr, t1.ptr)                  # broadcast of the member before
    seq.add("sub_f32", 199, 1, u64([199], [1], [1], 0, 1), x.ptr, t1.ptr, t2.ptr)                  # shifted view of it
    seq.add("mul_f32", 192, 2, u64([12, 16], [16, 1], [1, 12], 0, 0), t1.ptr, t2.ptr, t3.ptr)      # transposed read
    seq.add("sub_inplace_f32", 3, 1, u64([3], [1], [1], 0, 0), gw.ptr, w.ptr)
    seq.add("add_f32", 3, 1, u64([3], [1], [0], 0, 0), gw.ptr, gb.ptr, t4.ptr)
    fused(lib, seq, want_launches=7, want_nodes=1)


def linear_step(lib, seq, n, feats, r):
    """One training step of Linear(feats -> 1) + MSE + SGD spelled out in backend calls: a one-thread-per-output matmul,
    elementwise members over [n], a row reduction to a scalar, scalar stages, the weight gradient as a long-reduction
    matmul ([feats, n] x [n, 1], the left operand a transposed view) and the parameter updates."""
    x, y = seq.dev(r.standard_normal((n, feats)).astype(np.float32)), seq.dev(r.standard_normal(n).astype(np.float32))
    w, b = seq.dev(r.standard_normal(feats).astype(np.float32)), seq.dev(r.standard_normal(1).astype(np.float32))
    pred, pb, diff, sq = (seq.out(n * 4, "f4") for _ in range(4))
    loss, lossn, scale = seq.out(4, "f4"), seq.out(4, "f4"), seq.out(4, "f4")
    gpred, gx = seq.out(n * 4, "f4"), seq.out(n * feats * 4, "f4")
    gw, gb, wstep, bstep, wnew, bnew = (seq.out(k * 4, "f4") for k in (feats, 1, feats, 1, feats, 1))
    md1, md2 = u64([n], [1], 0), u64([n], [1], [1], 0, 0)
    # forward: x [n, feats] . w^T [feats, 1]
    seq.add("matmul_f32", n, u64(2, 2, 2, [n, 1], [n, feats], [feats, 1], [feats, 1], [1, feats], 0, 0), x.ptr, w.ptr, pred.ptr)
    seq.add("add_f32", n, 1, u64([n], [1], [0], 0, 0), pred.ptr, b.ptr, pb.ptr)
    seq.add("sub_f32", n, 1, md2, pb.ptr, y.ptr, diff.ptr)
    seq.add("square_f32", n, 1, md1, diff.ptr, sq.ptr)
    seq.add("sum_f32", n, 1, 1, u64([n], [1], [n], [1], 0), sq.ptr, loss.ptr)
    seq.add("div_scalar_f32", 1, 1, u64([1], [1], 0), loss.ptr, C.c_float(n), lossn.ptr)
    seq.add("fill_f32", 1, scale.ptr, C.c_float(2.0 / n))
    # backward: d loss / d pred, then the input gradient [n, 1] x [1, feats] (one term per output) ...
    seq.add("mul_f32", n, 1, u64([n], [1], [0], 0, 0), diff.ptr, scale.ptr, gpred.ptr)
    seq.add("matmul_f32", n * feats, u64(2, 2, 2, [n, feats], [n, 1], [1, feats], [1, 1], [feats, 1], 0, 0), gpred.ptr, w.ptr, gx.ptr)
    # ... the weight gradient x^T [feats, n] . gpred [n, 1], the bias gradient, and the updated parameters
    seq.add("matmul_f32", feats, u64(2, 2, 2, [feats, 1], [feats, n], [n, 1], [1, feats], [1, 1], 0, 0), x.ptr, gpred.ptr, gw.ptr)
    seq.add("sum_f32", n, 1, 1, u64([n], [1], [n], [1], 0), gpred.ptr, gb.ptr)
    seq.add("mul_scalar_f32", feats, 1, u64([feats], [1], 0), gw.ptr, C.c_float(0.01), wstep.ptr)
    seq.add("sub_f32", feats, 1, u64([feats], [1], [1], 0, 0), w.ptr, wstep.ptr, wnew.ptr)
    seq.add("mul_scalar_f32", 1, 1, u64([1], [1], 0), gb.ptr, C.c_float(0.01), bstep.ptr)
    seq.add("sub_f32", 1, 1, u64([1], [1], [1], 0, 0), b.ptr, bstep.ptr, bnew.ptr)


@pytest.mark.parametrize("n,feats", [(10000, 3), (4096, 4), (5000, 1), (12288, 2), (300, 3)])
def test_chain_with_matmuls_reductions_and_a_serial_tail(lib, n, feats):
    """A whole step becomes a few chains: matmul producers and elementwise members in the parallel phase, the sums, the
    long-reduction matmul and the scalar work in the tail of the group that finishes last.  Replays are the eager bytes."""
    r = np.random.default_rng(100 + n + feats)
    seq = Seq(lib)
    linear_step(lib, seq, n, feats, r)
    launches, nodes = fused(lib, seq, replays=3)
    if n >= 4096:
        assert launches == 15 and nodes <= 3, (launches, nodes)


def fused_nn_step(lib, seq, n, feats, r, seeded=True):
    """The step of linear_step() with the loss, its backward pass and the parameter updates as the fused calls; seeded:
    the gradient of the loss is a tensor filled with 1, else it is left out of the backward call (which then takes 1)."""
    x, y = seq.dev(r.standard_normal((n, feats)).astype(np.float32)), seq.dev(r.standard_normal(n).astype(np.float32))
    w0, b0 = r.standard_normal(feats).astype(np.float32), r.standard_normal(1).astype(np.float32)
    w, b = seq.out(feats * 4, "f4"), seq.out(4, "f4")          # updated in place: restored at the start of every run
    w_init, b_init = seq.dev(w0), seq.dev(b0)
    pred, pb, gpred = (seq.out(n * 4, "f4") for _ in range(3))
    loss, gloss, gw, gb = seq.out(4, "f4"), seq.out(4, "f4"), seq.out(feats * 4, "f4"), seq.out(4, "f4")
    seq.add("add_scalar_f32", feats, 1, u64([feats], [1], 0), w_init.ptr, C.c_float(0.0), w.ptr)
    seq.add("add_scalar_f32", 1, 1, u64([1], [1], 0), b_init.ptr, C.c_float(0.0), b.ptr)
    seq.add("matmul_f32", n, u64(2, 2, 2, [n, 1], [n, feats], [feats, 1], [feats, 1], [1, feats], 0, 0), x.ptr, w.ptr, pred.ptr)
    seq.add("add_f32", n, 1, u64([n], [1], [0], 0, 0), pred.ptr, b.ptr, pb.ptr)
    seq.add("mse_loss_f32", n, pb.ptr, y.ptr, loss.ptr)
    seq.add("fill_f32", 1, gloss.ptr, C.c_float(1.0))
    seq.add("mse_loss_backward_f32", n, pb.ptr, y.ptr, gloss.ptr if seeded else None, gpred.ptr, None)
    seq.add("matmul_f32", feats, u64(2, 2, 2, [feats, 1], [feats, n], [n, 1], [1, feats], [1, 1], 0, 0), x.ptr, gpred.ptr, gw.ptr)
    seq.add("sum_f32", n, 1, 1, u64([n], [1], [n], [1], 0), gpred.ptr, gb.ptr)
    seq.add("sgd_step_f32", feats, w.ptr, gw.ptr, C.c_float(0.01))
    seq.add("sgd_step_f32", 1, b.ptr, gb.ptr, C.c_float(0.01))


@pytest.mark.parametrize("n,feats", [(10000, 3), (4096, 4), (5001, 1), (65536, 2), (300, 3), (7, 2)])
def test_fused_loss_and_sgd_calls_join_the_chains(lib, n, feats):
    """hip_mse_loss_f32 (a stage of the serial phase), hip_mse_loss_backward_f32 (a member of the parallel phase whose
    scalar operand the stage before wrote: a new chain) and hip_sgd_step_f32 (an elementwise launch in place) inside a
    capture: every launch is taken by a chain and the replays are the eager bytes."""
    r = np.random.default_rng(300 + n + feats)
    seq = Seq(lib)
    fused_nn_step(lib, seq, n, feats, r)
    launches, nodes = fused(lib, seq, replays=3)
    if 4096 <= n <= 16384:           # (beyond that the weight gradient is a launch of its own: 1024 threads)
        assert launches == 11 and nodes <= 3, (launches, nodes)


@pytest.mark.parametrize("n,feats", [(10000, 3), (4096, 4), (5001, 1)])
def test_fused_loss_backward_without_a_seed_stays_in_the_forward_chain(lib, n, feats):
    """With no gradient tensor to wait for, the backward member meets the prediction element for element and is hoisted
    over the loss stage: the step is two chains (and the bytes of the seeded form)."""
    seqs = []
    for seeded in (True, False):
        seq = Seq(lib)
        fused_nn_step(lib, seq, n, feats, np.random.default_rng(300 + n + feats), seeded=seeded)
        launches, nodes = fused(lib, seq, replays=3)
        seqs.append((seq, nodes))
    assert seqs[1][1] == seqs[0][1] - 1, (seqs[0][1], seqs[1][1])
    for a, b in zip(seqs[0][0].read(), seqs[1][0].read()):
        assert a.tobytes() == b.tobytes()


def readme_step(lib, seq, n, feats, r):
    """The training step of the README example as the host layer issues it: fused_nn_step() without a seed, with the
    `0 + g` pass over the prediction's gradient, the input gradient [n,1] x [1,feats] and its accumulation."""
    x, y = seq.dev(r.standard_normal((n, feats)).astype(np.float32)), seq.dev(r.standard_normal(n).astype(np.float32))
    w0, b0 = r.standard_normal(feats).astype(np.float32), r.standard_normal(1).astype(np.float32)
    w, b = seq.out(feats * 4, "f4"), seq.out(4, "f4")
    w_init, b_init = seq.dev(w0), seq.dev(b0)
    pred, pb, gp0, gpred = (seq.out(n * 4, "f4") for _ in range(4))
    gx0, gx = seq.out(n * feats * 4, "f4"), seq.out(n * feats * 4, "f4")
    loss, gw, gb = seq.out(4, "f4"), seq.out(feats * 4, "f4"), seq.out(4, "f4")
    seq.add("add_scalar_f32", feats, 1, u64([feats], [1], 0), w_init.ptr, C.c_float(0.0), w.ptr)
    seq.add("add_scalar_f32", 1, 1, u64([1], [1], 0), b_init.ptr, C.c_float(0.0), b.ptr)
    seq.add("matmul_f32", n, u64(2, 2, 2, [n, 1], [n, feats], [feats, 1], [feats, 1], [1, feats], 0, 0), x.ptr, w.ptr, pred.ptr)
    seq.add("add_f32", n, 1, u64([n], [1], [0], 0, 0), pred.ptr, b.ptr, pb.ptr)
    seq.add("mse_loss_f32", n, pb.ptr, y.ptr, loss.ptr)
    seq.add("mse_loss_backward_f32", n, pb.ptr, y.ptr, None, gp0.ptr, None)
    seq.add("sum_to_shape_f32", n, 1, u64([n], [1], [n], 0), gp0.ptr, gpred.ptr)
    seq.add("sum_f32", n, 1, 1, u64([n], [1], [n], [1], 0), gpred.ptr, gb.ptr)
    seq.add("matmul_f32", n * feats, u64(2, 2, 2, [n, feats], [n, 1], [1, feats], [1, 1], [feats, 1], 0, 0), gpred.ptr, w.ptr, gx0.ptr)
    seq.add("sum_to_shape_f32", n * feats, 1, u64([n * feats], [1], [n * feats], 0), gx0.ptr, gx.ptr)
    seq.add("matmul_f32", feats, u64(2, 2, 2, [feats, 1], [feats, n], [n, 1], [1, feats], [1, 1], 0, 0), x.ptr, gpred.ptr, gw.ptr)
    seq.add("sgd_step_f32", feats, w.ptr, gw.ptr, C.c_float(0.01))
    seq.add("sgd_step_f32", 1, b.ptr, gb.ptr, C.c_float(0.01))


@pytest.mark.parametrize("n,feats", [(10000, 3), (4096, 4), (12288, 2), (5001, 2), (5003, 3), (300, 3), (1028, 4), (10000, 1), (10000, 5), (5002, 2)])
def test_input_gradient_of_a_one_output_layer_joins_the_step_as_a_wide_member(lib, n, feats):
    """[n,1] x [1,feats] over the rows a chain's own members wrote, and the pass that accumulates it, run in the same
    chain as the forward pass: work-group w, which staged rows [1024 w, 1024 w + 1024), also makes their feats-fold
    products.  The whole step is then one chain (the node before it restores the parameters)."""
    r = np.random.default_rng(500 + n + feats)
    seq = Seq(lib)
    readme_step(lib, seq, n, feats, r)
    launches, nodes = fused(lib, seq, replays=3)
    same_form = (n % 4 == 0) == (n * feats % 4 == 0)          # both spaces in 16-byte vectors, or both in elements
    if 2 <= feats <= 4 and 4096 <= n <= 16384 and same_form:
        assert launches == 13 and nodes == 2, (launches, nodes)
    if feats in (1, 5) or not same_form:          # as wide as the first space, too wide, or of the other form: a chain of its own
        assert nodes >= 3, (launches, nodes)


def test_wide_members_split_where_work_groups_would_meet(lib):
    """A member of the wide space runs with other work-groups' members of the first space still under way: apart from
    the rows of a one-term product it may not read what they write, nor write what they read or write."""
    n, m = 6000, 3
    r = np.random.default_rng(91)
    md1, mdw = u64([n], [1], 0), u64([n * m], [1], 0)
    outer = lambda: u64(2, 2, 2, [n, m], [n, 1], [1, m], [1, 1], [m, 1], 0, 0)

    def case(build, want_nodes):
        seq = Seq(lib)
        x, wide_in = seq.dev(r.standard_normal(n + 8).astype(np.float32)), seq.dev(r.standard_normal(n * m + 8).astype(np.float32))
        y3 = seq.dev(r.standard_normal(m).astype(np.float32))
        a, big, big2 = seq.out((n + 8) * 4, "f4"), seq.out((n * m + 8) * 4, "f4"), seq.out((n * m + 8) * 4, "f4")
        build(seq, x, wide_in, y3, a, big, big2)
        seq.clear_outputs()          # (no case writes every element of every buffer)
        launches, nodes = fused(lib, seq)
        assert nodes == want_nodes, (launches, nodes)

    def rows_of_own_group(seq, x, wide_in, y3, a, big, big2):
        seq.add("tanh_f32", n, 1, md1, x.ptr, a.ptr)
        seq.add("matmul_f32", n * m, outer(), a.ptr, y3.ptr, big.ptr)
        seq.add("mul_f32", n * m, 1, u64([n * m], [1], [1], 0, 0), big.ptr, wide_in.ptr, big2.ptr)
    case(rows_of_own_group, 1)

    def rows_from_memory(seq, x, wide_in, y3, a, big, big2):          # the left operand is nobody's output: read from memory
        seq.add("tanh_f32", n, 1, md1, x.ptr, a.ptr)
        seq.add("matmul_f32", n * m, outer(), x.ptr, y3.ptr, big.ptr)
    case(rows_from_memory, 1)

    def shifted_rows(seq, x, wide_in, y3, a, big, big2):              # rows 1 .. n of the output: another group's at the seams
        seq.add("tanh_f32", n + 1, 1, u64([n + 1], [1], 0), x.ptr, a.ptr)
        seq.add("matmul_f32", n * m, outer(), a.ptr + 4, y3.ptr, big.ptr)
    case(shifted_rows, 2)

    def elementwise_read_of_the_first_space(seq, x, wide_in, y3, a, big, big2):
        seq.add("tanh_f32", n, 1, md1, x.ptr, big.ptr)                 # writes big[0 .. n)
        seq.add("neg_f32", n * m, 1, mdw, big.ptr, big2.ptr)           # reads big[0 .. 3n)
    case(elementwise_read_of_the_first_space, 2)

    def write_over_what_the_first_space_reads(seq, x, wide_in, y3, a, big, big2):
        seq.add("tanh_f32", n, 1, md1, big.ptr + 4 * n, a.ptr)         # reads big[n .. 2n)
        seq.add("neg_f32", n * m, 1, mdw, wide_in.ptr, big.ptr)        # writes big[0 .. 3n)
    case(write_over_what_the_first_space_reads, 2)

    def write_over_what_the_first_space_writes(seq, x, wide_in, y3, a, big, big2):
        seq.add("tanh_f32", n, 1, md1, x.ptr, big.ptr)
        seq.add("neg_f32", n * m, 1, mdw, wide_in.ptr, big.ptr)
    case(write_over_what_the_first_space_writes, 2)

    def right_operand_written_by_the_first_space(seq, x, wide_in, y3, a, big, big2):
        seq.add("tanh_f32", n, 1, md1, x.ptr, a.ptr)
        seq.add("exp_f32", n, 1, md1, x.ptr, big2.ptr)
        seq.add("matmul_f32", n * m, outer(), a.ptr, big2.ptr + 16, big.ptr)
    case(right_operand_written_by_the_first_space, 2)

    def first_space_member_after_the_wide_ones(seq, x, wide_in, y3, a, big, big2):
        seq.add("tanh_f32", n, 1, md1, x.ptr, a.ptr)
        seq.add("matmul_f32", n * m, outer(), a.ptr, y3.ptr, big.ptr)
        seq.add("exp_f32", n, 1, md1, x.ptr, big2.ptr)                 # the first space is closed: a new chain
    case(first_space_member_after_the_wide_ones, 2)


@pytest.mark.parametrize("seed", range(16))
def test_fused_random_sequences_over_two_spaces(lib, seed):
    """Random launches over [n] and over [m n] - elementwise, one-term products [n,1] x [1,m], sums - on a small pool of
    buffers, so that operands overlap in every way: whatever the grouping decides, a replay leaves the eager bytes."""
    r = np.random.default_rng(4000 + seed)
    n = int(r.choice([300, 1024, 4096, 10000, 5001, 2052]))
    m = int(r.choice([2, 3, 4]))
    seq = Seq(lib)
    pool = [seq.out((n * m + 8) * 4, "f4") for _ in range(4)]
    src = [seq.dev(r.standard_normal(n * m + 8).astype(np.float32)) for _ in range(2)]
    for k, p in enumerate(pool):
        seq.add("add_scalar_f32", n * m + 8, 1, u64([n * m + 8], [1], 0), src[k % 2].ptr, C.c_float(0.25 * k), p.ptr)
    small = seq.out(64 * 4, "f4")
    seq.add("add_scalar_f32", 64, 1, u64([64], [1], 0), src[0].ptr, C.c_float(0.0), small.ptr)
    for _ in range(int(r.integers(4, 12))):
        kind = str(r.choice(["ew", "ew", "wide", "wide", "outer", "outer", "sum"]))
        oi = int(r.integers(0, len(pool)))
        others = [i for i in range(len(pool)) if i != oi]
        if kind in ("ew", "sum"):
            off = int(r.choice([0, 0, n, 1, 2 * n if m > 2 else n]))
            a_i = int(r.choice(others + [oi]))
            a_ptr = pool[a_i].ptr + 4 * (off if a_i == oi else int(r.choice([0, n, 3])))
            if kind == "sum":
                seq.add("sum_f32", n, 1, 1, u64([n], [1], [n], [1], 0), a_ptr, small.ptr + 4 * int(r.integers(0, 64)))
            elif r.random() < 0.5:
                seq.add(str(r.choice(["tanh_f32", "neg_f32", "square_f32"])), n, 1, u64([n], [1], 0), a_ptr, pool[oi].ptr + 4 * off)
            else:
                b_ptr = pool[int(r.choice(others))].ptr + 4 * int(r.choice([0, n]))
                seq.add(str(r.choice(["add_f32", "mul_f32"])), n, 1, u64([n], [1], [1], 0, 0), a_ptr, b_ptr, pool[oi].ptr + 4 * off)
        elif kind == "wide":
            a_i = int(r.choice(others + [oi]))
            a_ptr = pool[a_i].ptr + (0 if a_i == oi else 4 * int(r.choice([0, 0, 2])))
            if r.random() < 0.5:
                seq.add(str(r.choice(["neg_f32", "relu_f32"])), n * m, 1, u64([n * m], [1], 0), a_ptr, pool[oi].ptr)
            else:
                b_ptr = pool[int(r.choice(others))].ptr
                seq.add(str(r.choice(["add_f32", "sub_f32"])), n * m, 1, u64([n * m], [1], [1], 0, 0), a_ptr, b_ptr, pool[oi].ptr)
        else:
            xi = int(r.choice(others))
            x_ptr = pool[xi].ptr + 4 * int(r.choice([0, 0, 0, n, 1]))
            if r.random() < 0.5:
                y_ptr = small.ptr + 4 * int(r.integers(0, 60))
            else:
                y_ptr = pool[int(r.choice(others))].ptr + 4 * int(r.integers(0, n))
            seq.add("matmul_f32", n * m, u64(2, 2, 2, [n, m], [n, 1], [1, m], [1, 1], [m, 1], 0, 0), x_ptr, y_ptr, pool[oi].ptr)
    fused(lib, seq, replays=2)


def test_fused_loss_backward_waits_for_a_gradient_written_in_the_same_chain(lib):
    """The loss's gradient is read by every thread of the backward member: when an earlier member of the same space
    writes it (here: the buffer is a slice of a tensor the chain fills), the member must open a new chain; and a member
    that would overwrite it afterwards must not join either."""
    n = 4096
    r = np.random.default_rng(8)
    seq = Seq(lib)
    p, t = seq.dev(r.standard_normal(n).astype(np.float32)), seq.dev(r.standard_normal(n).astype(np.float32))
    g, gp, gp2 = seq.out(n * 4, "f4"), seq.out(n * 4, "f4"), seq.out(n * 4, "f4")
    md1 = u64([n], [1], 0)
    seq.add("add_scalar_f32", n, 1, md1, p.ptr, C.c_float(1.5), g.ptr)                     # writes g[0..n): g[5] is the "loss gradient"
    seq.add("mse_loss_backward_f32", n, p.ptr, t.ptr, g.ptr + 20, gp.ptr, None)
    seq.add("mul_scalar_f32", n, 1, md1, t.ptr, C.c_float(3.0), g.ptr)                     # overwrites it
    seq.add("mse_loss_backward_f32", n, p.ptr, t.ptr, g.ptr + 20, gp2.ptr, None)
    launches, nodes = fused(lib, seq, replays=3)
    assert launches == 4 and nodes == 4, (launches, nodes)


def test_chain_member_is_hoisted_over_tail_stages_only_when_independent(lib):
    """A member of the parallel phase that arrives after tail stages runs before them in the kernel: it is let in when it
    touches nothing they write and writes nothing they read, and opens a new chain otherwise."""
    r = np.random.default_rng(77)
    n = 6000
    seq = Seq(lib)
    x = seq.dev(r.standard_normal(n).astype(np.float32))
    a, s, t, b, c = seq.out(n * 4, "f4"), seq.out(4, "f4"), seq.out(4, "f4"), seq.out(n * 4, "f4"), seq.out(n * 4, "f4")
    md1, md2 = u64([n], [1], 0), u64([n], [1], [1], 0, 0)
    seq.add("tanh_f32", n, 1, md1, x.ptr, a.ptr)
    seq.add("sum_f32", n, 1, 1, u64([n], [1], [n], [1], 0), a.ptr, s.ptr)                   # tail
    seq.add("mul_scalar_f32", 1, 1, u64([1], [1], 0), s.ptr, C.c_float(0.5), t.ptr)        # tail
    seq.add("mul_f32", n, 1, md2, a.ptr, x.ptr, b.ptr)                                      # independent of the tail: hoisted
    seq.add("add_f32", n, 1, u64([n], [1], [0], 0, 0), b.ptr, t.ptr, c.ptr)                 # reads the tail's result: a new chain
    launches, nodes = fused(lib, seq)
    assert launches == 5 and nodes == 2, (launches, nodes)
    # ... and one that would overwrite what the reduction reads must not be hoisted either
    seq = Seq(lib)
    x = seq.dev(r.standard_normal(n).astype(np.float32))
    a, s = seq.out(n * 4, "f4"), seq.out(4, "f4")
    seq.add("exp_f32", n, 1, md1, x.ptr, a.ptr)
    seq.add("sum_f32", n, 1, 1, u64([n], [1], [n], [1], 0), a.ptr, s.ptr)
    seq.add("neg_f32", n, 1, md1, x.ptr, a.ptr)                                             # overwrites the sum's input
    launches, nodes = fused(lib, seq)
    assert launches == 3 and nodes == 2, (launches, nodes)


def test_chain_tail_reads_memory_late_when_no_mirror_holds_the_value(lib):
    """A tail stage whose input was written by two earlier stages (no single LDS mirror holds it), and one that writes
    across what two earlier stages wrote, wait for memory instead."""
    r = np.random.default_rng(78)
    seq = Seq(lib)
    x = seq.dev(r.standard_normal(64).astype(np.float32))
    xs = seq.dev(r.standard_normal(5000).astype(np.float32))
    big, halves, whole, across = seq.out(5000 * 4, "f4"), seq.out(64 * 4, "f4"), seq.out(64 * 4, "f4"), seq.out(32 * 4, "f4")
    seq.add("exp_f32", 5000, 1, u64([5000], [1], 0), xs.ptr, big.ptr)                                  # the parallel phase
    seq.add("mul_scalar_f32", 32, 1, u64([32], [1], 0), x.ptr, C.c_float(3.0), halves.ptr)             # halves[0:32]
    seq.add("mul_scalar_f32", 32, 1, u64([32], [1], 32), x.ptr, C.c_float(5.0), halves.ptr + 128)      # halves[32:64]
    seq.add("neg_f32", 64, 1, u64([64], [1], 0), halves.ptr, whole.ptr)                                # reads both
    seq.add("add_f32", 32, 1, u64([32], [1], [1], 16, 0), whole.ptr, x.ptr, halves.ptr + 64)           # writes halves[16:48]
    seq.add("sub_f32", 32, 1, u64([32], [1], [1], 0, 32), halves.ptr, halves.ptr, across.ptr)          # halves[0:32] - halves[32:64]
    launches, nodes = fused(lib, seq)
    assert launches == 6 and nodes == 1, (launches, nodes)


def test_fusion_can_be_switched_off(lib):
    r = np.random.default_rng(14)
    n = 1000
    seq = Seq(lib)
    x = seq.dev(r.standard_normal(n).astype(np.float32))
    a, b = seq.out(n * 4, "f4"), seq.out(n * 4, "f4")
    seq.add("exp_f32", n, 1, u64([n], [1], 0), x.ptr, a.ptr)
    seq.add("neg_f32", n, 1, u64([n], [1], 0), a.ptr, b.ptr)
    was = lib.hip_graph_set_fusion(0)
    try:
        fused(lib, seq, want_launches=0, want_nodes=0, replays=1)
    finally:
        lib.hip_graph_set_fusion(was)
    fused(lib, seq, want_launches=2, want_nodes=1, replays=1)


@pytest.mark.parametrize("seed", range(24))
def test_fused_random_sequences_with_aliasing(lib, seed):
    random_sequence_with_aliasing(lib, seed, resident=False)


def random_sequence_with_aliasing(lib, seed, resident):
    """Random chains over a small pool of buffers, with views that overlap in every way (same elements, shifted,
    broadcast, transposed, in place): whatever the grouping decides, a replay must leave the bytes of the eager run
    in every buffer.  resident: the capture holds nothing else and must become a resident step program."""
    r = np.random.default_rng(1000 + seed)
    n = int(r.choice([1, 3, 64, 200, 1024, 4096, 10000]))
    rows = int(r.choice([d for d in (1, 2, 4, 8, 16, 64) if n % d == 0]))
    cols = n // rows
    pool = [L.DeviceBuffer.from_numpy(r.standard_normal(n + 8).astype(np.float32)) for _ in range(5)]
    start = [p.to_numpy(np.float32).copy() for p in pool]
    esz = 4

    def view(kind, avoid=None):
        """(pointer, dims, strides) of a view into a random pool buffer, (buffer index) appended; `avoid`: a buffer the
        view must not touch unless it is the plain view of it (an op whose output overlaps its own input in any other
        way races with itself even as a single launch)"""
        bi = int(r.integers(0, len(pool)))
        if avoid is not None and bi == avoid and kind != "flat":
            bi = (bi + 1) % len(pool)
        b = pool[bi]
        if kind == "flat":
            return b.ptr, [n], [1]
        if kind == "shift":
            return b.ptr + esz * int(r.integers(1, 8)), [n], [1]
        if kind == "bcast":
            return b.ptr + esz * int(r.integers(0, 8)), [n], [0]
        if kind == "rowb":
            return b.ptr, [rows, cols], [0, 1]
        if kind == "colb":
            return b.ptr, [rows, cols], [1, 0]
        return b.ptr, [rows, cols], [1, rows]                      # transposed read of the same n elements

    calls = []
    for _ in range(int(r.integers(4, 14))):
        two_d = r.random() < 0.3
        out_i = int(r.integers(0, len(pool)))
        out_shift = 0 if r.random() < 0.8 else int(r.integers(1, 8))
        out_ptr = pool[out_i].ptr + esz * out_shift
        kinds = ["flat", "flat", "flat", "shift", "bcast"] + (["rowb", "colb", "tr"] if two_d else [])
        # inputs from other buffers, or exactly the output's own elements
        def operand():
            k = str(r.choice(kinds))
            v = view(k, avoid=out_i)
            if v[0] == pool[out_i].ptr and out_shift:          # the plain view of the output's buffer under a shifted output
                return (out_ptr, v[1], v[2])
            return v
        a, b = operand(), operand()
        dims = [rows, cols] if two_d else [n]
        full = lambda v: (v[2] if len(v[1]) == len(dims) else ([cols * v[2][0], v[2][0]] if two_d else v[2]))
        sa, sb = full(a), full(b)
        op = str(r.choice(["add", "mul", "sub", "neg", "relu", "mul_scalar", "add_inplace", "square"]))
        nd = len(dims)
        if op in ("add", "mul", "sub"):
            calls.append((f"{op}_f32", (n, nd, u64(dims, sa, sb, 0, 0), a[0], b[0], out_ptr)))
        elif op == "add_inplace":
            calls.append(("add_inplace_f32", (n, nd, u64(dims, [cols, 1] if two_d else [1], sb, 0, 0), out_ptr, b[0])))
        elif op == "mul_scalar":
            calls.append(("mul_scalar_f32", (n, nd, u64(dims, sa, 0), a[0], C.c_float(0.5), out_ptr)))
        else:
            calls.append((f"{op}_f32", (n, nd, u64(dims, sa, 0), a[0], out_ptr)))

    def run():
        for name, args in calls:
            getattr(lib, "hip_" + name)(*[x.ctypes.data if isinstance(x, np.ndarray) else x for x in args])

    def reset():
        for p, s in zip(pool, start):
            assert lib.hip_memcpy_h2d(p.ptr, s.ctypes.data, s.nbytes) == 0

    run()
    assert lib.hip_synchronize() == 0 and lib.hip_get_last_status() == 0, lib.hip_status_string()
    want = [p.to_numpy(np.float32).copy() for p in pool]
    big = L.DeviceBuffer(1 << 20)
    reset()
    assert lib.hip_graph_begin_capture() == 0
    if not resident:
        lib.hip_fill_f32((1 << 20) // 4, big.ptr, C.c_float(0.0))
    run()
    h = C.c_void_p()
    assert lib.hip_graph_end_capture(C.byref(h)) == 0
    try:
        assert (lib.hip_graph_is_resident(h, None, None) > 0) == resident
        for _ in range(2):
            reset()
            assert lib.hip_graph_launch(h) == 0 and lib.hip_synchronize() == 0
            for k, (p, w) in enumerate(zip(pool, want)):
                got = p.to_numpy(np.float32)
                assert got.tobytes() == w.tobytes(), (seed, k, n, [c[0] for c in calls])
    finally:
        assert lib.hip_graph_destroy(h) == 0
