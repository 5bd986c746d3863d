"""Resident step programs: a capture of small f32 launches is kept as a command list (nothing is launched while it is
recorded) and replayed by ONE work-group that holds the tensors in LDS.  Replays - one at a time or many in one launch -
must leave exactly the bytes the eager calls leave in every buffer that was not released."""
import ctypes as C

import numpy as np
import pytest

import maidenx_amd.lib as L
from test_gpu_program import Seq, elementwise_sequence, fused_nn_step, linear_step, random_sequence_with_aliasing, u64

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def lib():
    if L.device_count() < 1:
        pytest.skip("no GPU")
    return L.load()


@pytest.fixture(autouse=True)
def resident_programs_of_any_size(lib):
    """By default a capture stays a resident step program only while its tensors have at most 8192 elements (beyond that
    the fused chains are faster); these tests take the mechanism to its limits."""
    was = lib.hip_graph_set_resident(1 << 16)
    yield
    assert lib.hip_graph_set_resident(was) == 1 << 16


def resident_replay_equals_eager(lib, seq, expect=True, replays=3):
    seq.clear_outputs()                  # (elements no call writes hold the same thing in every run)
    seq.run()
    eager = seq.read()
    assert lib.hip_get_last_status() == 0, lib.hip_status_string()
    seq.clear_outputs()
    assert lib.hip_graph_begin_capture() == 0
    seq.run()
    h = C.c_void_p()
    assert lib.hip_graph_end_capture(C.byref(h)) == 0
    try:
        lds, bars = C.c_int(), C.c_int()
        cmds = lib.hip_graph_is_resident(h, C.byref(lds), C.byref(bars))
        assert (cmds > 0) == expect, cmds
        if expect:
            assert cmds == len(seq.calls) and lib.hip_graph_is_program(h) == 0
        for _ in range(replays):
            seq.clear_outputs()          # eager work and a synchronisation between the replays
            assert lib.hip_graph_launch(h) == 0
            got = seq.read()
            for k, (g, e) in enumerate(zip(got, eager)):
                assert g.tobytes() == e.tobytes(), k
    finally:
        assert lib.hip_graph_destroy(h) == 0
    assert lib.hip_get_last_status() == 0, lib.hip_status_string()
    return cmds, lds.value, bars.value


@pytest.mark.parametrize("n", [1, 3, 1000, 10000, 40004, 65536])
def test_dependent_elementwise_chain_needs_no_barrier(lib, n):
    """Every op reads what the one before wrote, element for element, some in place: the tensors stay in LDS and the
    only barrier of a replay is the one in front of it."""
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
    seq.add("div_f32", n, 1, md2, outs[4].ptr, outs[1].ptr, outs[5].ptr)
    seq.add("add_inplace_f32", n, 1, md2, outs[5].ptr, y.ptr)
    seq.add("neg_f32", n, 1, md1, outs[5].ptr, outs[6].ptr)
    cmds, lds, bars = resident_replay_equals_eager(lib, seq)
    assert cmds == 8 and bars == 1
    if n <= 4096:                                       # seven tensors of 16 KB fit the arena side by side
        assert lds >= 13


@pytest.mark.parametrize("shape,rhs_strides", [((1000,), None), ((37, 21), None), ((8, 128), (0, 1)), ((16, 64), (1, 0))],
                         ids=["vector", "odd", "row-bcast", "col-bcast"])
def test_every_f32_to_f32_elementwise_op(lib, shape, rhs_strides):
    """All f32 entry points on one pair of operands.  The comparisons (bool outputs) have no resident command: the first
    of them hands the capture to the fused chains and graph nodes, and the replay is still the eager bytes."""
    seq = elementwise_sequence(lib, shape, rhs_strides, 1)
    resident_replay_equals_eager(lib, seq, expect=False)
    f32_only = Seq(lib)
    f32_only.keep = seq.keep
    f32_only.outs = [o for o in seq.outs if o[2] == "f4"]
    keep = {o[0].ptr for o in f32_only.outs}
    f32_only.calls = [c for c in seq.calls if c[1][-1] in keep]
    cmds, lds, bars = resident_replay_equals_eager(lib, f32_only)
    assert cmds == len(f32_only.calls) >= 30


@pytest.mark.parametrize("n,feats", [(10000, 3), (4096, 4), (5000, 1), (12288, 2), (300, 3), (64, 2)])
def test_whole_training_step(lib, n, feats):
    """Linear(feats -> 1) + MSE + SGD spelled out in backend calls: the one-thread-per-output matmuls, elementwise
    launches over [n], sums to a scalar, the long-reduction weight gradient and scalar updates - one resident program."""
    r = np.random.default_rng(100 + n + feats)
    seq = Seq(lib)
    linear_step(lib, seq, n, feats, r)
    # (the weight gradient of 300 rows is a one-wave-per-output product: a command as well)
    cmds, lds, bars = resident_replay_equals_eager(lib, seq)
    assert cmds == 15


@pytest.mark.parametrize("n,feats", [(10000, 3), (4096, 4), (5001, 1), (64, 2), (7, 2)])
def test_training_step_with_the_fused_loss_and_sgd_calls(lib, n, feats):
    """The same step with hip_mse_loss_f32 (a command of its own: the eager kernel's one block run by the first 256
    threads), hip_mse_loss_backward_f32 without a gradient tensor (the seed of backward(): an elementwise functor) and
    hip_sgd_step_f32 (an elementwise functor in place): one resident program, the eager bytes."""
    r = np.random.default_rng(500 + n + feats)
    seq = Seq(lib)
    fused_nn_step(lib, seq, n, feats, r, seeded=False)
    cmds, lds, bars = resident_replay_equals_eager(lib, seq)
    assert cmds == 11


def test_a_seeded_loss_gradient_hands_the_capture_to_the_chains(lib):
    """hip_mse_loss_backward_f32 with a gradient tensor has no resident command: the launches kept so far go to the fused
    chains and the replay is still the eager bytes."""
    r = np.random.default_rng(9)
    seq = Seq(lib)
    fused_nn_step(lib, seq, 4096, 4, r, seeded=True)
    resident_replay_equals_eager(lib, seq, expect=False)


def training_loop(lib, n, feats, seed, discard):
    """A step with in-place parameter updates, so that one replay feeds the next."""
    r = np.random.default_rng(seed)
    seq = Seq(lib)
    x, y = seq.dev(r.standard_normal((n, feats)).astype(np.float32)), seq.dev(r.standard_normal(n).astype(np.float32))
    w, b = seq.out(feats * 4, "f4"), seq.out(4, "f4")
    w0, b0 = (r.standard_normal(feats) * 0.1).astype(np.float32), np.array([0.3], np.float32)
    pred, pb, diff, gpred = (seq.out(n * 4, "f4") for _ in range(4))
    scale, gw, gb, wstep, bstep = seq.out(4, "f4"), seq.out(feats * 4, "f4"), seq.out(4, "f4"), seq.out(feats * 4, "f4"), seq.out(4, "f4")
    md2 = u64([n], [1], [1], 0, 0)
    seq.add("matmul_f32", n, u64(2, 2, 2, [n, 1], [n, feats], [feats, 1], [feats, 1], [1, feats], 0, 0), x.ptr, w.ptr, pred.ptr)
    seq.add("add_f32", n, 1, u64([n], [1], [0], 0, 0), pred.ptr, b.ptr, pb.ptr)
    seq.add("sub_f32", n, 1, md2, pb.ptr, y.ptr, diff.ptr)
    seq.add("fill_f32", 1, scale.ptr, C.c_float(2.0 / n))
    seq.add("mul_f32", n, 1, u64([n], [1], [0], 0, 0), diff.ptr, scale.ptr, gpred.ptr)
    seq.add("matmul_f32", feats, u64(2, 2, 2, [feats, 1], [feats, n], [n, 1], [1, feats], [1, 1], 0, 0), x.ptr, gpred.ptr, gw.ptr)
    seq.add("sum_f32", n, 1, 1, u64([n], [1], [n], [1], 0), gpred.ptr, gb.ptr)
    seq.add("mul_scalar_f32", feats, 1, u64([feats], [1], 0), gw.ptr, C.c_float(0.05), wstep.ptr)
    seq.add("sub_inplace_f32", feats, 1, u64([feats], [1], [1], 0, 0), w.ptr, wstep.ptr)
    seq.add("mul_scalar_f32", 1, 1, u64([1], [1], 0), gb.ptr, C.c_float(0.05), bstep.ptr)
    seq.add("sub_inplace_f32", 1, 1, u64([1], [1], [1], 0, 0), b.ptr, bstep.ptr)
    temporaries = [pred, pb, diff, gpred, scale, wstep, bstep] if discard else []
    for t in temporaries:                                # released where a pool would release them: after their last use
        seq.add("buffer_discard", t.ptr, C.c_size_t(t.nbytes))

    def reset():
        assert lib.hip_memcpy_h2d(w.ptr, w0.ctypes.data, w0.nbytes) == 0 and lib.hip_memcpy_h2d(b.ptr, b0.ctypes.data, 4) == 0
        for t in (pred, pb, diff, gpred, scale, gw, gb, wstep, bstep):
            lib.hip_fill_f32(t.nbytes // 4, t.ptr, C.c_float(-7.0))
    kept = [i for i, (buf, _, _) in enumerate(seq.outs) if buf not in temporaries]
    return seq, reset, kept


@pytest.mark.parametrize("n,feats,discard", [(10000, 3, False), (10000, 3, True), (4096, 4, True), (50, 1, False)])
def test_many_replays_in_one_launch(lib, n, feats, discard):
    """hip_graph_launch_n: `times` passes over the command list in one launch, parameters staying in LDS between the
    passes, are `times` eager steps - bit for bit in everything that was not released."""
    seq, reset, kept = training_loop(lib, n, feats, 5, discard)
    for times in (1, 2, 7):
        reset()
        for _ in range(times):
            seq.run()
        want = seq.read()
        reset()
        assert lib.hip_graph_begin_capture() == 0
        seq.run()
        h = C.c_void_p()
        assert lib.hip_graph_end_capture(C.byref(h)) == 0
        try:
            assert lib.hip_graph_is_resident(h, None, None) == 11
            assert lib.hip_graph_launch_n(h, times) == 0
            got = seq.read()
            for k in kept:
                assert got[k].tobytes() == want[k].tobytes(), (times, k)
            # and once more on top, as single replays
            for _ in range(2):
                seq.run()
            want2 = seq.read()
            reset()
            assert lib.hip_graph_launch_n(h, times) == 0
            assert lib.hip_graph_launch(h) == 0 and lib.hip_graph_launch(h) == 0
            got2 = seq.read()
            for k in kept:
                assert got2[k].tobytes() == want2[k].tobytes(), (times, k)
        finally:
            assert lib.hip_graph_destroy(h) == 0
    assert lib.hip_get_last_status() == 0, lib.hip_status_string()


@pytest.mark.parametrize("n,feats", [(1000, 3), (5000, 3), (16000, 1), (12000, 3)])
def test_inputs_nothing_writes_are_read_again_at_every_launch(lib, n, feats):
    """The samples and the targets of a step - read by two or more commands, written by none - are copied into LDS when a
    launch starts (as long as they fit 64 KB of it; beyond that they stay in memory): data the host writes between two
    launches of the same program is what the second one computes on, and several passes of one launch see one copy."""
    r = np.random.default_rng(40 + n)
    seq = Seq(lib)
    xs = [r.standard_normal((n, feats)).astype(np.float32) for _ in range(2)]
    ys = [r.standard_normal(n).astype(np.float32) for _ in range(2)]
    x, y = seq.dev(xs[0]), seq.dev(ys[0])
    w, b = seq.out(feats * 4, "f4"), seq.out(4, "f4")
    w0, b0 = (r.standard_normal(feats) * 0.1).astype(np.float32), np.array([0.3], np.float32)
    pred, pb, gpred = (seq.out(n * 4, "f4") for _ in range(3))
    loss, gw, gb = seq.out(4, "f4"), seq.out(feats * 4, "f4"), seq.out(4, "f4")
    seq.add("matmul_f32", n, u64(2, 2, 2, [n, 1], [n, feats], [feats, 1], [feats, 1], [1, feats], 0, 0), x.ptr, w.ptr, pred.ptr)
    seq.add("add_f32", n, 1, u64([n], [1], [0], 0, 0), pred.ptr, b.ptr, pb.ptr)
    seq.add("mse_loss_f32", n, pb.ptr, y.ptr, loss.ptr)
    seq.add("mse_loss_backward_f32", n, pb.ptr, y.ptr, None, gpred.ptr, None)
    seq.add("matmul_f32", feats, u64(2, 2, 2, [feats, 1], [feats, n], [n, 1], [1, feats], [1, 1], 0, 0), x.ptr, gpred.ptr, gw.ptr)
    seq.add("sum_f32", n, 1, 1, u64([n], [1], [n], [1], 0), gpred.ptr, gb.ptr)
    seq.add("sgd_step_f32", feats, w.ptr, gw.ptr, C.c_float(0.05))
    seq.add("sgd_step_f32", 1, b.ptr, gb.ptr, C.c_float(0.05))

    def load(which):
        assert lib.hip_memcpy_h2d(x.ptr, xs[which].ctypes.data, xs[which].nbytes) == 0
        assert lib.hip_memcpy_h2d(y.ptr, ys[which].ctypes.data, ys[which].nbytes) == 0

    def reset():
        assert lib.hip_memcpy_h2d(w.ptr, w0.ctypes.data, w0.nbytes) == 0 and lib.hip_memcpy_h2d(b.ptr, b0.ctypes.data, 4) == 0

    # eager: three steps on the first data set, then two on the second
    seq.clear_outputs()
    reset()
    load(0)
    for _ in range(3):
        seq.run()
    load(1)
    for _ in range(2):
        seq.run()
    want = seq.read()
    assert lib.hip_get_last_status() == 0, lib.hip_status_string()
    seq.clear_outputs()
    reset()
    load(0)
    assert lib.hip_graph_begin_capture() == 0
    seq.run()
    h = C.c_void_p()
    assert lib.hip_graph_end_capture(C.byref(h)) == 0
    try:
        assert lib.hip_graph_is_resident(h, None, None) == len(seq.calls)
        assert lib.hip_graph_launch_n(h, 3) == 0
        load(1)
        assert lib.hip_graph_launch(h) == 0 and lib.hip_graph_launch(h) == 0
        got = seq.read()
        for k, (g, e) in enumerate(zip(got, want)):
            assert g.tobytes() == e.tobytes(), k
    finally:
        assert lib.hip_graph_destroy(h) == 0
    assert lib.hip_get_last_status() == 0, lib.hip_status_string()


def test_a_launch_of_another_kind_hands_the_capture_to_the_chains(lib):
    """A column reduction has no resident command: what was kept until then is fused or launched in order, the capture
    is a HIP graph, and the replay is the eager bytes."""
    r = np.random.default_rng(5)
    seq = Seq(lib)
    a = seq.dev(r.standard_normal((32, 48)).astype(np.float32))
    w = seq.dev(r.standard_normal((48, 2)).astype(np.float32))
    o1, o2, o3, o4 = seq.out(32 * 48 * 4, "f4"), seq.out(8 * 2 * 4, "f4"), seq.out(48 * 4, "f4"), seq.out(48 * 4, "f4")
    seq.add("neg_f32", 32 * 48, 2, u64([32, 48], [48, 1], 0), a.ptr, o1.ptr)
    # [8,48] x [48,2] on the first rows: 16 outputs of 48 terms, a product the chains refuse (it is launched when the
    # capture is handed over)
    seq.add("matmul_f32", 16, u64(2, 2, 2, [8, 2], [8, 48], [48, 2], [48, 1], [2, 1], 0, 0), o1.ptr, w.ptr, o2.ptr)
    seq.add("sum_f32", 32 * 48, 2, 1, u64([32, 48], [48, 1], [32], [48], 0), o1.ptr, o3.ptr)
    seq.add("exp_f32", 48, 1, u64([48], [1], 0), o3.ptr, o4.ptr)
    resident_replay_equals_eager(lib, seq, expect=False)
    # without the column reduction the same launches are a resident program, small product included
    seq.calls.pop(2)
    seq.outs = [o for o in seq.outs if o[0] is not o3]          # now an input: it keeps what the replays above left in it
    resident_replay_equals_eager(lib, seq, expect=True)


def test_a_tensor_beyond_the_arena_stays_in_memory(lib):
    """Three 64 KB tensors cannot all live in the 160 KB of LDS: whatever the plan leaves in memory is reached there."""
    r = np.random.default_rng(6)
    n = 16384
    seq = Seq(lib)
    x = seq.dev(r.standard_normal(n).astype(np.float32))
    a, b, c, d = (seq.out(n * 4, "f4") for _ in range(4))
    md1, md2 = u64([n], [1], 0), u64([n], [1], [1], 0, 0)
    seq.add("exp_f32", n, 1, md1, x.ptr, a.ptr)
    seq.add("neg_f32", n, 1, md1, a.ptr, b.ptr)
    seq.add("mul_f32", n, 1, md2, a.ptr, b.ptr, c.ptr)
    seq.add("add_f32", n - 4, 1, u64([n - 4], [1], [1], 0, 4), c.ptr, a.ptr, d.ptr)      # a shifted read of `a`: a barrier
    cmds, lds, bars = resident_replay_equals_eager(lib, seq)
    assert cmds == 4 and bars == 2


@pytest.mark.parametrize("seed", range(24))
def test_random_sequences_with_aliasing(lib, seed):
    random_sequence_with_aliasing(lib, seed, resident=True)


def test_switch_and_size_limit(lib):
    r = np.random.default_rng(14)

    def one(n):
        seq = Seq(lib)
        x = seq.dev(r.standard_normal(n).astype(np.float32))
        a = seq.out(4 * n, "f4")
        seq.add("exp_f32", n, 1, u64([n], [1], 0), x.ptr, a.ptr)
        return seq
    was = lib.hip_graph_set_resident(0)
    try:
        resident_replay_equals_eager(lib, one(100), expect=False, replays=1)
        assert lib.hip_graph_set_resident(8192) == 0          # the default limit
        resident_replay_equals_eager(lib, one(8192), expect=True, replays=1)
        resident_replay_equals_eager(lib, one(8196), expect=False, replays=1)
        assert lib.hip_graph_set_resident(1 << 20) == 8192 and lib.hip_graph_set_resident(5) == 1 << 16
    finally:
        lib.hip_graph_set_resident(was)
    resident_replay_equals_eager(lib, one(100), expect=True, replays=1)
