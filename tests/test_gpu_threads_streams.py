"""Host threads and caller-set streams.

The reference's buffers are Send + Sync (crates/maidenx_core/src/buffer/mod.rs:36) and every dispatch is a plain
function call, so two Rust threads can call into the backend at once: the entry points serialise themselves.  A
replay of a captured sequence is ordered with the eager work around it on whatever stream the caller has set."""
import ctypes as C
import threading

import numpy as np
import pytest

import maidenx_amd.lib as L
from test_gpu_program import Seq, replay_equals_eager, u64

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def lib():
    if L.device_count() < 1:
        pytest.skip("no GPU")
    return L.load()


def chain(lib, seed, n, steps):
    """A dependent chain on buffers of its own: x <- (x * a + b) alternating with in-place adds, then a row sum."""
    r = np.random.default_rng(seed)
    seq = Seq(lib)
    x0 = r.standard_normal(n).astype(np.float32)
    b = seq.dev(r.standard_normal(n).astype(np.float32))
    cur = seq.dev(x0)
    md1, md2 = u64([n], [1], 0), u64([n], [1], [1], 0, 0)
    for k in range(steps):
        nxt = seq.out(n * 4, "f4")
        if k % 3 == 0:
            seq.add("mul_scalar_f32", n, 1, md1, cur.ptr, C.c_float(0.75), nxt.ptr)
        elif k % 3 == 1:
            seq.add("add_f32", n, 1, md2, cur.ptr, b.ptr, nxt.ptr)
        else:
            seq.add("tanh_f32", n, 1, md1, cur.ptr, nxt.ptr)
        seq.add("add_inplace_f32", n, 1, md2, nxt.ptr, b.ptr)
        cur = nxt
    rows = n // 250
    total = seq.out(rows * 4, "f4")
    seq.add("sum_f32", rows * 250, 2, 1, u64([rows, 250], [250, 1], [250], [1], 0), cur.ptr, total.ptr)
    seq.last = cur
    return seq


def test_two_host_threads_run_independent_chains(lib):
    """Both threads issue a few hundred launches at once; each result must be the one the same chain gives alone."""
    alone = []
    for seed in (11, 12):
        seq = chain(lib, seed, 20000, 60)
        seq.run()
        alone.append(seq.read())
    assert lib.hip_get_last_status() == 0, lib.hip_status_string()
    seqs = [chain(lib, seed, 20000, 60) for seed in (11, 12)]
    start = threading.Barrier(2)
    errors = []

    def work(seq):
        try:
            start.wait()
            for _ in range(3):
                seq.run()
        except Exception as e:      # noqa: BLE001
            errors.append(e)

    threads = [threading.Thread(target=work, args=(s,)) for s in seqs]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errors
    assert lib.hip_get_last_status() == 0, lib.hip_status_string()
    for seq, want in zip(seqs, alone):
        for g, e in zip(seq.read(), want):
            assert g.tobytes() == e.tobytes()


def test_a_call_from_another_thread_during_a_capture_is_refused(lib):
    """The open capture belongs to the thread that began it: another thread's launch must not be recorded into it."""
    seq = chain(lib, 21, 3000, 6)
    seq.run()
    want = seq.read()
    seq.clear_outputs()
    other_out = L.DeviceBuffer(64 * 4)
    lib.hip_fill_f32(64, other_out.ptr, C.c_float(5.0))
    assert lib.hip_synchronize() == 0
    assert lib.hip_graph_begin_capture() == 0
    seq.run()
    refused = []

    def intruder():
        lib.hip_fill_f32(64, other_out.ptr, C.c_float(-1.0))
        refused.append(lib.hip_malloc(C.byref(C.c_void_p()), 16))

    t = threading.Thread(target=intruder)
    t.start()
    t.join()
    h = C.c_void_p()
    assert lib.hip_graph_end_capture(C.byref(h)) == 0
    try:
        assert refused and refused[0] != 0
        assert lib.hip_get_last_status() == 1 and b"another host thread" in lib.hip_status_string()
        assert lib.hip_graph_launch(h) == 0
        for g, e in zip(seq.read(), want):
            assert g.tobytes() == e.tobytes()
        assert (other_out.to_numpy(np.float32) == 5.0).all()      # the intruder's fill was neither run nor recorded
    finally:
        assert lib.hip_graph_destroy(h) == 0


@pytest.mark.parametrize("n,program", [(1000, True), (1 << 17, False)])
def test_replay_on_a_caller_set_stream_equals_eager(lib, n, program):
    """With a non-blocking stream of the caller's set, replays and the eager fills between them share buffers and the
    library's scratch: they are only ordered if the replay is queued on that same stream."""
    s = C.c_void_p()
    assert lib.hip_stream_create(C.byref(s)) == 0
    assert lib.hip_set_stream(s) == 0
    try:
        seq = chain(lib, 31, n, 9)
        if not program:
            # a column reduction with chunk partials in the library's scratch, after the chain
            rows = n // 64
            o = seq.out(64 * 4, "f4")
            seq.add("sum_f32", rows * 64, 2, 1, u64([rows, 64], [64, 1], [rows], [64], 0), seq.last.ptr, o.ptr)
        replay_equals_eager(lib, seq, expect_program=program, replays=4)
    finally:
        assert lib.hip_set_stream(None) == 0
        assert lib.hip_stream_synchronize(s) == 0
        assert lib.hip_stream_destroy(s) == 0
    assert lib.hip_get_last_status() == 0, lib.hip_status_string()
