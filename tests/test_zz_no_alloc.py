"""hip_sum_f32_noalloc: the sum for callers that cannot allocate.  Same kernels as hip_sum_f32 with the chunk partials
in a fixed array inside the library, so its output must be hip_sum_f32's bit for bit — also on a second call with a
smaller input, which reuses the array while it still holds the first call's partials."""
import numpy as np
import pytest

import maidenx_amd.lib as L
from helpers import In, Out, meta_reduce, rng

pytestmark = pytest.mark.gpu

# (dims, reduced dim): shapes whose reduced axis is cut into chunks (partials in scratch), first a larger then a smaller one
PAIRS = [
    (([4096, 2048], 0), ([1024, 512], 0)),        # column reduce, 16-wave split kernel with chunks
    (([8, 1 << 18], 1), ([3, 1 << 16], 1)),       # few long rows: the row is cut into chunks
    (([2, 2000, 96], 1), ([1, 700, 40], 1)),      # narrow columns: one thread per column vector, chunks folded twice
]


def sums(hip, name, dims, dim, x, strides=None):
    strides = strides or [int(np.prod(dims[i + 1:])) for i in range(len(dims))]
    n_out = x.size // dims[dim]
    allocs = L.load().hip_scratch_allocations()
    (o,) = hip.call(name, x.size, len(dims), 1, meta_reduce(dims, strides, dim), In(x), Out(n_out, "f32"))
    if name.endswith("_noalloc"):
        assert L.load().hip_scratch_allocations() == allocs, "the no-alloc entry point grew the library's scratch"
    return o


@pytest.mark.parametrize("first,second", PAIRS)
def test_two_calls_in_a_row_equal_the_allocating_entry_point(hip, first, second):
    assert L.load().hip_noalloc_prepare() == 0
    r = rng(401)
    for dims, dim in (first, second):
        x = r.uniform(-1, 1, int(np.prod(dims))).astype(np.float32)
        want = sums(hip, "sum_f32", dims, dim, x)
        got = sums(hip, "sum_f32_noalloc", dims, dim, x)
        assert got.tobytes() == want.tobytes(), (dims, dim)
        ref = x.astype(np.float64).reshape(dims).sum(axis=dim).ravel()
        assert np.abs(got - ref).max() <= 1e-5 * np.abs(x).astype(np.float64).reshape(dims).sum(axis=dim).max()


def test_shapes_without_partials(hip):
    r = rng(402)
    for dims, dim in (([300, 70], 1), ([5, 1, 9], 1), ([64, 33], 0)):
        x = r.standard_normal(int(np.prod(dims))).astype(np.float32)
        assert sums(hip, "sum_f32_noalloc", dims, dim, x).tobytes() == sums(hip, "sum_f32", dims, dim, x).tobytes()


@pytest.mark.parametrize("dims,dim", [([20000, 5], 0), ([3, 16384, 17], 1), ([70001, 33], 0)])
def test_narrow_rows_under_a_long_axis_keep_the_allocating_bits(hip, dims, dim):
    """[L, S] with S < 64 and L >= 8192 is regrouped into wide rows whose partial rows need a buffer of their own: the last
    MiB of the fixed array here, scratch slot 2 in hip_sum_f32.  Same kernels, same order, same bits."""
    x = rng(403).uniform(-1, 1, int(np.prod(dims))).astype(np.float32)
    got = sums(hip, "sum_f32_noalloc", dims, dim, x)
    assert got.tobytes() == sums(hip, "sum_f32", dims, dim, x).tobytes()
    x64 = x.astype(np.float64).reshape(dims)
    assert np.abs(got - x64.sum(axis=dim).ravel()).max() <= 1e-5 * np.abs(x64).sum(axis=dim).max()


@pytest.mark.parametrize("dims,perm,dim", [([640, 512], (1, 0), 0), ([640, 512], (1, 0), 1), ([96, 64, 80], (2, 0, 1), 1),
                                           ([40, 30], (1, 0), 0)])
def test_permuted_views_are_summed_without_the_logical_order_copy(hip, oracle, dims, perm, dim):
    """A strided input of 2^18 elements or more: hip_sum_f32 copies it into logical order in grown scratch; the no-alloc
    entry point must not (the counter checked in sums()), and sums one thread per output in ascending order.  The values
    are the reference's for its non-contiguous branch, which hands over the memory stride of the reduced dim as the
    slice stride (crates/maidenx_tensor/src/ops/reduction.rs:728-729): compared with the oracle and with hip_sum_f32."""
    base = rng(404).uniform(-1, 1, int(np.prod(dims))).astype(np.float32)
    cs = [int(np.prod(dims[i + 1:])) for i in range(len(dims))]
    vdims, vstrides = [dims[p] for p in perm], [cs[p] for p in perm]
    got = sums(hip, "sum_f32_noalloc", vdims, dim, base, vstrides)
    want = sums(hip, "sum_f32", vdims, dim, base, vstrides)
    scale = np.abs(base).astype(np.float64).sum() / got.size * 4
    assert np.abs(got.astype(np.float64) - want).max() <= 1e-5 * scale
    (orc,) = oracle.call("sum_f32", base.size, len(vdims), 1, meta_reduce(vdims, vstrides, dim), In(base), Out(got.size, "f32"))
    assert np.abs(got.astype(np.float64) - orc).max() <= 1e-5 * scale


def test_partials_beyond_the_fixed_array_are_refused(hip):
    """[1700, 256, 63] along dim 1: odd-width columns take the thread-per-column kernel, which cuts the axis in two and
    needs (2 + 8) x 1700 x 63 partials, just over 4 MiB.  The host refuses before anything is queued, so the output keeps
    its poison, and the allocating entry point still works afterwards."""
    dims, dim = [1700, 256, 63], 1
    strides = [256 * 63, 63, 1]
    x = np.ones(int(np.prod(dims)), dtype=np.float32)
    out = Out(1700 * 63, "f32")
    with pytest.raises(L.HipError, match="exceed their 3 MiB"):
        hip.call("sum_f32_noalloc", x.size, 3, 1, meta_reduce(dims, strides, dim), In(x), out)
    assert (out.arr.view(np.uint8) == 0xCD).all()
    (o,) = hip.call("sum_f32", x.size, 3, 1, meta_reduce(dims, strides, dim), In(x), Out(1700 * 63, "f32"))
    assert (o == 256.0).all()
