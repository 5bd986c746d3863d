"""The host layer (maidenx_amd/host/mx_tensor.hpp) on the CPU oracle: the reference's tensor-level tests with
their gradients, error behaviour, and the two training workloads against closed forms."""
import numpy as np
import pytest

from host_programs import (TKAT, bf16_round, check_case, conv_inputs, conv_numpy, conv_step, elementwise_program, mlp_numpy, mlp_run,
                           run_case)
from maidenx_amd.tensor import MxError


@pytest.mark.parametrize("case", TKAT, ids=[f"{c['program'][0][1]}@{c['cite'].split('/')[-1]}" for c in TKAT])
def test_reference_tensor_cases(mx_oracle, case):
    check_case(run_case(mx_oracle, case), case)


def test_layout_rules(mx_oracle):
    mx = mx_oracle
    x = mx.tensor(np.arange(24, dtype=np.float32).reshape(2, 3, 4))
    assert x.strides == (12, 4, 1) and x.is_contiguous()
    t = x.transpose(0, 2)
    assert t.shape == (4, 3, 2) and t.strides == (1, 4, 12) and not t.is_contiguous()
    np.testing.assert_array_equal(t.numpy(), np.arange(24, dtype=np.float32).reshape(2, 3, 4).transpose(2, 1, 0))
    b = mx.tensor([1.0, 2.0, 3.0, 4.0]).broadcast((2, 3, 4))
    assert b.strides == (0, 0, 1)                      # crates/maidenx_core/src/layout.rs:252-296
    r = t.reshape((-1, 2))                             # non-contiguous reshape copies (ops/transform.rs:364-366)
    assert r.shape == (12, 2) and r.is_contiguous()
    s = mx.tensor([5.0]).squeeze(0)
    assert s.shape == (1,)                             # a squeezed [1] stays [1] (ops/transform.rs:50-52)
    d = mx.tensor([1.0, 2.0, 3.0]).matmul(mx.tensor([4.0, 5.0, 6.0]))
    assert d.shape == ()                               # tests/ops_matmul.rs:53


@pytest.mark.parametrize("build,kind", [
    (lambda mx: mx.tensor([1.0, 2.0, 3.0]).add(mx.tensor([1.0, 2.0])), "InvalidShape"),
    (lambda mx: mx.tensor(np.ones((2, 3), np.float32)).matmul(mx.tensor(np.ones((4, 2), np.float32))), "InvalidShape"),
    (lambda mx: mx.tensor(np.ones((2, 3), np.float32)).sum(2), "DimensionOutOfBounds"),
    (lambda mx: mx.tensor(np.ones((2, 3), np.float32)).transpose(0, 1).view((6,)), "InvalidOperation"),
    (lambda mx: mx.tensor(np.ones((2, 3), np.float32)).view((4,)), "InvalidShape"),
    (lambda mx: mx.tensor(np.ones((2, 3), np.float32)).reshape((-1, -1)), "InvalidShape"),
    (lambda mx: mx.tensor(np.ones((2, 3), np.float32)).sum_to_shape((2, 2)), "ShapeMismatch"),
    (lambda mx: mx.tensor(np.ones((2, 3), np.float32)).sum_to_shape((1, 2, 3)), "ShapeMismatch"),
    (lambda mx: mx.tensor(np.ones((2, 3), np.float32)).broadcast((3,)), "InvalidArgument"),
    (lambda mx: mx.tensor(np.ones((2, 3), np.float32)).broadcast((4, 3)), "InvalidShape"),
])
def test_errors_are_the_reference_variants(mx_oracle, build, kind):
    with pytest.raises(MxError) as e:
        build(mx_oracle)
    assert e.value.kind == kind


def test_backward_visits_a_buffer_once(mx_oracle):
    # crates/maidenx_tensor/src/lib.rs:308-323: the walk is keyed on the buffer, so the second use of x in
    # y = x*x receives its gradient through accumulate_grad only once per path, and both paths are taken
    mx = mx_oracle
    x = mx.tensor([1.0, 2.0, 3.0]).with_grad()
    y = x.mul(x)
    y.backward()
    np.testing.assert_array_equal(x.grad().numpy(), [2.0, 4.0, 6.0])


def test_broadcast_gradients_reduce(mx_oracle):
    mx = mx_oracle
    rng = np.random.default_rng(1)
    a, b = rng.standard_normal((4, 5)).astype(np.float32), rng.standard_normal((1, 5)).astype(np.float32)
    x, y = mx.tensor(a).with_grad(), mx.tensor(b).with_grad()
    z = x.mul(y).exp().relu().sum_all()
    z.backward()
    e = np.exp(a.astype(np.float64) * b)
    np.testing.assert_allclose(x.grad().numpy(), e * b, rtol=1e-5)
    np.testing.assert_allclose(y.grad().numpy(), (e * a).sum(0, keepdims=True), rtol=1e-5)
    s = mx.tensor(np.array(2.0, np.float32), shape=()).with_grad()        # 0-d operand: item + fill path
    w = x.detach().mul(s).sum_all()
    w.backward()
    np.testing.assert_allclose(s.grad().numpy(), a.astype(np.float64).sum(), rtol=1e-5)


def test_mlp_training_matches_gradient_descent(mx_oracle):
    # configs[0]: README Linear(3->1)+MSE+SGD; 60 epochs against float64 gradient descent from the same start
    got = mlp_run(mx_oracle, 60)
    losses, w, b = mlp_numpy(60)
    np.testing.assert_allclose(got["losses"], losses, rtol=2e-4)
    np.testing.assert_allclose(got["weight"], w, rtol=1e-4, atol=1e-6)
    np.testing.assert_allclose(got["bias"], b, rtol=1e-4, atol=1e-6)
    assert got["losses"][-1] < got["losses"][0] * 0.5
    assert mx_oracle.device_allocations() > 0


def test_run_steps_on_the_cpu_build_is_the_plain_loop(mx_oracle):
    """mxt_run_steps without a graph-capable backend: n calls of the step, failures handed on."""
    mx = mx_oracle
    a = mx.tensor(np.full((2, 3), 3.0, np.float32)).with_grad()
    calls = []

    def step():
        calls.append(1)
        a.mul(a).sum_all().backward()
    mx.run_steps(step, 40)
    assert len(calls) == 40 and mx.last_train_replayed() == 0
    np.testing.assert_array_equal(a.grad().numpy(), np.full((2, 3), 40 * 6.0, np.float32))

    def bad():
        raise ValueError("no")
    with pytest.raises(ValueError):
        mx.run_steps(bad, 3)


def test_adam_training_matches_the_update_rule(mx_oracle):
    """adam.rs through the tensor API on the CPU oracle (op by op) against the update rule in float64."""
    from host_programs import mlp_adam_numpy, mlp_adam_run
    got = mlp_adam_run(mx_oracle, 25)
    losses, w, b = mlp_adam_numpy(25)
    assert losses[-1] < 0.8 * losses[0]
    np.testing.assert_allclose(got["losses"], losses, rtol=2e-4)
    np.testing.assert_allclose(got["weight"], w, rtol=2e-4, atol=1e-6)
    np.testing.assert_allclose(got["bias"], b, rtol=2e-4, atol=1e-6)


def test_sqrt_forward_and_backward(mx_oracle):
    x = np.array([0.25, 1.0, 4.0, 9.0], np.float32)
    t = mx_oracle.tensor(x).with_grad()
    y = t.sqrt()
    np.testing.assert_array_equal(y.numpy(), np.sqrt(x))
    y.sum_all().backward()
    np.testing.assert_allclose(t.grad().numpy(), 0.5 / np.sqrt(x), rtol=1e-6)          # unary.rs:176-178: go / (2 * sqrt(x))


def test_the_two_builds_of_the_host_layer_keep_their_own_state(mx_oracle):
    """libmaidenx_host.so (over the HIP backend) and the oracle's build of the same headers live in one process in the
    GPU tests and in bench.py: counters and switches of one must not be those of the other (as GNU-unique symbols the
    function-local statics of the layer's inline functions would be shared)."""
    import ctypes as C
    from maidenx_amd.tensor import HOST_LIB_PATH
    hip_host = C.CDLL(HOST_LIB_PATH)                 # loading needs no GPU; nothing below touches the device
    hip_host.mxt_backend_calls.restype = C.c_size_t
    hip_host.mxt_reset_backend_calls()
    mx = mx_oracle
    mx.reset_backend_calls()
    t = mx.tensor(np.arange(6, dtype=np.float32).reshape(2, 3))
    t.mul(t).add(t)
    assert mx.backend_calls() == 2
    assert hip_host.mxt_backend_calls() == 0


def test_mlp_call_count_is_stable(mx_oracle):
    mx = mx_oracle
    mlp_run(mx, 2, n=100)
    counts = []
    for steps in (10, 20):
        mx.reset_backend_calls()
        mlp_run(mx, steps, n=100)
        counts.append(mx.backend_calls())
    # (the first step of a run may need a call less: a gradient that is accumulated into for the first time can become the
    # gradient as it is)
    assert (counts[1] - counts[0]) % 10 == 0
    assert 15 <= (counts[1] - counts[0]) // 10 <= 60   # about 45 `be` calls per step in the reference (a few are fills here)


@pytest.mark.parametrize("B,Cin,H,W,Cout,k,stride,pad", [(2, 3, 6, 5, 4, 3, 1, 1), (1, 2, 7, 7, 3, 3, 2, 2), (3, 4, 5, 5, 2, 1, 1, 1)])
def test_conv2d_forward_backward(mx_oracle, B, Cin, H, W, Cout, k, stride, pad):
    # only stride == pad: the layer stores (stride, pad) where the kernels read (pad, stride)
    # (nn/layers/conv.rs:352-365 vs crates/maidenx_cpu/src/nn/conv.rs:31-34)
    x, w, b = conv_inputs(B, Cin, H, W, Cout, k, seed=B * 100 + H)
    oh, ow = (H + 2 * pad - k) // stride + 1, (W + 2 * pad - k) // stride + 1
    target = np.random.default_rng(5).standard_normal((B, Cout, oh, ow)).astype(np.float32)
    got = conv_step(mx_oracle, x, w, b, stride, pad, target)
    ref = conv_numpy(x, w, b, stride, pad, target)
    for key in ("out", "loss", "grad_b", "grad_w", "grad_x"):
        np.testing.assert_allclose(got[key], ref[key], rtol=1e-4, atol=1e-6, err_msg=key)


def test_sum_all_in_one_pass_or_dim_by_dim(mx_oracle):
    """sum_all() of a contiguous f32 tensor (and the bias gradient of Conv2d) as one reduction, or dim by dim as
    reduction.rs:76-83 does it: the same gradients bit for bit, the sums within the f32 tolerance of a reduction of each
    other and of float64."""
    mx = mx_oracle
    rng = np.random.default_rng(31)
    a = rng.standard_normal((5, 7, 9, 11)).astype(np.float32)
    x, w, bias = conv_inputs(2, 3, 6, 5, 4, 3, seed=22)
    target = rng.standard_normal((2, 4, 6, 5)).astype(np.float32)
    res = {}
    try:
        for one_pass in (False, True):
            mx.set_sum_all_in_one_pass(one_pass)
            t = mx.tensor(a).with_grad()
            mx.reset_backend_calls()
            z = t.mul(t).sum_all()
            z.backward()
            res[one_pass] = dict(z=z.numpy(), g=t.grad().numpy(), calls=mx.backend_calls(), **conv_step(mx, x, w, bias, 1, 1, target))
    finally:
        mx.set_sum_all_in_one_pass(True)
    assert res[True]["calls"] < res[False]["calls"]
    for key in ("g", "grad_x", "grad_w", "out"):
        np.testing.assert_array_equal(res[True][key].view(np.uint32), res[False][key].view(np.uint32), err_msg=key)
    # the bias gradient of Conv2d is itself a sum over W, H and the batch (conv.rs:287-291): one pass or three
    scale = np.abs(res[False]["grad_b"]).max()
    assert np.abs(res[True]["grad_b"] - res[False]["grad_b"]).max() <= 1e-5 * scale
    exact = float(np.sum(a.astype(np.float64) ** 2))
    for one_pass in (False, True):
        assert abs(float(res[one_pass]["z"]) - exact) <= 1e-5 * exact
    assert abs(float(res[True]["loss"]) - float(res[False]["loss"])) <= 1e-5 * abs(float(res[False]["loss"]))


def _shortcut_programs(mx):
    """Programs whose backward passes contain what the shortcuts leave out: operands without a gradient, pow(2),
    gradients that arrive as broadcast views (sum over dims, a broadcast operand, the MSE loss)."""
    out = {}
    rng = np.random.default_rng(12)
    a = rng.standard_normal((6, 5, 4)).astype(np.float32)
    b = (rng.standard_normal((1, 5, 1)) + 3.0).astype(np.float32)
    for op in ("add", "sub", "mul", "div"):
        for ga, gb in ((True, False), (False, True), (True, True)):
            ta, tb = mx.tensor(a), mx.tensor(b)
            if ga:
                ta = ta.with_grad()
            if gb:
                tb = tb.with_grad()
            z = getattr(ta, op)(tb).pow(2.0).sum_all()
            z.backward()
            key = f"{op}_{int(ga)}{int(gb)}"
            out[key + "_z"] = z.numpy()
            if ga:
                out[key + "_ga"] = ta.grad().numpy()
            if gb:
                out[key + "_gb"] = tb.grad().numpy()
    # a 0-d operand (materialised by the reference, read through zero strides with the shortcuts), zeros of both signs in
    # the data, and a matmul whose gradients are sums of a single term
    az = a.copy()
    az[::2, 1, :] = 0.0
    az[1::2, 2, :] = -0.0
    for op in ("add", "sub", "mul", "div"):
        for sval in (-2.5, 0.0):
            if op == "div" and sval == 0.0:
                continue
            ta, ts = mx.tensor(az).with_grad(), mx.tensor(np.array(sval, np.float32), shape=()).with_grad()
            y = getattr(ta, op)(ts)
            z = y.mul(y).sum_all()
            z.backward()
            key = f"scalar_{op}_{sval}"
            out[key + "_y"], out[key + "_ga"], out[key + "_gs"] = y.numpy(), ta.grad().numpy(), ts.grad().numpy()
    m1, m2 = mx.tensor(az.reshape(30, 4)).with_grad(), mx.tensor(rng.standard_normal((4, 1)).astype(np.float32)).with_grad()
    mm = m1.matmul(m2)
    mm.sum_all().backward()
    out["mm_y"], out["mm_g1"], out["mm_g2"] = mm.numpy(), m1.grad().numpy(), m2.grad().numpy()
    x, w, bias = conv_inputs(2, 3, 6, 5, 4, 3, seed=21)
    target = rng.standard_normal((2, 4, 6, 5)).astype(np.float32)
    for k, v in conv_step(mx, x, w, bias, 1, 1, target).items():
        out["conv_" + k] = v
    for k, v in mlp_run(mx, 3, n=200).items():
        out["mlp_" + k] = v
    return out


def test_backward_shortcuts_change_no_bit(mx_oracle):
    mx = mx_oracle
    try:
        mx.set_autograd_shortcuts(False)
        mx.reset_backend_calls()
        whole = _shortcut_programs(mx)
        calls_whole = mx.backend_calls()
        mx.set_autograd_shortcuts(True)
        mx.reset_backend_calls()
        short = _shortcut_programs(mx)
        calls_short = mx.backend_calls()
    finally:
        mx.set_autograd_shortcuts(True)
    assert calls_short < calls_whole
    assert whole.keys() == short.keys()
    for key in whole:
        np.testing.assert_array_equal(np.asarray(short[key]).view(np.uint32), np.asarray(whole[key]).view(np.uint32), err_msg=key)


@pytest.mark.parametrize("B,Cin,H,W,Cout,k,stride,pad", [(2, 3, 6, 5, 4, 3, 1, 1), (1, 2, 7, 7, 3, 3, 2, 2), (3, 4, 5, 5, 2, 1, 1, 1)])
def test_conv2d_backward_makes_only_the_rows_of_grad_cols_that_col2im_reads(mx_oracle, B, Cin, H, W, Cout, k, stride, pad):
    # col2im gets num_els = B*C*H*W and reads nothing at or beyond that flat index (conv.rs:391, cpu/nn/conv.rs:135): the
    # product restricted to the leading rows must give the bytes of the whole product, with one matmul call either way
    x, w, b = conv_inputs(B, Cin, H, W, Cout, k, seed=B * 10 + W)
    oh, ow = (H + 2 * pad - k) // stride + 1, (W + 2 * pad - k) // stride + 1
    target = np.random.default_rng(6).standard_normal((B, Cout, oh, ow)).astype(np.float32)
    mx = mx_oracle
    try:
        mx.set_conv_skip_unread_grad_cols(False)
        mx.reset_backend_calls()
        whole = conv_step(mx, x, w, b, stride, pad, target)
        calls_whole = mx.backend_calls()
        mx.set_conv_skip_unread_grad_cols(True)
        mx.reset_backend_calls()
        lead = conv_step(mx, x, w, b, stride, pad, target)
        calls_lead = mx.backend_calls()
    finally:
        mx.set_conv_skip_unread_grad_cols(True)
    assert calls_lead == calls_whole
    for key in ("out", "loss", "grad_b", "grad_w", "grad_x"):
        np.testing.assert_array_equal(lead[key].view(np.uint32), whole[key].view(np.uint32), err_msg=key)


def test_conv2d_backward_with_zero_padding_is_an_error(mx_oracle):
    # padding 0 lands in the slots col2im reads as its stride: the reference panics on the division
    x, w, b = conv_inputs(1, 2, 5, 5, 2, 3, seed=3)
    target = np.zeros((1, 2, 3, 3), np.float32)
    with pytest.raises(MxError) as e:
        conv_step(mx_oracle, x, w, b, 1, 0, target)
    assert e.value.kind == "InvalidOperation"


@pytest.mark.parametrize("op", ["add", "mul", "div", "exp", "relu", "gelu"])
@pytest.mark.parametrize("case", ["contig", "bcast", "transposed"])
def test_bench_chain_is_the_host_layers_call_sequence(mx_oracle, op, case):
    """bench.py's ChainBuilder spells out, call by call, what forward + backward of each op dispatches to the
    backend.  The host layer derives the same thing from the reference's backward closures (with none of its own
    shortcuts); the number of backend calls must agree (device-side casts are not backend calls in the reference and are
    not counted)."""
    import bench
    if op in ("exp", "relu", "gelu") and case == "bcast":
        pytest.skip("unary ops have no broadcast case")
    mx = mx_oracle
    R, C = 6, 8

    class FakeLib:
        def __getattr__(self, name):
            return lambda *a: None
    b = bench.ChainBuilder(FakeLib(), "x_", lambda count, dtag, init: (0, None), "f32", R, C, seed=1)
    getattr(b, op)(case)
    want = sum(1 for c in b.calls if not c.tag.startswith("cast_bool"))

    rng = np.random.default_rng(3)
    if case == "transposed":
        base = mx.tensor(rng.standard_normal((C, R)).astype(np.float32)).with_grad()
        x = base.transpose(0, 1)
    else:
        x = mx.tensor(rng.standard_normal((R, C)).astype(np.float32)).with_grad()
    y = mx.tensor(rng.standard_normal((1, C) if case == "bcast" else (R, C)).astype(np.float32) + 3.0).with_grad()
    # (the chain is the reference's own sequence: backward() with nothing left out)
    try:
        mx.set_autograd_shortcuts(False)
        mx.reset_backend_calls()
        z = getattr(x, op)(y) if op in ("add", "mul", "div") else getattr(x, op)()
        z.backward()
        assert mx.backend_calls() == want, (op, case, mx.backend_calls(), want)
    finally:
        mx.set_autograd_shortcuts(True)


@pytest.mark.parametrize("dt", ["f32", "bf16"])
def test_bench_chain_tags_name_one_launch_class(dt):
    """bench.py averages the launch times of a tag and divides ONE byte count by that average, so launches that share a
    tag must move the same bytes (x * x reads one operand, x * y two: two tags)."""
    import bench

    class FakeLib:
        def __getattr__(self, name):
            return lambda *a: None
    ptr = iter(range(1, 1000))
    b = bench.ChainBuilder(FakeLib(), "x_", lambda count, dtag, init: (next(ptr) << 20, None), dt, 16, 32, seed=1)
    seen = {}
    for c in b.build():
        assert seen.setdefault(c.tag, c.bytes) == c.bytes, c.tag
    e = 4 if dt == "f32" else 2
    assert seen[f"mul_{dt}/contig+contig"] == 3 * 16 * 32 * e
    assert any(t.endswith("+same") and v == 2 * 16 * 32 * ESZ_OF[t.split("/")[0].rsplit("_", 1)[1]] for t, v in seen.items())


ESZ_OF = {"f32": 4, "bf16": 2}


# ---- bf16 through the host layer --------------------------------------------------------------------------
@pytest.mark.parametrize("case", TKAT, ids=[f"{c['program'][0][1]}@{c['cite'].split('/')[-1]}" for c in TKAT])
def test_reference_tensor_cases_bf16(mx_oracle, case):
    # the reference runs the same tests for bf16 with |error| < 0.1 (e.g. tests/ops_binary.rs:28-45)
    check_case(run_case(mx_oracle, case, dtype="bf16"), case, tol=0.1)


def test_dtype_promotion_rules(mx_oracle):
    mx = mx_oracle
    x = mx.tensor([1.0, 2.0, 3.0], dtype="bf16")
    assert x.dtype == "bf16" and x.mul_scalar(2.0).dtype == "bf16"          # integer-valued scalar keeps the dtype
    assert x.mul_scalar(0.5).dtype == "f32" and x.add_scalar(0.25).dtype == "f32"   # ops/unary.rs:796-800, 872-876
    assert x.add_scalar(1.0).dtype == "bf16" and x.div_scalar(3.0).dtype == "bf16"  # ops/unary.rs:911-915
    assert x.pow(2.0).dtype == "bf16" and x.pow(0.5).dtype == "f32"         # ops/unary.rs:1044-1048
    f = mx.tensor([1.0, 2.0, 3.0])
    assert x.add(f).dtype == "f32" and f.mul(x).dtype == "f32"              # utils/promotion.rs:16-33
    assert x.gt_scalar(1.5).dtype == "bool"
    np.testing.assert_array_equal(x.gt_scalar(1.5).to_dtype("bf16").numpy(), [0.0, 1.0, 1.0])
    np.testing.assert_array_equal(mx.tensor([1.00390625, 3.14159], dtype="bf16").numpy(), bf16_round([1.00390625, 3.14159]))
    g = mx.tensor([0.5, -1.5], dtype="bf16").with_grad()
    g.gelu().backward()
    assert g.grad().dtype == "bf16"                                          # cast back when accumulated (ops/binary.rs:660-662)


@pytest.mark.parametrize("op", ["add", "mul", "div", "exp", "relu", "gelu"])
@pytest.mark.parametrize("case", ["contig", "bcast", "transposed"])
def test_bench_chain_is_the_host_layers_call_sequence_bf16(mx_oracle, op, case):
    """As above for bf16, where the gelu closure promotes to f32: kernel calls and whole-buffer casts both agree."""
    import bench
    if op in ("exp", "relu", "gelu") and case == "bcast":
        pytest.skip("unary ops have no broadcast case")
    mx = mx_oracle

    class FakeLib:
        def __getattr__(self, name):
            return lambda *a: None
    b = bench.ChainBuilder(FakeLib(), "x_", lambda count, dtag, init: (0, None), "bf16", 6, 8, seed=1)
    getattr(b, op)(case)
    want_casts = sum(1 for c in b.calls if c.tag.startswith("cast_"))
    want_calls = len(b.calls) - want_casts
    try:
        mx.set_autograd_shortcuts(False)
        mx.reset_backend_calls()
        elementwise_program(mx, op, case, "bf16", R=6, C=8)
        assert (mx.backend_calls(), mx.cast_calls()) == (want_calls, want_casts), (op, case)
    finally:
        mx.set_autograd_shortcuts(True)


@pytest.mark.parametrize("case", ["contig", "bcast", "transposed"])
def test_bf16_forward_backward_values(mx_oracle, case):
    """add / mul / div on bf16 tensors against per-operation bf16 rounding in numpy."""
    for op in ("add", "mul", "div"):
        r = elementwise_program(mx_oracle, op, case, "bf16")
        x = bf16_round(r["xs"].T if case == "transposed" else r["xs"])
        y = np.broadcast_to(bf16_round(r["ys"]), x.shape)
        assert r["z.dtype"] == "bf16" and r["gx.dtype"] == "bf16"
        fwd = {"add": x + y, "mul": x * y, "div": x / y}[op]
        np.testing.assert_array_equal(r["z"], bf16_round(fwd), err_msg=op)
        ones = np.ones_like(x)
        if op == "add":
            gx, gy_full = ones, ones
        elif op == "mul":
            gx, gy_full = bf16_round(ones * y), bf16_round(ones * x)
        else:
            gx = bf16_round(ones / y)
            gy_full = -bf16_round(bf16_round(ones * x) / bf16_round(y * y))
        if case == "transposed":
            gx = gx.T                                           # gradient of the tensor the view was taken from
        np.testing.assert_array_equal(r["gx"], gx, err_msg=op)
        if case == "bcast":
            # summed over rows in f32 and rounded once (crates/maidenx_cpu/src/ops/reduction.rs:568 accumulates in bf16;
            # the column sums here are short enough for a loose bound)
            ref = gy_full.astype(np.float64).sum(0, keepdims=True)
            assert np.all(np.abs(r["gy"] - ref) <= np.abs(gy_full).sum(0, keepdims=True) * 2.0 ** -6), op
        else:
            np.testing.assert_array_equal(r["gy"], gy_full, err_msg=op)
