"""The host layer (maidenx_amd/host/mx_tensor.hpp) on the CPU oracle: the reference's tensor-level tests with
their gradients, error behaviour, and the two training workloads against closed forms."""
import numpy as np
import pytest

from host_programs import TKAT, check_case, conv_inputs, conv_numpy, conv_step, mlp_numpy, mlp_run, run_case
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


def test_mlp_call_count_is_stable(mx_oracle):
    mx = mx_oracle
    mlp_run(mx, 2, n=100)
    mx.reset_backend_calls()
    mlp_run(mx, 10, n=100)
    assert mx.backend_calls() % 10 == 0
    assert 25 <= mx.backend_calls() // 10 <= 60        # about 45 `be` calls per step in the reference (a few are fills here)


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
    backend.  The host layer derives the same thing from the reference's backward closures; the number of backend
    calls must agree (device-side casts are not backend calls in the reference and are not counted)."""
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
    mx.reset_backend_calls()
    z = getattr(x, op)(y) if op in ("add", "mul", "div") else getattr(x, op)()
    z.backward()
    assert mx.backend_calls() == want, (op, case, mx.backend_calls(), want)
