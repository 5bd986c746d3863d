"""The host layer on the HIP backend (libmaidenx_host.so -> libmaidenx_hip.so) against the same programs on the
CPU oracle and against the reference's own expectations."""
import numpy as np
import pytest

from host_programs import TKAT, check_case, conv_inputs, conv_numpy, conv_step, elementwise_program, mlp_numpy, mlp_run, run_case
from maidenx_amd.tensor import MxError

pytestmark = pytest.mark.gpu


def test_adam_fused_step_equals_the_op_sequence(mx_hip, mx_oracle):
    """The HIP host layer's Adam updates a contiguous f32 parameter with one fused call; weights and bias must be the
    bits the fourteen-op form leaves, and both must agree with the CPU oracle's op-by-op run."""
    from host_programs import mlp_adam_run
    fused = mlp_adam_run(mx_hip, 30, fused=True)
    calls_fused = mx_hip.backend_calls()
    plain = mlp_adam_run(mx_hip, 30, fused=False)
    calls_plain = mx_hip.backend_calls() - calls_fused
    assert np.array_equal(fused["weight"], plain["weight"]) and np.array_equal(fused["bias"], plain["bias"])
    assert np.array_equal(fused["losses"], plain["losses"])
    ref = mlp_adam_run(mx_oracle, 30)
    np.testing.assert_allclose(fused["losses"], ref["losses"], rtol=2e-5)
    np.testing.assert_allclose(fused["weight"], ref["weight"], rtol=2e-4, atol=1e-6)
    np.testing.assert_allclose(fused["bias"], ref["bias"], rtol=2e-4, atol=1e-6)
    assert fused["losses"][-1] < 0.8 * fused["losses"][0]
    assert calls_plain > calls_fused + 30 * 2 * 10          # thirteen fewer backend calls per parameter and step


def test_fused_mse_and_sgd_leave_the_op_sequences_weights(mx_hip, mx_oracle):
    """MSELoss and SGD.step as one backend call each (the default on the HIP build) against the op sequences: the same
    weights, bias and input gradient bit for bit after 25 epochs, losses within the tolerance of a sum; fewer calls."""
    from host_programs import mlp_run
    try:
        mx_hip.set_graph_replay(False)
        mx_hip.reset_backend_calls()
        fused = mlp_run(mx_hip, 25, n=3000)
        calls_fused = mx_hip.backend_calls()
        mx_hip.set_fused_nn_kernels(False)
        plain = mlp_run(mx_hip, 25, n=3000)
        calls_plain = mx_hip.backend_calls() - calls_fused
    finally:
        mx_hip.set_fused_nn_kernels(True)
        mx_hip.set_graph_replay(True)
    for key in ("weight", "bias", "input_grad"):
        assert np.array_equal(fused[key], plain[key]), key
    np.testing.assert_allclose(fused["losses"], plain["losses"], rtol=2e-6)
    ref = mlp_run(mx_oracle, 25, n=3000)
    np.testing.assert_allclose(fused["losses"], ref["losses"], rtol=2e-5)
    np.testing.assert_allclose(fused["weight"], ref["weight"], rtol=2e-4, atol=1e-6)
    assert calls_plain >= calls_fused + 25 * 8          # the loss: 10 calls -> 2; the two parameter updates: 4 -> 2


@pytest.mark.parametrize("case", TKAT, ids=[f"{c['program'][0][1]}@{c['cite'].split('/')[-1]}" for c in TKAT])
def test_reference_tensor_cases(mx_hip, case):
    check_case(run_case(mx_hip, case), case)


def test_backend_is_hip(mx_hip):
    assert mx_hip.name == "hip"


def test_errors_match(mx_hip):
    mx = mx_hip
    with pytest.raises(MxError) as e:
        mx.tensor([1.0, 2.0, 3.0]).add(mx.tensor([1.0, 2.0]))
    assert e.value.kind == "InvalidShape"
    with pytest.raises(MxError) as e:
        mx.tensor(np.ones((2, 3), np.float32)).transpose(0, 1).view((6,))
    assert e.value.kind == "InvalidOperation"
    x, w, b = conv_inputs(1, 2, 5, 5, 2, 3, seed=3)
    with pytest.raises(MxError) as e:
        conv_step(mx, x, w, b, 1, 0, np.zeros((1, 2, 3, 3), np.float32))
    assert e.value.kind == "InvalidOperation"


def composite(mx, a, b, c):
    x, y, z = mx.tensor(a).with_grad(), mx.tensor(b).with_grad(), mx.tensor(c).with_grad()
    h = x.matmul(y).add(z).gelu()                      # [M,K]x[K,N] + [N] broadcast
    t = h.transpose(0, 1).mul(h.transpose(0, 1)).relu().tanh()
    r = t.div(t.exp().add_scalar(1.5)).sum(0).mean(0).mul_scalar(3.0)
    r.backward()
    return {"r": r.numpy(), "gx": x.grad().numpy(), "gy": y.grad().numpy(), "gz": z.grad().numpy(), "h": h.numpy()}


def test_composite_graph_matches_oracle(mx_hip, mx_oracle):
    rng = np.random.default_rng(11)
    a, b, c = (rng.standard_normal(s).astype(np.float32) for s in ((37, 19), (19, 23), (23,)))
    got, ref = composite(mx_hip, a, b, c), composite(mx_oracle, a, b, c)
    for k in ref:
        scale = np.abs(ref[k]).max() + 1e-30
        assert np.abs(got[k] - ref[k]).max() <= 2e-5 * scale, k       # f32 sums in a different order


def test_scalar_operand_and_views(mx_hip, mx_oracle):
    def prog(mx):
        x = mx.tensor(np.linspace(-2, 2, 24, dtype=np.float32).reshape(2, 3, 4)).with_grad()
        s = mx.tensor(np.array(0.75, np.float32), shape=()).with_grad()
        y = x.transpose(0, 2).reshape((-1, 2)).mul(s).pow(2.0).sum_to_shape((1, 2)).sum_all()
        y.backward()
        return {"y": y.numpy(), "gs": s.grad().numpy(), "gx": x.grad().numpy()}
    got, ref = prog(mx_hip), prog(mx_oracle)
    for k in ref:
        np.testing.assert_allclose(got[k], ref[k], rtol=1e-5, atol=1e-6, err_msg=k)


def test_mlp_training(mx_hip, mx_oracle):
    got = mlp_run(mx_hip, 60)
    ref = mlp_run(mx_oracle, 60)
    np.testing.assert_allclose(got["losses"], ref["losses"], rtol=1e-4)
    np.testing.assert_allclose(got["weight"], ref["weight"], rtol=1e-4, atol=1e-6)
    np.testing.assert_allclose(got["bias"], ref["bias"], rtol=1e-4, atol=1e-6)
    np.testing.assert_allclose(got["input_grad"], ref["input_grad"], rtol=1e-3, atol=1e-7)
    losses, w, b = mlp_numpy(60)
    np.testing.assert_allclose(got["losses"], losses, rtol=2e-4)
    np.testing.assert_allclose(got["weight"], w, rtol=1e-4, atol=1e-6)


def test_mlp_steps_do_not_allocate_after_warmup(mx_hip):
    mlp_run(mx_hip, 3)
    before = mx_hip.device_allocations()
    mlp_run(mx_hip, 20)
    assert mx_hip.device_allocations() == before          # every buffer of a step comes from the pool


@pytest.mark.parametrize("B,Cin,H,W,Cout,k,stride,pad", [(2, 3, 6, 5, 4, 3, 1, 1), (1, 2, 7, 7, 3, 3, 2, 2), (3, 4, 5, 5, 2, 1, 1, 1),
                                                         (4, 16, 14, 14, 32, 3, 1, 1)])
def test_conv2d_forward_backward(mx_hip, mx_oracle, B, Cin, H, W, Cout, k, stride, pad):
    x, w, b = conv_inputs(B, Cin, H, W, Cout, k, seed=B * 100 + H)
    oh, ow = (H + 2 * pad - k) // stride + 1, (W + 2 * pad - k) // stride + 1
    target = np.random.default_rng(5).standard_normal((B, Cout, oh, ow)).astype(np.float32)
    got = conv_step(mx_hip, x, w, b, stride, pad, target)
    ref = conv_step(mx_oracle, x, w, b, stride, pad, target)
    num = conv_numpy(x, w, b, stride, pad, target)
    for key in ("out", "loss", "grad_b", "grad_w", "grad_x"):
        scale = np.abs(ref[key]).max() + 1e-30
        assert np.abs(got[key] - ref[key]).max() <= 2e-5 * scale, key
        assert np.abs(got[key] - num[key]).max() <= 1e-4 * scale, key


def test_sum_all_in_one_pass_or_dim_by_dim(mx_hip):
    """sum_all() of a contiguous f32 tensor as one reduction, or dim by dim as reduction.rs:76-83 does it: the same
    gradients bit for bit, the sums within the f32 tolerance of a reduction of each other and of float64."""
    mx = mx_hip
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


def test_backward_shortcuts_change_no_bit(mx_hip):
    mx = mx_hip
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


@pytest.mark.parametrize("B,Cin,H,W,Cout,k,stride,pad", [(2, 3, 6, 5, 4, 3, 1, 1), (3, 4, 5, 5, 2, 1, 1, 1), (4, 16, 14, 14, 32, 3, 1, 1),
                                                         (8, 64, 28, 28, 64, 3, 1, 1)])
def test_conv2d_backward_makes_only_the_rows_of_grad_cols_that_col2im_reads(mx_hip, B, Cin, H, W, Cout, k, stride, pad):
    """The product behind the input gradient is made for the leading rows that col2im reads (conv.rs:391,
    crates/maidenx_cpu/src/nn/conv.rs:135); every gradient is the bytes that the whole product gives."""
    x, w, b = conv_inputs(B, Cin, H, W, Cout, k, seed=B * 10 + W)
    oh, ow = (H + 2 * pad - k) // stride + 1, (W + 2 * pad - k) // stride + 1
    target = np.random.default_rng(6).standard_normal((B, Cout, oh, ow)).astype(np.float32)
    try:
        mx_hip.set_conv_skip_unread_grad_cols(False)
        whole = conv_step(mx_hip, x, w, b, stride, pad, target)
        mx_hip.set_conv_skip_unread_grad_cols(True)
        lead = conv_step(mx_hip, x, w, b, stride, pad, target)
    finally:
        mx_hip.set_conv_skip_unread_grad_cols(True)
    for key in ("out", "loss", "grad_b", "grad_w", "grad_x"):
        np.testing.assert_array_equal(lead[key].view(np.uint32), whole[key].view(np.uint32), err_msg=key)


@pytest.mark.parametrize("B,Cin,H,W,Cout,k,stride,pad", [(2, 3, 6, 5, 4, 3, 1, 1), (1, 2, 7, 7, 3, 3, 2, 2), (4, 16, 14, 14, 32, 3, 1, 1),
                                                         (8, 64, 28, 28, 64, 3, 1, 1)])
def test_conv2d_with_the_column_matrix_stored_or_gathered(mx_hip, B, Cin, H, W, Cout, k, stride, pad):
    """The layer multiplies the column matrix without storing it (hip_conv2d_cols_matmul_f32, mode 2) or stores it with
    im2col first as the reference does (mode 0): the same numbers within the f32 matmul tolerance everywhere, and the same
    bits where both products run on the matrix cores (the two larger cases).  By default (mode 1) a forward without a
    recorded backward gathers, a recorded one stores."""
    x, w, b = conv_inputs(B, Cin, H, W, Cout, k, seed=B * 7 + W)
    oh, ow = (H + 2 * pad - k) // stride + 1, (W + 2 * pad - k) // stride + 1
    target = np.random.default_rng(8).standard_normal((B, Cout, oh, ow)).astype(np.float32)
    try:
        mx_hip.set_conv_gathered_products(0)
        mx_hip.reset_backend_calls()
        stored = conv_step(mx_hip, x, w, b, stride, pad, target)
        calls_stored = mx_hip.backend_calls()
        mx_hip.set_conv_gathered_products(2)
        mx_hip.reset_backend_calls()
        gathered = conv_step(mx_hip, x, w, b, stride, pad, target)
        calls_gathered = mx_hip.backend_calls()
        # the default: gathered exactly when no backward is recorded
        mx_hip.set_conv_gathered_products(1)
        conv = mx_hip.Conv2d(mx_hip.tensor(w), mx_hip.tensor(b), stride=(stride, stride), padding=(pad, pad))
        mx_hip.reset_backend_calls()
        plain = conv.forward(mx_hip.tensor(x)).numpy()
        calls_plain = mx_hip.backend_calls()
        mx_hip.reset_backend_calls()
        conv.forward(mx_hip.tensor(x).with_grad())
        calls_recorded = mx_hip.backend_calls()
    finally:
        mx_hip.set_conv_gathered_products(1)
    assert calls_recorded == calls_plain + 1            # im2col, then the product
    np.testing.assert_array_equal(plain.view(np.uint32), gathered["out"].view(np.uint32))
    assert calls_gathered == calls_stored - 1           # no im2col
    for key in ("out", "loss", "grad_b", "grad_w", "grad_x"):
        scale = np.abs(stored[key]).max() + 1e-30
        assert np.abs(gathered[key] - stored[key]).max() <= 2e-5 * scale, key
        if B * oh * ow >= 128 and Cout >= 32:
            np.testing.assert_array_equal(gathered[key].view(np.uint32), stored[key].view(np.uint32), err_msg=key)


def test_graph_replayed_training_equals_eager(mx_hip):
    """mxt_train records the step as a HIP graph and replays it; every run is compared with the eager loop, with
    eager work and synchronisations in between (the same graph machinery is set up and torn down each time)."""
    from host_programs import mlp_data
    mx = mx_hip
    x, y = mlp_data()

    def run(epochs, graphs):
        mx.set_graph_replay(graphs)
        lin = mx.Linear(mx.tensor(np.array([[0.3, -0.2, 0.5]], np.float32)), mx.tensor(np.array(0.1, np.float32), shape=()))
        xin = mx.tensor(x).with_grad()
        mx.train(lin, xin, mx.tensor(y), 0.01, epochs)
        mx.synchronize()
        replayed = mx.last_train_replayed()
        return lin.weight.numpy(), lin.bias.numpy(), xin.grad().numpy(), replayed
    try:
        for epochs in (40, 41, 100, 75):       # eager until the addresses repeat, whole periods of recorded steps, the rest eager
            w0, b0, g0, r0 = run(epochs, False)
            assert r0 == 0
            w1, b1, g1, r1 = run(epochs, True)
            assert r1 >= epochs // 2 - 4, "the loop fell back to eager launches"
            assert np.array_equal(w0, w1) and np.array_equal(b0, b1) and np.array_equal(g0, g1), epochs
            # eager work between the runs
            t = mx.tensor(np.arange(12, dtype=np.float32).reshape(3, 4)).with_grad()
            t.mul(t).sum_all().backward()
            np.testing.assert_array_equal(t.grad().numpy(), 2 * np.arange(12, dtype=np.float32).reshape(3, 4))
    finally:
        mx.set_graph_replay(True)


def test_run_steps_replays_a_conv_step_and_equals_the_eager_loop(mx_hip):
    """mxt_run_steps with a step written by the caller (Conv2d forward, MSE, backward, zero_grad of the layer, the
    input's gradient accumulating from step to step): eager until the addresses repeat, then replays of a recorded
    graph; the accumulated input gradient is the eager loop's, bit for bit."""
    mx = mx_hip
    rng = np.random.default_rng(21)
    x = rng.standard_normal((4, 8, 12, 12), dtype=np.float32)
    w = rng.uniform(-0.2, 0.2, (6, 8, 3, 3)).astype(np.float32)
    b = rng.uniform(-0.2, 0.2, (6,)).astype(np.float32)
    t = rng.standard_normal((4, 6, 12, 12), dtype=np.float32)

    def run(steps, graphs):
        mx.set_graph_replay(graphs)
        conv = mx.Conv2d(mx.tensor(w), mx.tensor(b), stride=(1, 1), padding=(1, 1))
        xin, target = mx.tensor(x).with_grad(), mx.tensor(t)

        def step():
            loss = mx.mse_loss(conv.forward(xin), target)
            loss.backward()
            conv.zero_grad()
        mx.run_steps(step, steps)
        mx.synchronize()
        return xin.grad().numpy(), mx.last_train_replayed()
    try:
        for steps in (40, 57):
            g0, r0 = run(steps, False)
            assert r0 == 0
            g1, r1 = run(steps, True)
            assert r1 >= steps // 2 - 4, "the loop fell back to eager launches"
            np.testing.assert_array_equal(g0.view(np.uint32), g1.view(np.uint32))
        # few steps: eager
        g2, r2 = run(5, True)
        assert r2 == 0
    finally:
        mx.set_graph_replay(True)


def test_conv_input_gradient_accumulated_by_col2im_equals_the_separate_add(mx_hip):
    """From the second backward() on, the input (a leaf) has a gradient and the layer's closure lets col2im add into it
    (hip_conv2d_col2im_add_f32) instead of handing back a tensor for backward() to add: the accumulated gradient after
    several steps is the bits of the op-by-op way, also when the input feeds a second consumer."""
    mx = mx_hip
    rng = np.random.default_rng(33)
    x = rng.standard_normal((2, 4, 8, 8), dtype=np.float32)
    w = rng.uniform(-0.3, 0.3, (4, 4, 3, 3)).astype(np.float32)
    b = rng.uniform(-0.3, 0.3, (4,)).astype(np.float32)
    t = rng.standard_normal((2, 4, 8, 8), dtype=np.float32)

    def run(fused):
        mx.set_fused_nn_kernels(fused)
        conv = mx.Conv2d(mx.tensor(w), mx.tensor(b), stride=(1, 1), padding=(1, 1))
        xin, target = mx.tensor(x).with_grad(), mx.tensor(t)
        grads = []
        for _ in range(4):
            y = conv.forward(xin)
            loss = mx.mse_loss(y.add(xin.mul(xin)), target)           # xin also reaches the loss directly
            loss.backward()
            conv.zero_grad()
            grads.append(xin.grad().numpy().copy())
        return grads
    try:
        a, c = run(True), run(False)
    finally:
        mx.set_fused_nn_kernels(True)
    for step, (ga, gc) in enumerate(zip(a, c)):
        np.testing.assert_array_equal(ga.view(np.uint32), gc.view(np.uint32), err_msg=str(step))


def test_run_steps_hands_on_a_failure_of_the_step(mx_hip):
    """An exception inside the step ends the loop (and an open recording) and reaches the caller as it was raised; the
    library works on afterwards."""
    mx = mx_hip
    a = mx.tensor(np.ones((3, 4), np.float32)).with_grad()
    calls = []

    def step():
        calls.append(1)
        if len(calls) == 20:
            raise KeyError("step 20")
        a.mul(a).sum_all().backward()
    with pytest.raises(KeyError):
        mx.run_steps(step, 64)
    assert len(calls) == 20
    mx.synchronize()
    a2 = mx.tensor(np.full((3, 4), 2.0, np.float32)).with_grad()
    a2.mul(a2).sum_all().backward()
    np.testing.assert_array_equal(a2.grad().numpy(), np.full((3, 4), 4.0, np.float32))


@pytest.mark.parametrize("case", TKAT, ids=[f"{c['program'][0][1]}@{c['cite'].split('/')[-1]}" for c in TKAT])
def test_reference_tensor_cases_bf16(mx_hip, case):
    check_case(run_case(mx_hip, case, dtype="bf16"), case, tol=0.1)


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
@pytest.mark.parametrize("op", ["add", "mul", "div", "exp", "relu", "gelu"])
@pytest.mark.parametrize("case", ["contig", "bcast", "transposed"])
def test_elementwise_forward_backward_matches_oracle(mx_hip, mx_oracle, op, case, dtype):
    """configs[1] through the tensor API at a small size: forward value and every gradient, both dtypes (the bf16 gelu
    closure runs mostly in f32 after the reference's promotions).  Elementwise kernels are bit-exact; the broadcast
    gradient is a column sum (different order) and gets the reduction tolerance."""
    if op in ("exp", "relu", "gelu") and case == "bcast":
        pytest.skip("unary ops have no broadcast case")
    got = elementwise_program(mx_hip, op, case, dtype, R=48, C=72)
    ref = elementwise_program(mx_oracle, op, case, dtype, R=48, C=72)
    assert got["z.dtype"] == ref["z.dtype"] and got["gx.dtype"] == ref["gx.dtype"]
    np.testing.assert_array_equal(got["z"], ref["z"])
    np.testing.assert_array_equal(got["gx"], ref["gx"])
    if "gy" in ref:
        if case == "bcast":
            tol = 1e-5 if dtype == "f32" else 1e-2
            assert np.max(np.abs(got["gy"] - ref["gy"])) <= tol * 48 * np.max(np.abs(ref["gy"]) + 1)
        else:
            np.testing.assert_array_equal(got["gy"], ref["gy"])
