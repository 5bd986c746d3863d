"""Tensor-level programs that run on any host-layer library (maidenx_amd.tensor.Host): the reference's own
tensor tests (tests/golden/reference_tensor_kat.json) and the two training workloads."""
import json
import os

import numpy as np

TKAT = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "reference_tensor_kat.json")))["cases"]


def run_case(mx, case, dtype="f32"):
    """Returns {name: ndarray} for every named tensor and '<input>.grad'."""
    env = {}
    for name, spec in case["inputs"].items():
        t = mx.tensor(np.array(spec["data"], np.float32).reshape(spec["shape"]), dtype=dtype)
        if spec.get("grad"):
            t.with_grad()
        env[name] = t
    for step in case["program"]:
        out, op, src, *args = step
        x = env[src]
        if op in ("add", "sub", "mul", "div", "matmul"):
            r = getattr(x, op)(env[args[0]])
        elif op == "mse_loss":
            r = mx.mse_loss(x, env[args[0]])
        else:
            r = getattr(x, op)(*args)
        env[out] = r
    if case.get("backward"):
        env[case["backward"]].backward()
    res = {k: v.numpy() for k, v in env.items()}
    res.update({f"{k}.shape": v.shape for k, v in env.items()})
    res.update({f"{k}.strides": v.strides for k, v in env.items()})
    for name in case["inputs"]:
        g = env[name].grad()
        if g is not None:
            res[f"{name}.grad"] = g.numpy()
    return res


def check_case(res, case, tol=None):
    tol = case["tol"] if tol is None else tol
    for key, exp in case["expect"].items():
        got = np.asarray(res[key], np.float64).ravel()
        exp = np.asarray(exp, np.float64)
        if tol == 0:
            assert np.array_equal(got.astype(np.float32), exp.astype(np.float32)), (case["cite"], key, got, exp)
        else:
            assert np.all(np.abs(got - exp) < tol), (case["cite"], key, got, exp)
    for key, shp in case.get("expect_shape", {}).items():
        assert tuple(res[f"{key}.shape"]) == tuple(shp), (case["cite"], key)
    for key, st in case.get("expect_strides", {}).items():
        assert tuple(res[f"{key}.strides"]) == tuple(st), (case["cite"], key)


# ---- configs[0]: examples/device/cpu.rs:10-38 ---------------------------------------------------------
def mlp_data(n=10000):
    i = np.arange(n)
    x = np.stack([(i % 100) / 100.0, (i % 100 + 1) / 100.0, (i % 100 + 2) / 100.0], 1).astype(np.float32)
    y = ((i % 100) * 10 / 1000.0).astype(np.float32).reshape(-1, 1)
    return x, y


def mlp_run(mx, epochs, n=10000, w0=(0.3, -0.2, 0.5), b0=0.1, lr=0.01):
    x, y = mlp_data(n)
    lin = mx.Linear(mx.tensor(np.array([w0], np.float32)), mx.tensor(np.array(b0, np.float32), shape=()))
    xin = mx.tensor(x).with_grad()
    losses = mx.train(lin, xin, mx.tensor(y), lr, epochs, record_losses=True)
    return {"losses": losses, "weight": lin.weight.numpy(), "bias": lin.bias.numpy(), "input_grad": xin.grad().numpy()}


def mlp_numpy(epochs, n=10000, w0=(0.3, -0.2, 0.5), b0=0.1, lr=0.01):
    """Full-batch gradient descent on mean((xW^T + b - y)^2) in float64: what the loop computes."""
    x, y = mlp_data(n)
    x, y = x.astype(np.float64), y.astype(np.float64)
    w, b = np.array([w0], np.float64), float(b0)
    losses = []
    for _ in range(epochs):
        d = x @ w.T + b - y
        losses.append(float(np.mean(d * d)))
        g = 2.0 * d / d.size
        w -= lr * (g.T @ x)
        b -= lr * float(g.sum())
    return np.array(losses), w, b


def mlp_adam_run(mx, epochs, n=2000, w0=(0.3, -0.2, 0.5), b0=0.1, hyper=(0.01, 0.9, 0.999, 1e-8), fused=True):
    """The README model trained with Adam through the tensor API (forward, MSE, backward, step, zero_grad)."""
    x, y = mlp_data(n)
    lin = mx.Linear(mx.tensor(np.array([w0], np.float32)), mx.tensor(np.array(b0, np.float32), shape=()))
    xin, yt = mx.tensor(x), mx.tensor(y)
    opt = mx.Adam(*hyper)
    opt.set_fused(fused)
    losses = []
    for _ in range(epochs):
        loss = mx.mse_loss(lin.forward(xin), yt)
        losses.append(float(loss.numpy()))
        loss.backward()
        opt.step(lin)
        lin.zero_grad()
    return {"losses": np.array(losses), "weight": lin.weight.numpy(), "bias": lin.bias.numpy()}


def mlp_adam_numpy(epochs, n=2000, w0=(0.3, -0.2, 0.5), b0=0.1, hyper=(0.01, 0.9, 0.999, 1e-8)):
    """adam.rs:34-88 in float64 arithmetic on float64 gradients, with the reference's beta^(t+1) bias terms."""
    lr, b1, b2, eps = hyper
    x, y = mlp_data(n)
    x, y = x.astype(np.float64), y.astype(np.float64)
    p = [np.array([w0], np.float64), np.array(float(b0))]
    m, v = [np.zeros_like(q) for q in p], [np.zeros_like(q) for q in p]
    losses = []
    for t in range(1, epochs + 1):
        d = x @ p[0].T + p[1] - y
        losses.append(float(np.mean(d * d)))
        g = 2.0 * d / d.size
        grads = [g.T @ x, np.array(float(g.sum()))]
        c1, c2 = 1.0 - b1 ** (t + 1), 1.0 - b2 ** (t + 1)
        lr_t = lr * np.sqrt(c2) / c1
        for i in range(2):
            m[i] = m[i] * b1 + grads[i] * (1.0 - b1)
            v[i] = v[i] * b2 + grads[i] ** 2 * (1.0 - b2)
            p[i] = p[i] - (m[i] / c1) / (np.sqrt(v[i] / c2) + eps) * lr_t
    return np.array(losses), p[0], float(p[1])


# ---- configs[4]: Conv2d + MSE forward/backward ---------------------------------------------------------
def conv_inputs(B, Cin, H, W, Cout, k, seed):
    rng = np.random.default_rng(seed)
    bound = 1.0 / np.sqrt(Cin * k * k)
    x = rng.standard_normal((B, Cin, H, W)).astype(np.float32)
    w = rng.uniform(-bound, bound, (Cout, Cin, k, k)).astype(np.float32)
    b = rng.uniform(-bound, bound, (Cout,)).astype(np.float32)
    return x, w, b


def conv_step(mx, x, w, b, stride, pad, target):
    xt = mx.tensor(x).with_grad()
    conv = mx.Conv2d(mx.tensor(w), mx.tensor(b), stride=(stride, stride), padding=(pad, pad))
    out = conv.forward(xt)
    loss = mx.mse_loss(out, mx.tensor(target))
    loss.backward()
    return {"out": out.numpy(), "loss": loss.numpy(), "grad_x": xt.grad().numpy(), "grad_w": conv.weight.grad().numpy(),
            "grad_b": conv.bias.grad().numpy()}


def conv_numpy(x, w, b, stride, pad, target):
    """The data flow of nn/layers/conv.rs:185-310 in float64 numpy, written from the layer's own steps rather than
    from the kernels: im2col produces [B][C*kh*kw][oh*ow] (crates/maidenx_cpu/src/nn/conv.rs:43-48), the layer
    reads that buffer as a [B*oh*ow, C*kh*kw] matrix (conv.rs:345-348), multiplies by W^T, views the product as
    [B,oh,ow,Cout] and permutes.  Backward: grad_cols = grad_flat.W is handed to col2im as if it were
    [B][C*kh*kw][oh*ow], entries at flat index >= B*C*H*W dropped (conv.rs:393; cpu/nn/conv.rs:135); grad_w =
    cols^T.grad_flat reshaped (not transposed) to [Cout,Cin,kh,kw] (conv.rs:276-278)."""
    x64, w64 = x.astype(np.float64), w.astype(np.float64)
    B, Cin, H, W = x.shape
    Cout, _, kh, kw = w.shape
    oh, ow = (H + 2 * pad - kh) // stride + 1, (W + 2 * pad - kw) // stride + 1
    xp = np.pad(x64, ((0, 0), (0, 0), (pad, pad), (pad, pad)))
    col = np.zeros((B, Cin, kh, kw, oh, ow))
    for i in range(kh):
        for j in range(kw):
            col[:, :, i, j] = xp[:, :, i:i + stride * oh:stride, j:j + stride * ow:stride]
    cols = col.reshape(B * oh * ow, Cin * kh * kw)             # the reinterpretation
    wm = w64.reshape(Cout, Cin * kh * kw)
    out = (cols @ wm.T).reshape(B, oh, ow, Cout).transpose(0, 3, 1, 2) + b.astype(np.float64)[None, :, None, None]
    d = out - target
    loss = np.mean(d * d)
    go = 2.0 * d / d.size
    grad_flat = go.transpose(0, 2, 3, 1).reshape(B * oh * ow, Cout)
    grad_cols = (grad_flat @ wm).ravel().copy()
    grad_cols[B * Cin * H * W:] = 0.0                          # dropped by col2im
    gc = grad_cols.reshape(B, Cin, kh, kw, oh, ow)
    gxp = np.zeros_like(xp)
    for i in range(kh):
        for j in range(kw):
            gxp[:, :, i:i + stride * oh:stride, j:j + stride * ow:stride] += gc[:, :, i, j]
    gx = gxp[:, :, pad:pad + H, pad:pad + W]
    gw = (cols.T @ grad_flat).reshape(Cout, Cin, kh, kw)
    return {"out": out, "loss": loss, "grad_x": gx, "grad_w": gw, "grad_b": go.sum((0, 2, 3))}


# ---- bf16 helpers and the elementwise forward + backward programs of configs[1] ------------------------
def bf16_round(a):
    """float32 values rounded to bf16 (nearest even), returned as float32."""
    x = np.ascontiguousarray(a, dtype=np.float32).view(np.uint32).astype(np.uint64)
    r = ((x + 0x7FFF + ((x >> 16) & 1)) >> 16) << 16
    return r.astype(np.uint32).view(np.float32).reshape(np.shape(a))


def elementwise_program(mx, op, case, dtype, R=12, C=20, seed=5):
    """z = op(x[, y]); z.backward().  case: contig | bcast (rhs [1,C]) | transposed (x is a transposed view)."""
    rng = np.random.default_rng(seed)
    xs = rng.standard_normal((C, R) if case == "transposed" else (R, C)).astype(np.float32)
    ys = (rng.standard_normal((1, C) if case == "bcast" else (R, C)) + 2.5).astype(np.float32)
    base = mx.tensor(xs, dtype=dtype).with_grad()
    x = base.transpose(0, 1) if case == "transposed" else base
    y = mx.tensor(ys, dtype=dtype).with_grad()
    z = getattr(x, op)(y) if op in ("add", "mul", "div") else getattr(x, op)()
    z.backward()
    out = {"z": z.numpy(), "gx": base.grad().numpy(), "z.dtype": z.dtype, "gx.dtype": base.grad().dtype, "xs": xs, "ys": ys}
    if op in ("add", "mul", "div"):
        out["gy"] = y.grad().numpy()
    return out
