"""GPU parity at the full sizes of the benchmark configurations, through checks that do not need the (slow) CPU oracle at
those sizes: single IEEE operations against numpy bit for bit, reductions and products against float64 numpy,
data-movement kernels against numpy indexing, and size-independent properties (linearity, adjointness,
transposition symmetry)."""
import numpy as np
import pytest

from helpers import In, Out, f32_to_bf16, meta_binary, meta_conv, meta_matmul, meta_pad, meta_reduce, meta_sum_to_shape, meta_unary, to_float

pytestmark = pytest.mark.gpu

R = C = 8192


def same_bits(a, b):
    return np.array_equal(np.ascontiguousarray(a).view(np.uint8), np.ascontiguousarray(b).view(np.uint8))


@pytest.fixture(scope="module")
def xy():
    r = np.random.default_rng(0x5EED0002)
    return r.standard_normal((R, C), dtype=np.float32), r.standard_normal((R, C), dtype=np.float32)


@pytest.mark.parametrize("case", ["contiguous", "rhs_row", "lhs_transposed"])
def test_elementwise_8192_f32_bit_exact(hip, xy, case):
    x, y = xy
    n = R * C
    if case == "contiguous":
        md, lhs, rhs, a, b = meta_binary([R, C], [C, 1], [C, 1]), x, y, x, y
    elif case == "rhs_row":
        row = y[0].copy()
        md, lhs, rhs, a, b = meta_binary([R, C], [C, 1], [0, 1]), x, row, x, row[None, :]
    else:
        md, lhs, rhs, a, b = meta_binary([R, C], [1, R], [C, 1]), x, y, x.T, y      # x's buffer viewed transposed
    for op, fn in (("add", np.add), ("mul", np.multiply)):
        (out,) = hip.call(f"{op}_f32", n, 2, md, In(lhs.ravel()), In(rhs.ravel()), Out(n, "f32"))
        assert same_bits(out.reshape(R, C), fn(a, b)), (op, case)
    (out,) = hip.call("div_f32", n, 2, md, In(lhs.ravel()), In(rhs.ravel()), Out(n, "f32"))
    with np.errstate(all="ignore"):
        want = np.divide(a, b)
    zero = np.broadcast_to(b == 0, want.shape)          # the float32 normal generator does emit a few exact zeros
    want = np.where(zero, np.where(a == 0, np.float32(0), np.float32(np.inf)), want)   # crates/maidenx_cpu/src/ops/binary.rs:440-452
    assert same_bits(out.reshape(R, C), want.astype(np.float32))


def test_elementwise_8192_bf16_bit_exact(hip, xy):
    x, y = xy
    xb, yb = f32_to_bf16(x.ravel()), f32_to_bf16(y.ravel())
    n = R * C
    (out,) = hip.call("mul_bf16", n, 2, meta_binary([R, C], [C, 1], [C, 1]), In(xb), In(yb), Out(n, "bf16"))
    want = f32_to_bf16(to_float(xb, "bf16") * to_float(yb, "bf16"))
    assert same_bits(out, want)
    (out,) = hip.call("relu_bf16", n, 2, meta_unary([R, C], [1, R]), In(xb), Out(n, "bf16"))   # transposed view
    want = np.maximum(to_float(xb, "bf16").reshape(C, R).T, 0).ravel()
    assert same_bits(to_float(out, "bf16"), want.astype(np.float32))


def test_unary_8192_f32(hip, xy):
    x, _ = xy
    n = R * C
    (out,) = hip.call("relu_f32", n, 2, meta_unary([R, C], [C, 1]), In(x.ravel()), Out(n, "f32"))
    assert same_bits(out, np.where(x > 0, x, np.float32(0)).ravel())
    (out,) = hip.call("exp_f32", n, 2, meta_unary([R, C], [C, 1]), In(x.ravel()), Out(n, "f32"))
    ref = np.exp(x.astype(np.float64)).ravel()
    assert np.max(np.abs(out - ref) / ref) < 1.2e-7                                    # within 1 ulp of the true value
    # gelu: odd-symmetry identity of the tanh form, gelu(x) - gelu(-x) = x (to rounding)
    (g1,) = hip.call("gelu_f32", n, 2, meta_unary([R, C], [C, 1]), In(x.ravel()), Out(n, "f32"))
    (g2,) = hip.call("gelu_f32", n, 2, meta_unary([R, C], [C, 1]), In((-x).ravel()), Out(n, "f32"))
    assert np.max(np.abs((g1.astype(np.float64) - g2) - x.ravel())) < 1e-6


@pytest.mark.parametrize("shape", [(8192, 8192), (64, 512, 1024)], ids=["8192x8192", "64x512x1024"])
def test_reductions_fullsize(hip, shape):
    r = np.random.default_rng(0x5EED0003)
    x = r.uniform(-1, 1, shape).astype(np.float32)
    n = x.size
    strides = [int(np.prod(shape[i + 1:])) for i in range(len(shape))]
    x64 = x.astype(np.float64)
    for dim in range(len(shape)):
        L = shape[dim]
        md = meta_reduce(list(shape), strides, dim)
        (s,) = hip.call("sum_f32", n, len(shape), 1, md, In(x.ravel()), Out(n // L, "f32"))
        scale = np.abs(x64).sum(dim).ravel()
        assert np.max(np.abs(s - x64.sum(dim).ravel()) / scale) <= 1e-5
        (m,) = hip.call("mean_f32", n, len(shape), 1, md, In(x.ravel()), Out(n // L, "f32"))
        assert np.max(np.abs(m - x64.mean(dim).ravel()) / (scale / L)) <= 1e-5
        (mx,) = hip.call("max_f32", n, len(shape), 1, md, In(x.ravel()), Out(n // L, "f32"))
        assert same_bits(mx, x.max(dim).ravel())                                       # exact, order-independent
    if len(shape) == 3:
        md = meta_sum_to_shape(list(shape), strides, [1, shape[1], 1])
        (s,) = hip.call("sum_to_shape_f32", n, 3, md, In(x.ravel()), Out(shape[1], "f32"))
        assert np.max(np.abs(s - x64.sum((0, 2))) / np.abs(x64).sum((0, 2))) <= 1e-5
    else:
        md = meta_sum_to_shape(list(shape), strides, list(shape))
        (s,) = hip.call("sum_to_shape_f32", n, 2, md, In(x.ravel()), Out(n, "f32"))
        assert same_bits(s, (x + np.float32(0)).ravel())                               # identity, -0 -> +0


@pytest.mark.parametrize("dt", ["f32", "bf16"])
def test_matmul_4096_sampled_and_linear(hip, dt):
    M = K = N = 4096
    r = np.random.default_rng(0x5EED0004)
    a = r.standard_normal((M, K), dtype=np.float32)
    b = (r.standard_normal((K, N), dtype=np.float32) * np.float32(0.02))
    go = r.standard_normal((M, N), dtype=np.float32)
    st = (lambda v: f32_to_bf16(v.ravel())) if dt == "bf16" else (lambda v: v.ravel())
    val = (lambda s: to_float(s, dt).astype(np.float64))
    sa, sb, sg = st(a), st(b), st(go)
    av, bv, gv = val(sa).reshape(M, K), val(sb).reshape(K, N), val(sg).reshape(M, N)
    md = meta_matmul([M, N], [M, K], [K, N], [K, 1], [N, 1])
    (c,) = hip.call(f"matmul_{dt}", M * N, md, In(sa), In(sb), Out(M * N, dt))
    ga, gb = hip.call(f"matmul_backward_{dt}", M * K, K * N, md, In(sg), In(sa), In(sb), Out(M * K, dt), Out(K * N, dt))
    tol = 1e-5 if dt == "f32" else 1e-2
    rows = r.choice(M, 48, replace=False)
    cv = val(c).reshape(M, N)
    assert np.max(np.abs(cv[rows] - av[rows] @ bv) / (np.abs(av[rows]) @ np.abs(bv))) <= tol
    gav = val(ga).reshape(M, K)
    assert np.max(np.abs(gav[rows] - gv[rows] @ bv.T) / (np.abs(gv[rows]) @ np.abs(bv.T))) <= tol
    krows = r.choice(K, 48, replace=False)
    gbv = val(gb).reshape(K, N)
    assert np.max(np.abs(gbv[krows] - av[:, krows].T @ gv) / (np.abs(av[:, krows].T) @ np.abs(gv))) <= tol
    # every output tile is touched: column and row checksums of C against (1^T A) B and A (B 1)
    assert np.max(np.abs(cv.sum(0) - av.sum(0) @ bv) / (np.abs(av).sum(0) @ np.abs(bv))) <= tol
    assert np.max(np.abs(cv.sum(1) - av @ bv.sum(1)) / (np.abs(av) @ np.abs(bv).sum(1))) <= tol
    assert np.max(np.abs(gbv.sum(1) - av.T @ gv.sum(1)) / (np.abs(av.T) @ np.abs(gv).sum(1))) <= tol


def test_matmul_batched_config(hip):
    Bt, M, K, N = 32, 512, 1024, 1024
    r = np.random.default_rng(7)
    a = r.standard_normal((Bt, M, K), dtype=np.float32)
    b = r.standard_normal((Bt, K, N), dtype=np.float32) * np.float32(0.02)
    md = meta_matmul([Bt, M, N], [Bt, M, K], [Bt, K, N], [M * K, K, 1], [K * N, N, 1])
    (c,) = hip.call("matmul_f32", Bt * M * N, md, In(a.ravel()), In(b.ravel()), Out(Bt * M * N, "f32"))
    c = c.reshape(Bt, M, N).astype(np.float64)
    for bi in (0, 13, 31):
        ref = a[bi].astype(np.float64) @ b[bi]
        assert np.max(np.abs(c[bi] - ref) / (np.abs(a[bi].astype(np.float64)) @ np.abs(b[bi]))) <= 1e-5


def test_conv_kernels_config_size(hip):
    Bn, Cc, H, W, k = 32, 64, 56, 56, 3
    r = np.random.default_rng(0x5EED0005)
    x = r.standard_normal((Bn, Cc, H, W), dtype=np.float32)
    ncol = Bn * Cc * k * k * H * W
    md = meta_conv(Bn, Cc, H, W, k, k, H, W, 1, 1, 1, 1)
    (col,) = hip.call("conv2d_im2col_f32", ncol, md, In(x.ravel()), Out(ncol, "f32"))
    xp = np.pad(x, ((0, 0), (0, 0), (1, 1), (1, 1)))
    ref = np.empty((Bn, Cc, k, k, H, W), np.float32)
    for i in range(k):
        for j in range(k):
            ref[:, :, i, j] = xp[:, :, i:i + H, j:j + W]
    assert same_bits(col, ref.ravel())
    # col2im of the whole column matrix: every pixel is the sum of its (up to 9) copies, in a fixed order
    (img,) = hip.call("conv2d_col2im_f32", ncol, md, In(col), Out(x.size, "f32"))
    cnt = np.zeros((H + 2, W + 2))
    for i in range(k):
        for j in range(k):
            cnt[i:i + H, j:j + W] += 1
    cnt = cnt[1:H + 1, 1:W + 1]
    np.testing.assert_allclose(img.reshape(x.shape), x * cnt.astype(np.float32), rtol=1e-6, atol=0)
    # the layer's call: num_els = B*C*H*W, columns beyond it dropped (nn/layers/conv.rs:393)
    (img2,) = hip.call("conv2d_col2im_f32", x.size, md, In(col), Out(x.size, "f32"))
    g = ref.ravel().copy()
    g[x.size:] = 0
    g = g.reshape(Bn, Cc, k, k, H, W).astype(np.float64)
    acc = np.zeros((Bn, Cc, H + 2, W + 2))
    for i in range(k):
        for j in range(k):
            acc[:, :, i:i + H, j:j + W] += g[:, :, i, j]
    np.testing.assert_allclose(img2.reshape(x.shape), acc[:, :, 1:H + 1, 1:W + 1], rtol=1e-6, atol=1e-6)
    # pad [32,64,56,56] -> [32,64,58,58] and its backward
    mdp = meta_pad([Bn, Cc, H, W], [Cc * H * W, H * W, W, 1], 0, [Bn, Cc, H + 2, W + 2], [(0, 0), (0, 0), (1, 1), (1, 1)])
    (p,) = hip.call("pad_with_constant_f32", x.size, xp.size, 4, mdp, In(x.ravel()), Out(xp.size, "f32"), 0.0)
    assert same_bits(p, xp.ravel())
    (gi,) = hip.call("pad_with_constant_backward_f32", x.size, xp.size, 4, mdp, In(xp.ravel()), Out(x.size, "f32"))
    assert same_bits(gi, (x + np.float32(0)).ravel())


@pytest.mark.parametrize("mode,np_mode", [("reflection", "reflect"), ("replication", "edge")])
def test_edge_pads_config_size(hip, mode, np_mode):
    """[32,64,56,56] padded by (1,2) x (2,1) on H and W: forward against numpy.pad bit for bit, backward against the
    transpose of that map accumulated in float64 (at most 9 terms per element) and through the adjoint identity."""
    Bn, Cc, H, W = 32, 64, 56, 56
    pads = [(0, 0), (0, 0), (1, 2), (2, 1)]
    r = np.random.default_rng(0x5EED0006)
    x = r.standard_normal((Bn, Cc, H, W), dtype=np.float32)
    xp = np.pad(x, pads, mode=np_mode)
    md = meta_pad([Bn, Cc, H, W], [Cc * H * W, H * W, W, 1], 0, list(xp.shape), pads)
    (p,) = hip.call(f"pad_with_{mode}_f32", x.size, xp.size, 4, md, In(x.ravel()), Out(xp.size, "f32"))
    assert same_bits(p, xp.ravel())
    go = r.standard_normal(xp.shape, dtype=np.float32)
    (gi,) = hip.call(f"pad_with_{mode}_backward_f32", x.size, xp.size, 4, md, In(go.ravel()), Out(x.size, "f32"))
    # the index map of the forward, from padding an index tensor
    idx = np.pad(np.arange(H * W, dtype=np.int64).reshape(H, W), pads[2:], mode=np_mode).ravel()
    ref = np.zeros((Bn * Cc, H * W))
    np.add.at(ref, (slice(None), idx), go.reshape(Bn * Cc, -1).astype(np.float64))
    np.testing.assert_allclose(gi.reshape(Bn * Cc, H * W), ref, rtol=2e-6, atol=2e-6)
    assert abs(float(np.vdot(xp.astype(np.float64), go)) - float(np.vdot(x.astype(np.float64), gi.reshape(x.shape)))) < 1e-6 * x.size ** 0.5 * 10


def test_conv_layer_products_config_size(hip):
    """The three f32 products of the Conv2d(64->64, 3x3) step at [32,64,56,56] (64x64 tiles, the unchecked body,
    split-K for the weight gradient): sampled rows and columns against float64."""
    M, K, N = 32 * 56 * 56, 576, 64
    r = np.random.default_rng(0x5EED0007)
    cols = r.standard_normal((M, K), dtype=np.float32)
    w = (r.standard_normal((N, K), dtype=np.float32) * np.float32(0.05))
    g = r.standard_normal((M, N), dtype=np.float32)
    rows = r.integers(0, M, 64)
    (out,) = hip.call("matmul_f32", M * N, meta_matmul([M, N], [M, K], [K, N], [K, 1], [1, K]), In(cols.ravel()), In(w.ravel()), Out(M * N, "f32"))
    np.testing.assert_allclose(out.reshape(M, N)[rows], cols[rows].astype(np.float64) @ w.T.astype(np.float64), rtol=2e-5, atol=2e-5)
    (gin,) = hip.call("matmul_f32", M * K, meta_matmul([M, K], [M, N], [N, K], [N, 1], [K, 1]), In(g.ravel()), In(w.ravel()), Out(M * K, "f32"))
    np.testing.assert_allclose(gin.reshape(M, K)[rows], g[rows].astype(np.float64) @ w.astype(np.float64), rtol=2e-5, atol=2e-5)
    (gw,) = hip.call("matmul_f32", K * N, meta_matmul([K, N], [K, M], [M, N], [1, K], [N, 1]), In(cols.ravel()), In(g.ravel()), Out(K * N, "f32"))
    ks = r.integers(0, K, 16)
    np.testing.assert_allclose(gw.reshape(K, N)[ks], cols[:, ks].T.astype(np.float64) @ g.astype(np.float64), rtol=1e-4, atol=2e-3)


def test_fused_adam_16m_elements_bit_exact(hip):
    """Every step of adam.rs:46-86 is one correctly rounded IEEE operation, so numpy's float32 arithmetic gives the
    reference's bits; three steps on 2^24 elements."""
    n = 1 << 24
    r = np.random.default_rng(0x5EED0008)
    p = r.standard_normal(n, dtype=np.float32)
    m, v = np.zeros(n, np.float32), np.zeros(n, np.float32)
    hp, hm, hv = p.copy(), m.copy(), v.copy()
    f = np.float32
    lr, b1, b2, eps = 0.001, 0.9, 0.999, 1e-8
    from helpers import InOut
    for t in range(1, 4):
        g = r.standard_normal(n, dtype=np.float32)
        c1, c2 = 1 - b1 ** (t + 1), 1 - b2 ** (t + 1)
        sc = [f(b1), f(1 - b1), f(b2), f(1 - b2), f(c1), f(c2), f(eps), f(lr * np.sqrt(c2) / c1)]
        m = m * sc[0] + g * sc[1]
        v = v * sc[2] + (g * g) * sc[3]
        p = p - ((m / sc[4]) / (np.sqrt(v / sc[5]) + sc[6])) * sc[7]
        hp, hm, hv = hip.call("adam_step_f32", n, InOut(hp), In(g), InOut(hm), InOut(hv), *[float(c) for c in sc])
        assert same_bits(hm, m) and same_bits(hv, v) and same_bits(hp, p), t


@pytest.mark.parametrize("dt", ["f32", "bf16"])
def test_matmul_batched_config_forward_and_backward(hip, dt):
    """[32,512,1024] x [32,1024,1024]: forward, dA = dC.B^T and dB = A^T.dC of sampled batches against float64, and
    checksums over every batch (so that no batch or tile is skipped)."""
    Bt, M, K, N = 32, 512, 1024, 1024
    r = np.random.default_rng(0x5EED0014)
    a = r.standard_normal((Bt, M, K), dtype=np.float32)
    b = r.standard_normal((Bt, K, N), dtype=np.float32) * np.float32(0.02)
    go = r.standard_normal((Bt, M, N), dtype=np.float32)
    st = (lambda v: f32_to_bf16(v.ravel())) if dt == "bf16" else (lambda v: v.ravel())
    val = lambda s, shape: to_float(s, dt).astype(np.float64).reshape(shape)
    sa, sb, sg = st(a), st(b), st(go)
    av, bv, gv = val(sa, a.shape), val(sb, b.shape), val(sg, go.shape)
    md = meta_matmul([Bt, M, N], [Bt, M, K], [Bt, K, N], [M * K, K, 1], [K * N, N, 1])
    tol = 1e-5 if dt == "f32" else 1e-2
    (c,) = hip.call(f"matmul_{dt}", Bt * M * N, md, In(sa), In(sb), Out(Bt * M * N, dt))
    ga, gb = hip.call(f"matmul_backward_{dt}", Bt * M * K, Bt * K * N, md, In(sg), In(sa), In(sb), Out(Bt * M * K, dt), Out(Bt * K * N, dt))
    cv, gav, gbv = val(c, go.shape), val(ga, a.shape), val(gb, b.shape)
    for bi in (0, 7, 18, 31):
        assert np.max(np.abs(cv[bi] - av[bi] @ bv[bi]) / (np.abs(av[bi]) @ np.abs(bv[bi]))) <= tol, ("fwd", bi)
        assert np.max(np.abs(gav[bi] - gv[bi] @ bv[bi].T) / (np.abs(gv[bi]) @ np.abs(bv[bi].T))) <= tol, ("dA", bi)
        assert np.max(np.abs(gbv[bi] - av[bi].T @ gv[bi]) / (np.abs(av[bi].T) @ np.abs(gv[bi]))) <= tol, ("dB", bi)
    # row sums of every batch: C 1 = A (B 1), dA 1 = dC (B^T 1), dB 1 = A^T (dC 1)
    ones_n, ones_k = np.ones(N), np.ones(K)
    assert np.max(np.abs(cv @ ones_n - np.einsum("bmk,bk->bm", av, bv @ ones_n)) / np.einsum("bmk,bk->bm", np.abs(av), np.abs(bv) @ ones_n)) <= tol
    assert np.max(np.abs(gav @ ones_k - np.einsum("bmn,bn->bm", gv, np.einsum("bkn->bn", bv))) / np.einsum("bmn,bn->bm", np.abs(gv), np.einsum("bkn->bn", np.abs(bv)))) <= tol
    assert np.max(np.abs(gbv @ ones_n - np.einsum("bmk,bm->bk", av, gv @ ones_n)) / np.einsum("bmk,bm->bk", np.abs(av), np.abs(gv) @ ones_n)) <= tol


@pytest.mark.parametrize("case", ["rhs_row", "lhs_transposed"])
def test_elementwise_8192_bf16_broadcast_and_transposed(hip, xy, case):
    """bf16 add / div bit for bit against the f32-operation-then-round model, exp / gelu against the library's own results
    on the 65536 codes (which test_unary_transcendental_16bit pins to the oracle), on a [1,8192] rhs and a transposed lhs."""
    x, y = xy
    xb, yb = f32_to_bf16(x.ravel()), f32_to_bf16(y.ravel())
    xf, yf = to_float(xb, "bf16").reshape(R, C), to_float(yb, "bf16").reshape(R, C)
    n = R * C
    if case == "rhs_row":
        md, rhs, a, b = meta_binary([R, C], [C, 1], [0, 1]), yb[:C], xf, yf[:1]
        mdu, au = meta_unary([R, C], [C, 1]), xb.reshape(R, C)
    else:
        md, rhs, a, b = meta_binary([R, C], [1, R], [C, 1]), yb, xf.T, yf
        mdu, au = meta_unary([R, C], [1, R]), xb.reshape(C, R).T
    (out,) = hip.call("add_bf16", n, 2, md, In(xb), In(rhs), Out(n, "bf16"))
    assert same_bits(out.reshape(R, C), f32_to_bf16(a + b).reshape(R, C))
    (out,) = hip.call("div_bf16", n, 2, md, In(xb), In(rhs), Out(n, "bf16"))
    with np.errstate(all="ignore"):
        want = np.divide(a, b)
    zero = np.broadcast_to(b == 0, want.shape)
    want = np.where(zero, np.where(a == 0, np.float32(0), np.float32(np.inf)), want).astype(np.float32)
    assert same_bits(out.reshape(R, C), f32_to_bf16(want).reshape(R, C))
    codes = np.arange(1 << 16, dtype=np.uint16)
    for op in ("exp", "gelu"):
        (small,) = hip.call(f"{op}_bf16", codes.size, 1, meta_unary([codes.size], [1]), In(codes), Out(codes.size, "bf16"))
        (out,) = hip.call(f"{op}_bf16", n, 2, mdu, In(xb), Out(n, "bf16"))
        assert same_bits(out.reshape(R, C), small[au]), op


@pytest.mark.parametrize("dt", ["f32", "bf16"])
def test_broadcast_gradient_chain_8192(hip, xy, dt):
    """The backward of a [8192,8192] op [1,8192] pair at full size: sum_to_shape -> [1,8192] against float64, and the
    transposed-back add_inplace (the accumulate of a transposed view's gradient into its base) bit for bit."""
    x, y = xy
    st = (lambda v: f32_to_bf16(v.ravel())) if dt == "bf16" else (lambda v: np.ascontiguousarray(v.ravel()))
    sx, sy = st(x), st(y)
    xv, yv = to_float(sx, dt).reshape(R, C), to_float(sy, dt).reshape(R, C)
    n = R * C
    (s,) = hip.call(f"sum_to_shape_{dt}", n, 2, meta_sum_to_shape([R, C], [C, 1], [1, C]), In(sx), Out(C, dt))
    x64 = xv.astype(np.float64)
    tol = 1e-5 if dt == "f32" else 1e-2
    assert np.max(np.abs(to_float(s, dt) - x64.sum(0)) / np.abs(x64).sum(0)) <= tol
    # base[C,R] += g[R,C]^T : lhs contiguous [C,R], rhs strides [1,R]... the rhs is g viewed transposed
    from helpers import InOut
    (acc,) = hip.call(f"add_inplace_{dt}", n, 2, meta_binary([C, R], [R, 1], [1, C]), InOut(sy.copy()), In(sx))
    want = yv.reshape(C, R) + xv.T
    want = f32_to_bf16(want.ravel()) if dt == "bf16" else want.ravel()
    assert same_bits(acc, want)


def test_conv2d_layer_step_config_size(mx_hip):
    """One full Conv2d(64->64, 3x3, stride 1, pad 1, bias) + MSE step on [32,64,56,56] through the host layer against the
    float64 restatement of the layer's data flow (host_programs.conv_numpy): output, loss and the three gradients."""
    from host_programs import conv_inputs, conv_numpy, conv_step
    x, w, b = conv_inputs(32, 64, 56, 56, 64, 3, seed=0x5EED0005)
    target = np.random.default_rng(0x5EED0015).standard_normal((32, 64, 56, 56)).astype(np.float32)
    got = conv_step(mx_hip, x, w, b, 1, 1, target)
    num = conv_numpy(x, w, b, 1, 1, target)
    for key, tol in (("out", 1e-5), ("loss", 1e-5), ("grad_b", 2e-5), ("grad_w", 1e-4), ("grad_x", 2e-5)):
        scale = np.abs(num[key]).max() + 1e-30
        assert np.abs(got[key] - num[key]).max() <= tol * scale, key
    # the reference's truncation (col2im is handed num_els = B*C*H*W): only the first 227 planes and 5/9 of plane 227 get a gradient
    gx = got["grad_x"].reshape(32 * 64, 56 * 56)
    assert np.abs(gx[:227]).max() > 0 and not gx[228:].any()


def test_conv2d_layer_step_config_size_every_way_gives_the_same_gradients(mx_hip):
    """The same full-size step with the switches of the host layer turned the reference's way: the column matrix stored
    (im2col) or gathered inside the products, grad_cols whole or only the rows col2im reads, backward() with and without
    its shortcuts.  Outputs and all gradients are the same bits; with sums dim by dim only the loss and the bias gradient
    (sums themselves) may differ, within the reduction tolerance."""
    from host_programs import conv_inputs, conv_step
    x, w, b = conv_inputs(32, 64, 56, 56, 64, 3, seed=0x5EED0006)
    target = np.random.default_rng(0x5EED0016).standard_normal((32, 64, 56, 56)).astype(np.float32)
    mx = mx_hip
    try:
        base = conv_step(mx, x, w, b, 1, 1, target)
        variants = {}
        mx.set_conv_gathered_products(2)
        variants["gathered"] = conv_step(mx, x, w, b, 1, 1, target)
        mx.set_conv_gathered_products(1)
        mx.set_conv_skip_unread_grad_cols(False)
        variants["whole grad_cols"] = conv_step(mx, x, w, b, 1, 1, target)
        mx.set_conv_skip_unread_grad_cols(True)
        mx.set_autograd_shortcuts(False)
        variants["no shortcuts"] = conv_step(mx, x, w, b, 1, 1, target)
        mx.set_autograd_shortcuts(True)
        mx.set_fused_nn_kernels(False)
        op_by_op = conv_step(mx, x, w, b, 1, 1, target)
        mx.set_fused_nn_kernels(True)
        mx.set_sum_all_in_one_pass(False)
        dim_by_dim = conv_step(mx, x, w, b, 1, 1, target)
    finally:
        mx.set_fused_nn_kernels(True)
        mx.set_conv_gathered_products(1)
        mx.set_conv_skip_unread_grad_cols(True)
        mx.set_autograd_shortcuts(True)
        mx.set_sum_all_in_one_pass(True)
    for name, got in variants.items():
        for key in ("out", "loss", "grad_b", "grad_w", "grad_x"):
            assert np.array_equal(got[key].view(np.uint32), base[key].view(np.uint32)), (name, key)
    # the loss, its backward pass and the forward product's store as the separate ops of the reference: the loss is summed in
    # another order, everything else is the same bits
    for key in ("out", "grad_b", "grad_w", "grad_x"):
        assert np.array_equal(op_by_op[key].view(np.uint32), base[key].view(np.uint32)), ("op by op", key)
    assert abs(float(op_by_op["loss"]) - float(base["loss"])) <= 1e-5 * abs(float(base["loss"]))
    for key in ("out", "grad_w", "grad_x"):
        assert np.array_equal(dim_by_dim[key].view(np.uint32), base[key].view(np.uint32)), ("sum_all dim by dim", key)
    assert abs(float(dim_by_dim["loss"]) - float(base["loss"])) <= 1e-5 * abs(float(base["loss"]))
    # (the bias gradient is a sum over W, H and the batch: 100352 terms each, in one pass or dim by dim)
    assert np.abs(dim_by_dim["grad_b"] - base["grad_b"]).max() <= 1e-5 * np.abs(base["grad_b"]).max()


def test_bf16_accumulation_gpu_is_closer_to_exact_than_the_reference(hip, oracle):
    """4096-term bf16 dot products and sums: the reference accumulates in bf16 (crates/maidenx_cpu/src/ops/matmul.rs:74-86,
    reduction.rs:58), the GPU in f32 with one rounding.  Both are measured against float64, normalised by the sum of
    |terms|; the GPU must be within the bf16 tolerance and no further from exact than the reference's own arithmetic, and
    the GPU-to-reference distance is bounded by the sum of the two."""
    r = np.random.default_rng(0x5EED0044)
    M = N = 64
    K = 4096
    a16 = f32_to_bf16(r.standard_normal((M, K), dtype=np.float32).ravel())
    b16 = f32_to_bf16((r.standard_normal((K, N), dtype=np.float32) * np.float32(0.02)).ravel())
    av, bv = to_float(a16, "bf16").astype(np.float64).reshape(M, K), to_float(b16, "bf16").astype(np.float64).reshape(K, N)
    md = meta_matmul([M, N], [M, K], [K, N], [K, 1], [N, 1])
    oracle.set_threads(1)
    (g,) = hip.call("matmul_bf16", M * N, md, In(a16), In(b16), Out(M * N, "bf16"))
    (o,) = oracle.call("matmul_bf16", M * N, md, In(a16), In(b16), Out(M * N, "bf16"))
    exact, scale = av @ bv, (np.abs(av) @ np.abs(bv)).max()
    eg = np.abs(to_float(g, "bf16").reshape(M, N) - exact).max() / scale
    eo = np.abs(to_float(o, "bf16").reshape(M, N) - exact).max() / scale
    ego = np.abs(to_float(g, "bf16").astype(np.float64) - to_float(o, "bf16")).max() / scale
    print(f"matmul bf16 K=4096: gpu-f64 {eg:.2e}  cpu-f64 {eo:.2e}  gpu-cpu {ego:.2e}")
    assert eg <= 1e-2 and eg <= eo and ego <= eg + eo
    mdr = meta_reduce([M, K], [K, 1], 1)
    (g,) = hip.call("sum_bf16", M * K, 2, 1, mdr, In(a16), Out(M, "bf16"))
    (o,) = oracle.call("sum_bf16", M * K, 2, 1, mdr, In(a16), Out(M, "bf16"))
    exact, scale = av.sum(1), np.abs(av).sum(1).max()
    eg = np.abs(to_float(g, "bf16") - exact).max() / scale
    eo = np.abs(to_float(o, "bf16") - exact).max() / scale
    ego = np.abs(to_float(g, "bf16").astype(np.float64) - to_float(o, "bf16")).max() / scale
    print(f"sum bf16 L=4096: gpu-f64 {eg:.2e}  cpu-f64 {eo:.2e}  gpu-cpu {ego:.2e}")
    assert eg <= 1e-2 and eg <= eo and ego <= eg + eo
