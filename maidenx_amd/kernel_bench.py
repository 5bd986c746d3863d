"""Per-kernel micro-benchmark of the HIP backend through its C ABI.

    python -m maidenx_amd.kernel_bench [filter] [--sets N] [--random-grad] [--json]

Every call is timed with HIP events on the backend's stream over `reps` back-to-back launches.  Buffers
rotate among `--sets` (default 4) distinct allocations, so that no launch finds its operands in the 256 MB
last-level cache left there by the previous one: the GB/s column is what HBM delivers.  (`bench.py` times
the same kernels inside their workloads, where some operands are cache-warm.)  bytes = algorithmic bytes:
every input element read once, every output element written once.
"""
import argparse
import ctypes as C
import json
import sys

import numpy as np

from . import lib as L

R = Cc = 8192
N = R * Cc


class Bench:
    def __init__(self, flt="", sets=4, random_grad=False, out=sys.stdout):
        self.lib = L.load()
        self.flt, self.sets, self.random_grad, self.out = flt, sets, random_grad, out
        self.bufs, self.set = {}, [0]
        self.rs = np.random.default_rng(0)
        self.rows = []

    # a pointer that rotates among `sets` distinct allocations
    class Rot:
        def __init__(self, bench, name, nbytes):
            self.bench = bench
            self.ptrs = [bench._buf(f"{name}#{i}", nbytes, name) for i in range(bench.sets)]

        @property
        def _as_parameter_(self):
            return C.c_void_p(self.ptrs[self.bench.set[0] % len(self.ptrs)])

    def buf(self, name, nbytes):
        return Bench.Rot(self, name, nbytes)

    def _buf(self, key, nbytes, kind):
        if key not in self.bufs:
            if kind in ("x", "y") or (self.random_grad and kind == "z"):
                a = self.rs.standard_normal(nbytes // 4, dtype=np.float32)
                # as pairs of 16-bit floats the same bytes are still finite, well-scaled values
                a = (a.view(np.uint32) & 0xFFFF0000 | (a.view(np.uint32) >> 16)).view(np.float32)
                self.bufs[key] = L.DeviceBuffer.from_numpy(a)
            else:
                self.bufs[key] = L.DeviceBuffer(nbytes)
                self.lib.hip_fill_f32(nbytes // 4, self.bufs[key].ptr, 1.0)
        return self.bufs[key].ptr

    def timeit(self, label, fn, nbytes, reps=20, flops=None):
        if self.flt and self.flt not in label:
            return
        lib = self.lib
        for i in range(3):
            self.set[0] = i
            fn()
        a, b = C.c_void_p(), C.c_void_p()
        lib.hip_event_create(C.byref(a))
        lib.hip_event_create(C.byref(b))
        lib.hip_event_record(a)
        for i in range(reps):
            self.set[0] = i
            fn()
        lib.hip_event_record(b)
        lib.hip_event_synchronize(b)
        ms = C.c_float()
        lib.hip_event_elapsed_ms(a, b, C.byref(ms))
        lib.hip_event_destroy(a)
        lib.hip_event_destroy(b)
        L.check()
        us = ms.value * 1e3 / reps
        row = {"kernel": label, "us": round(us, 1), "GB/s": round(nbytes / us / 1e3, 1), "hbm_frac": round(nbytes / us / 1e3 / 8000, 3)}
        if flops:
            row["TFLOP/s"] = round(flops / us / 1e6, 1)
        self.rows.append(row)
        extra = f" {row['TFLOP/s']:8.1f} TFLOP/s" if flops else ""
        print(f"{label:52s} {us:9.1f} us {row['GB/s']:8.1f} GB/s {100 * row['hbm_frac']:5.1f}%{extra}", file=self.out, flush=True)


def u64(*parts):
    out = []
    for p in parts:
        out.extend([int(p)] if np.isscalar(p) else [int(v) for v in p])
    return np.array(out, dtype=np.uint64)


def run(flt="", sets=4, random_grad=False, out=sys.stdout):
    """Runs every entry whose label contains `flt`; returns the rows."""
    bn = Bench(flt, sets, random_grad, out)
    lib, buf, timeit = bn.lib, bn.buf, bn.timeit
    cont, tr, row = [Cc, 1], [1, R], [0, 1]
    one = {"f32": 2.0, "bf16": 0x4000, "f16": 0x4000}

    # ---- elementwise and reductions on [8192,8192] / [64,512,1024] ---------------------------------------
    for dt, e in (("f32", 4), ("bf16", 2), ("f16", 2)):
        x, y, z = buf("x", N * 4), buf("y", N * 4), buf("z", N * 4)
        m = lambda ls, rs: u64([R, Cc], ls, rs, 0, 0)
        mu = lambda s: u64([R, Cc], s, 0)
        f = getattr(lib, f"hip_mul_{dt}")
        for name, md, nb in (("contig", m(cont, cont), 3 * N * e), ("bcast_row", m(cont, row), 2 * N * e),
                             ("transposed", m(tr, cont), 3 * N * e), ("both_tr", m(tr, tr), 3 * N * e)):
            timeit(f"mul_{dt}/{name}", lambda: f(N, 2, md.ctypes.data, x, y, z), nb)
        f = getattr(lib, f"hip_add_inplace_{dt}")
        md = m(cont, cont)
        timeit(f"add_inplace_{dt}/contig", lambda: f(N, 2, md.ctypes.data, x, y), 3 * N * e)
        md2 = m(cont, tr)
        timeit(f"add_inplace_{dt}/rhs_transposed", lambda: f(N, 2, md2.ctypes.data, x, y), 3 * N * e)
        for op in ("neg", "exp", "relu", "tanh", "gelu"):
            f = getattr(lib, f"hip_{op}_{dt}")
            for name, md in (("contig", mu(cont)), ("transposed", mu(tr))):
                timeit(f"{op}_{dt}/{name}", lambda: f(N, 2, md.ctypes.data, x, z), 2 * N * e)
        f = getattr(lib, f"hip_mul_scalar_{dt}")
        md = mu(cont)
        timeit(f"mul_scalar_{dt}/contig", lambda: f(N, 2, md.ctypes.data, x, one[dt], z), 2 * N * e)
        for op in ("sum", "max"):
            f = getattr(lib, f"hip_{op}_{dt}")
            for dim in (0, 1):
                md = u64([R, Cc], cont, [R, Cc][dim], cont[dim], 0)
                timeit(f"{op}_{dt}/[8192,8192] dim{dim}", lambda: f(N, 2, 1, md.ctypes.data, x, z), N * e)
            sh, st, n3 = [64, 512, 1024], [512 * 1024, 1024, 1], 64 * 512 * 1024
            for dim in (0, 1, 2):
                md = u64(sh, st, sh[dim], st[dim], 0)
                timeit(f"{op}_{dt}/[64,512,1024] dim{dim}", lambda: f(n3, 3, 1, md.ctypes.data, x, z), n3 * e)
        f = getattr(lib, f"hip_sum_to_shape_{dt}")
        md = u64([64, 512, 1024], [512 * 1024, 1024, 1], [1, 512, 1], 0)
        timeit(f"sum_to_shape_{dt}/[64,512,1024]->[1,512,1]", lambda: f(64 * 512 * 1024, 3, md.ctypes.data, x, z), 64 * 512 * 1024 * e)
        md = u64([R, Cc], cont, [1, Cc], 0)
        timeit(f"sum_to_shape_{dt}/->[1,8192]", lambda: f(N, 2, md.ctypes.data, x, z), N * e)
        md = u64([R, Cc], cont, [R, Cc], 0)
        timeit(f"sum_to_shape_{dt}/identity", lambda: f(N, 2, md.ctypes.data, x, z), 2 * N * e)
        f = getattr(lib, f"hip_softmax_{dt}")
        md = u64([R, Cc], cont, 0)
        timeit(f"softmax_{dt}/[8192,8192] dim1", lambda: f(N, 2, 1, md.ctypes.data, x, z), 2 * N * e)
        timeit(f"softmax_{dt}/[8192,8192] dim0", lambda: f(N, 2, 0, md.ctypes.data, x, z), 2 * N * e, reps=5)

    # ---- the binary family on the other dtypes: the 64 M-element buffers read as 1-, 4- and 8-byte elements ----------
    for dt, e in (("u8", 1), ("i32", 4), ("i64", 8), ("f64", 8)):
        x, y, z = buf("x", N * 4), buf("y", N * 4), buf("z", N * 4)
        rows = R * 4 // e                                   # the same 256 MB per operand
        n = rows * Cc
        for op, out_e in (("add", e), ("lt", 1)):
            f = getattr(lib, f"hip_{op}_{dt}")
            md = u64([rows, Cc], cont, cont, 0, 0)
            timeit(f"{op}_{dt}/contig", lambda: f(n, 2, md.ctypes.data, x, y, z), n * (2 * e + out_e))
        md = u64([rows, Cc], cont, row, 0, 0)
        f = getattr(lib, f"hip_mul_{dt}")
        timeit(f"mul_{dt}/bcast_row", lambda: f(n, 2, md.ctypes.data, x, y, z), n * 2 * e)

    # ---- reductions on the other dtypes: 256 MB read as [rows, 8192] of 4- and 8-byte elements ---------------------------
    for dt, e in (("i32", 4), ("i64", 8), ("f64", 8)):
        x, z = buf("x", N * 4), buf("z", N * 4)
        rows = R * 4 // e
        n = rows * Cc
        for op in ("sum", "max"):
            f = getattr(lib, f"hip_{op}_{dt}")
            for dim, red_stride in ((0, Cc), (1, 1)):
                md = u64([rows, Cc], cont, [rows, Cc][dim], red_stride, 0)
                timeit(f"{op}_{dt}/[{rows},{Cc}] dim {dim}", lambda: f(n, 2, 1, md.ctypes.data, x, z), n * e + (n // [rows, Cc][dim]) * e)

    # ---- what the memory system gives a plain stream -------------------------------------------------------
    zf = buf("z", N * 4)
    timeit("fill_f32/268MB (write only)", lambda: lib.hip_fill_f32(N, zf, 1.0), N * 4)
    src, dst = buf("x", N * 4), buf("z", N * 4)
    timeit("memcpy_d2d 268MB (read+write)", lambda: lib.hip_memcpy_d2d(dst, src, N * 4), 2 * N * 4)

    # ---- matmul forward, dA, dB --------------------------------------------------------------------------------
    for dt, e in (("bf16", 2), ("f16", 2), ("f32", 4)):
        for (b, m_, k, n) in ((1, 4096, 4096, 4096), (32, 512, 1024, 1024)):
            a, bb, c = buf("x", N * 4), buf("y", N * 4), buf("z", N * 4)
            ga, gb = buf("ga", N * 4), buf("gb", N * 4)
            md = u64(3, 3, 3, [b, m_, n], [b, m_, k], [b, k, n], [m_ * k, k, 1], [k * n, n, 1], 0, 0)
            fl = 2.0 * b * m_ * k * n
            nb = (b * m_ * k + b * k * n + b * m_ * n) * e
            f, g = getattr(lib, f"hip_matmul_{dt}"), getattr(lib, f"hip_matmul_backward_{dt}")
            timeit(f"matmul_{dt}/{b}x{m_}x{k}x{n} fwd", lambda: f(b * m_ * n, md.ctypes.data, a, bb, c), nb, reps=5, flops=fl)
            timeit(f"matmul_{dt}/{b}x{m_}x{k}x{n} dA", lambda: g(b * m_ * k, b * k * n, md.ctypes.data, c, a, bb, ga, None), nb, reps=5, flops=fl)
            timeit(f"matmul_{dt}/{b}x{m_}x{k}x{n} dB", lambda: g(b * m_ * k, b * k * n, md.ctypes.data, c, a, bb, None, gb), nb, reps=5, flops=fl)

    # ---- matmul on f64 / i32: LDS-tiled products without a matrix instruction ------------------------------------------
    for dt, e in (("f64", 8), ("i32", 4)):
        b, m_, k, n = 1, 2048, 2048, 2048
        a, bb, c = buf("x", N * 4), buf("y", N * 4), buf("z", N * 4)
        md = u64(3, 3, 3, [b, m_, n], [b, m_, k], [b, k, n], [m_ * k, k, 1], [k * n, n, 1], 0, 0)
        f = getattr(lib, f"hip_matmul_{dt}")
        timeit(f"matmul_{dt}/{b}x{m_}x{k}x{n} fwd", lambda: f(b * m_ * n, md.ctypes.data, a, bb, c), 3 * m_ * k * e, reps=3, flops=2.0 * m_ * k * n)

    # ---- fused Adam step: 4 tensors read, 3 written (the reference's fourteen ops move about 40) -------------------
    for dt, e in (("f32", 4), ("bf16", 2)):
        n = N if dt == "f32" else 2 * N
        pa, g, mm, vv = buf("x", N * 4), buf("y", N * 4), buf("z", N * 4), buf("ga", N * 4)
        c = (lambda v: C.c_float(v)) if dt == "f32" else (lambda v: C.c_uint16(int(np.array([v], np.float32).view(np.uint32)[0] >> 16)))
        sc = [c(v) for v in (0.9, 0.1, 0.999, 0.001, 0.19, 0.002, 1e-8, 2.4e-4)]
        f = getattr(lib, f"hip_adam_step_{dt}")
        timeit(f"adam_step_{dt}/{n} elements (one call for adam.rs:46-86)", lambda: f(n, pa, g, mm, vv, *sc), 7 * n * e)

    # ---- the pieces of Conv2d(64 -> 64, 3x3, s1, p1) on [32,64,56,56] and the pad kernels at that size -------------
    B, Ci, H, W = 32, 64, 56, 56
    md = u64(B, Ci, H, W, 3, 3, 56, 56, 1, 1, 1, 1)
    n_in, ncol, n_pad = B * Ci * H * W, B * Ci * 9 * 56 * 56, B * Ci * 58 * 58
    xin, col = buf("x", N * 4), buf("col", ncol * 4)
    timeit("im2col_f32/[32,64,56,56] 3x3", lambda: lib.hip_conv2d_im2col_f32(ncol, md.ctypes.data, xin, col), (n_in + ncol) * 4)
    timeit("col2im_f32/num_els = B*C*H*W (the layer's call)", lambda: lib.hip_conv2d_col2im_f32(n_in, md.ctypes.data, col, xin), 2 * n_in * 4)
    timeit("col2im_f32/whole column matrix", lambda: lib.hip_conv2d_col2im_f32(ncol, md.ctypes.data, col, xin), (n_in + ncol) * 4)
    mdp = u64([B, Ci, H, W], [Ci * H * W, H * W, W, 1], 0, [B, Ci, 58, 58], [0, 0, 0, 0, 1, 1, 1, 1])
    # calibration: a plain copy that moves as many bytes as a pad at this size (launch and ramp included)
    timeit("memcpy_d2d 26.6MB (as much as one pad)", lambda: lib.hip_memcpy_d2d(col, xin, (n_in + n_pad) * 2), (n_in + n_pad) * 4)
    timeit("pad_with_constant_f32/[32,64,56,56]+1", lambda: lib.hip_pad_with_constant_f32(n_in, n_pad, 4, mdp.ctypes.data, xin, col, 0.0), (n_in + n_pad) * 4)
    timeit("pad_with_constant_backward_f32/[32,64,56,56]+1", lambda: lib.hip_pad_with_constant_backward_f32(n_in, n_pad, 4, mdp.ctypes.data, col, xin), (n_in + n_pad) * 4)
    for mode in ("reflection", "replication"):
        f, g = getattr(lib, f"hip_pad_with_{mode}_f32"), getattr(lib, f"hip_pad_with_{mode}_backward_f32")
        timeit(f"pad_with_{mode}_f32/[32,64,56,56]+1", lambda: f(n_in, n_pad, 4, mdp.ctypes.data, xin, col), (n_in + n_pad) * 4)
        timeit(f"pad_with_{mode}_backward_f32/[32,64,56,56]+1", lambda: g(n_in, n_pad, 4, mdp.ctypes.data, col, xin), (n_in + n_pad) * 4)
    mdn = u64([n_in], [1], 0)
    timeit("same size, plain copy: neg_f32 6.4M contiguous", lambda: lib.hip_neg_f32(n_in, 1, mdn.ctypes.data, xin, col), 2 * n_in * 4)

    # ---- index ops: an embedding lookup and its gradient, a label pick ---------------------------------------------
    V, E, NI = 50000, 1024, 65536
    emb, outb = buf("x", N * 4), buf("z", N * 4)
    ids = L.DeviceBuffer.from_numpy(bn.rs.integers(0, V, NI).astype(np.int32))
    lab = L.DeviceBuffer.from_numpy(bn.rs.integers(0, 1000, 65536).astype(np.int64))
    lay_e, lay_o = u64([V, E], [E, 1], 0), u64([NI, E], [E, 1], 0)
    lay_l, lay_i = u64([65536, 1000], [1000, 1], 0), u64([65536, 1], [1, 1], 0)
    timeit("index_select_f32_i32/[50000,1024] x 65536 rows",
           lambda: lib.hip_index_select_f32_i32(2, 0, lay_e.ctypes.data, NI, 1, 0, C.c_void_p(ids.ptr), emb, outb), 2 * NI * E * 4)
    timeit("index_add_f32_i32/[50000,1024] += 65536 rows",
           lambda: lib.hip_index_add_f32_i32(2, 0, lay_e.ctypes.data, lay_o.ctypes.data, NI, 1, 0, C.c_void_p(ids.ptr), outb, emb), 3 * NI * E * 4)
    timeit("gather_f32_i64/[65536,1000] one per row",
           lambda: lib.hip_gather_f32_i64(2, 1, lay_l.ctypes.data, lay_i.ctypes.data, C.c_void_p(lab.ptr), emb, outb), 65536 * (4 + 8 + 4))
    L.synchronize()
    return bn.rows


def main():
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("filter", nargs="?", default="", help="run only the entries whose label contains this text")
    ap.add_argument("--sets", type=int, default=4, help="distinct allocations each buffer rotates among")
    ap.add_argument("--random-grad", action="store_true", help="random data in the output/gradient buffers too (matmul backward)")
    ap.add_argument("--json", action="store_true", help="print the rows as one JSON line at the end")
    a = ap.parse_args()
    rows = run(a.filter, a.sets, a.random_grad, sys.stderr if a.json else sys.stdout)
    if a.json:
        print(json.dumps(rows))


if __name__ == "__main__":
    main()
