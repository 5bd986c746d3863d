"""Benchmark of the maidenx_hip backend on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload all|elementwise|reduce|matmul|mlp|conv|copy|kernels]

The default (`all`) runs the five configurations one after the other in this process and prints ONE JSON line.  Its
top-level `value`, `roofline` and `cpu_baseline` are those of the elementwise configuration (configs[1]): forward +
backward of add, mul, div, exp, relu, gelu on [8192,8192] tensors, f32 and bf16, for contiguous operands, a [1,8192]
broadcast rhs and a transposed lhs view, with the gradients taken through sum_to_shape and accumulated in place.  One
"step" issues, through the C ABI, the chain of backend kernels the reference's tensor layer issues for all of these
(crates/maidenx_tensor/src/ops/{binary,unary}.rs backward closures).  `config.results` holds, per configuration
(mlp = configs[0], elementwise, reduce = configs[2], matmul = configs[3], conv = configs[4]), its own value, unit,
ms_per_step, roofline and cpu_baseline: train steps/s, HBM GB/s and matmul TFLOP/s all come from this one run.
Inputs are resident in HBM before the timed region starts.  Per-kernel roofline figures are taken with HIP events on
the backend's stream, on launches whose operands were not touched by the launch before (other buffers, or rotating
copies), so the 256 MB last-level cache does not serve them.
"""
import argparse
import ctypes as C
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
MFMA_PEAK_TFLOPS = {"bf16": 2500.0, "f32": 157.3}
ESZ = {"f32": 4, "bf16": 2, "bool": 1}


def u64(*parts):
    out = []
    for p in parts:
        out.extend([int(p)] if np.isscalar(p) else [int(v) for v in p])
    return np.array(out, dtype=np.uint64)


def f32_to_bf16(a):
    x = np.ascontiguousarray(a, dtype=np.float32).view(np.uint32).astype(np.uint64)
    return ((x + 0x7FFF + ((x >> 16) & 1)) >> 16).astype(np.uint16)


def const(v, dt):
    return float(v) if dt == "f32" else int(f32_to_bf16(np.array([v], np.float32))[0])


class Call:
    """One backend call with its C arguments ready, plus the bytes it must move at the least."""
    __slots__ = ("fn", "args", "bytes", "tag", "keep")

    def __init__(self, fn, args, nbytes, tag, keep):
        self.fn, self.args, self.bytes, self.tag, self.keep = fn, args, nbytes, tag, keep


class ChainBuilder:
    """Builds the elementwise fwd+bwd kernel chains for one dtype on a backend.

    alloc(count, dtag, init) -> (pointer, keepalive).  Buffers: x, y [R,C]; xT storage [C,R] for the
    transposed view; row [C]; temporaries; gradient accumulators."""

    def __init__(self, lib, prefix, alloc, dt, R, Cc, seed):
        self.lib, self.prefix, self.dt, self.R, self.C = lib, prefix, dt, R, Cc
        self.N = R * Cc
        rng = np.random.default_rng(seed)
        self.keep = []

        def new(count, dtag=dt, init=None):
            p, k = alloc(count, dtag, init)
            self.keep.append(k)
            return p
        normal = lambda n: rng.standard_normal(n, dtype=np.float32)
        self.x, self.y, self.xT = new(self.N, init=normal(self.N)), new(self.N, init=normal(self.N)), new(self.N, init=normal(self.N))
        self.row = new(Cc, init=normal(Cc))
        self.go = new(self.N, init=np.ones(self.N, np.float32))
        self.z = new(self.N)
        self.t = [new(self.N) for _ in range(8)]
        self.tf = [new(self.N, "f32") for _ in range(8)] if dt == "bf16" else []      # promoted intermediates (gelu backward)
        self.mask = new(self.N, "bool")
        self.gx, self.gy, self.gbase, self.gxv = (new(self.N, init=np.zeros(self.N, np.float32)) for _ in range(4))
        self.grow = new(Cc, init=np.zeros(Cc, np.float32))
        self.trow = new(Cc)
        cs = [Cc, 1]
        self.lay = {                                   # (strides, footprint in elements)
            "contig": (cs, self.N), "row": ([0, 1], Cc), "transposed": ([1, R], self.N),
        }
        self.calls = []

    # -- emitters ----------------------------------------------------------------------------------
    def _fn(self, name):
        return getattr(self.lib, self.prefix + name)

    def binary(self, op, a, la, b, lb, out, tag=None, out_dt=None, dt=None):
        dt = dt or self.dt
        e = ESZ[dt]
        md = u64([self.R, self.C], self.lay[la][0], self.lay[lb][0], 0, 0)
        # an operand given twice (x * x) is read from HBM once
        same = b == a and lb == la
        nb = (self.lay[la][1] + (0 if same else self.lay[lb][1])) * e + self.N * ESZ[out_dt or dt]
        # ... and is a launch class of its own: fewer bytes, a shorter launch than one with two distinct operands
        self.calls.append(Call(self._fn(f"{op}_{dt}"), (self.N, 2, md.ctypes.data, a, b, out), nb,
                               tag or (f"{op}_{dt}/{la}+same" if same else f"{op}_{dt}/{la}+{lb}"), md))

    def inplace(self, op, acc, b, lb, dims=None):
        dims = dims or [self.R, self.C]
        n = dims[0] * dims[1]
        strides = {"contig": [dims[1], 1], "transposed_back": [1, dims[0]]}[lb]
        md = u64(dims, [dims[1], 1], strides, 0, 0)
        self.calls.append(Call(self._fn(f"{op}_inplace_{self.dt}"), (n, 2, md.ctypes.data, acc, b), 3 * n * ESZ[self.dt],
                               f"{op}_inplace_{self.dt}/{lb}", md))

    def inplace_row(self, acc, b):
        md = u64([1, self.C], [self.C, 1], [self.C, 1], 0, 0)
        self.calls.append(Call(self._fn(f"add_inplace_{self.dt}"), (self.C, 2, md.ctypes.data, acc, b), 3 * self.C * ESZ[self.dt],
                               f"add_inplace_{self.dt}/row", md))

    def unary(self, op, a, la, out, c=None, out_dt=None, dt=None):
        dt = dt or self.dt
        md = u64([self.R, self.C], self.lay[la][0], 0)
        nb = self.lay[la][1] * ESZ[dt] + self.N * ESZ[out_dt or dt]
        args = (self.N, 2, md.ctypes.data, a, out) if c is None else (self.N, 2, md.ctypes.data, a, const(c, dt), out)
        self.calls.append(Call(self._fn(f"{op}_{dt}"), args, nb, f"{op}_{dt}/{la}", md))

    def cast(self, src, dst, a, out):
        """with_dtype of a whole buffer (crates/maidenx_tensor/src/wt.rs:65-84): a host loop in the reference, a device kernel here."""
        self.calls.append(Call(self._fn(f"cast_{src}_{dst}"), (self.N, a, out), self.N * (ESZ[src] + ESZ[dst]), f"cast_{src}_{dst}", None))

    def cast_bool(self, a, out):
        self.calls.append(Call(self._fn(f"cast_bool_{self.dt}"), (self.N, a, out), self.N * (1 + ESZ[self.dt]), f"cast_bool_{self.dt}", None))

    def sts(self, a, out, to_row):
        out_dims = [1, self.C] if to_row else [self.R, self.C]
        md = u64([self.R, self.C], [self.C, 1], out_dims, 0)
        nb = (self.N + (self.C if to_row else self.N)) * ESZ[self.dt]
        self.calls.append(Call(self._fn(f"sum_to_shape_{self.dt}"), (self.N, 2, md.ctypes.data, a, out), nb,
                               f"sum_to_shape_{self.dt}/{'to_row' if to_row else 'identity'}", md))

    # -- accumulate_grad of the lhs (and, for a transposed view, of the tensor it views) ---------------
    def acc_lhs(self, g, case):
        if case == "transposed":
            self.inplace("add", self.gxv, g, "contig")                                  # the view's own grad
            self.inplace("add", self.gbase, g, "transposed_back", dims=[self.C, self.R])  # transpose backward
        else:
            self.inplace("add", self.gx, g, "contig")

    def acc_rhs(self, g, case):
        if case == "bcast":
            self.inplace_row(self.grow, g)
        else:
            self.inplace("add", self.gy, g, "contig")

    def operands(self, case):
        x, lx = (self.xT, "transposed") if case == "transposed" else (self.x, "contig")
        y, ly = (self.row, "row") if case == "bcast" else (self.y, "contig")
        return x, lx, y, ly

    # -- the chains (crates/maidenx_tensor/src/ops/binary.rs:48-53,152-157,207-215; unary.rs:214-216,325-345,611-613)
    def add(self, case):
        x, lx, y, ly = self.operands(case)
        t = self.t
        self.binary("add", x, lx, y, ly, self.z)
        self.sts(self.go, t[0], False)
        gr = self.trow if case == "bcast" else t[1]
        self.sts(self.go, gr, case == "bcast")
        self.acc_lhs(t[0], case)
        self.acc_rhs(gr, case)

    def mul(self, case):
        x, lx, y, ly = self.operands(case)
        t = self.t
        self.binary("mul", x, lx, y, ly, self.z)
        self.binary("mul", self.go, "contig", y, ly, t[0])
        self.sts(t[0], t[1], False)
        self.binary("mul", self.go, "contig", x, lx, t[2])
        gr = self.trow if case == "bcast" else t[3]
        self.sts(t[2], gr, case == "bcast")
        self.acc_lhs(t[1], case)
        self.acc_rhs(gr, case)

    def div(self, case):
        x, lx, y, ly = self.operands(case)
        t = self.t
        self.binary("div", x, lx, y, ly, self.z)
        self.binary("div", self.go, "contig", y, ly, t[0])
        self.sts(t[0], t[1], False)
        self.binary("mul", self.go, "contig", x, lx, t[2])
        self.unary("square", y, ly, t[3])
        self.binary("div", t[2], "contig", t[3], "contig", t[4])
        self.unary("neg", t[4], "contig", t[5])
        gr = self.trow if case == "bcast" else t[6]
        self.sts(t[5], gr, case == "bcast")
        self.acc_lhs(t[1], case)
        self.acc_rhs(gr, case)

    def exp(self, case):
        x, lx, _, _ = self.operands(case)
        self.unary("exp", x, lx, self.z)
        self.binary("mul", self.go, "contig", self.z, "contig", self.t[0])
        self.acc_lhs(self.t[0], case)

    def relu(self, case):
        x, lx, _, _ = self.operands(case)
        self.unary("relu", x, lx, self.z)
        self.unary("gt_scalar", x, lx, self.mask, c=0.0, out_dt="bool")
        self.cast_bool(self.mask, self.t[0])
        self.binary("mul", self.go, "contig", self.t[0], "contig", self.t[1])
        self.acc_lhs(self.t[1], case)

    def gelu(self, case):
        if self.dt == "bf16":
            return self.gelu_bf16(case)
        x, lx, _, _ = self.operands(case)
        t = self.t
        c0, coeff = 0.7978845608028654, 0.044715
        self.unary("gelu", x, lx, self.z)
        self.binary("mul", x, lx, x, lx, t[0])                      # x_squared
        self.binary("mul", t[0], "contig", x, lx, t[1])             # x_cubed
        self.unary("mul_scalar", t[1], "contig", t[2], c=coeff)
        self.binary("add", x, lx, t[2], "contig", t[1])
        self.unary("mul_scalar", t[1], "contig", t[2], c=c0)        # tanh_arg
        self.unary("tanh", t[2], "contig", t[1])                    # tanh_val
        self.binary("mul", t[1], "contig", t[1], "contig", t[2])
        self.unary("mul_scalar", t[2], "contig", t[3], c=-1.0)
        self.unary("add_scalar", t[3], "contig", t[2], c=1.0)       # sech_squared
        self.unary("mul_scalar", t[0], "contig", t[3], c=3.0 * coeff)
        self.unary("add_scalar", t[3], "contig", t[4], c=1.0)
        self.unary("mul_scalar", t[4], "contig", t[3], c=c0)        # inner_derivative
        self.unary("add_scalar", t[1], "contig", t[4], c=1.0)
        self.unary("mul_scalar", t[4], "contig", t[5], c=0.5)       # term1
        self.binary("mul", x, lx, t[2], "contig", t[4])
        self.binary("mul", t[4], "contig", t[3], "contig", t[6])
        self.unary("mul_scalar", t[6], "contig", t[4], c=0.5)       # term2
        self.binary("add", t[5], "contig", t[4], "contig", t[6])
        self.binary("mul", self.go, "contig", t[6], "contig", t[7])
        self.acc_lhs(t[7], case)

    def gelu_bf16(self, case):
        """The same closure on bf16 tensors.  A scalar that is not integer-valued promotes its tensor to f32
        (ops/unary.rs:870-878), and a bf16 x f32 binary op promotes to f32 (utils/promotion.rs:16-33), so from the first
        `mul_scalar(0.044715)` on the chain runs in f32 and the gradient is cast back when it is accumulated
        (ops/binary.rs:660-662).  Every promotion is a with_dtype of a whole buffer."""
        x, lx, _, _ = self.operands(case)
        t, f = self.t, self.tf
        c0, coeff = 0.7978845608028654, 0.044715
        F = dict(dt="f32")
        self.unary("gelu", x, lx, self.z)
        self.binary("mul", x, lx, x, lx, t[0])                      # x_squared (bf16)
        self.binary("mul", t[0], "contig", x, lx, t[1])             # x_cubed (bf16)
        self.cast("bf16", "f32", t[1], f[0])
        self.unary("mul_scalar", f[0], "contig", f[1], c=coeff, **F)
        self.cast("bf16", "f32", x, f[0])                           # input promoted for the add (keeps its layout)
        self.binary("add", f[0], lx, f[1], "contig", f[2], **F)
        self.unary("mul_scalar", f[2], "contig", f[1], c=c0, **F)   # tanh_arg
        self.unary("tanh", f[1], "contig", f[2], **F)               # tanh_val
        self.binary("mul", f[2], "contig", f[2], "contig", f[1], **F)
        self.unary("mul_scalar", f[1], "contig", f[3], c=-1.0, **F)
        self.unary("add_scalar", f[3], "contig", f[1], c=1.0, **F)  # sech_squared
        self.cast("bf16", "f32", t[0], f[3])                        # x_squared promoted
        self.unary("mul_scalar", f[3], "contig", f[4], c=3.0 * coeff, **F)
        self.unary("add_scalar", f[4], "contig", f[3], c=1.0, **F)
        self.unary("mul_scalar", f[3], "contig", f[4], c=c0, **F)   # inner_derivative
        self.unary("add_scalar", f[2], "contig", f[3], c=1.0, **F)
        self.unary("mul_scalar", f[3], "contig", f[5], c=0.5, **F)  # term1
        self.cast("bf16", "f32", x, f[0])                           # input promoted again for input * sech_squared
        self.binary("mul", f[0], lx, f[1], "contig", f[3], **F)
        self.binary("mul", f[3], "contig", f[4], "contig", f[6], **F)
        self.unary("mul_scalar", f[6], "contig", f[3], c=0.5, **F)  # term2
        self.binary("add", f[5], "contig", f[3], "contig", f[6], **F)
        self.cast("bf16", "f32", self.go, f[0])                     # grad_out promoted
        self.binary("mul", f[0], "contig", f[6], "contig", f[7], **F)
        # accumulate_grad casts the f32 gradient to the parameter's dtype, once per add_
        self.cast("f32", "bf16", f[7], t[7])
        if case == "transposed":
            self.inplace("add", self.gxv, t[7], "contig")
            self.cast("f32", "bf16", f[7], t[6])
            self.inplace("add", self.gbase, t[6], "transposed_back", dims=[self.C, self.R])
        else:
            self.inplace("add", self.gx, t[7], "contig")

    def build(self):
        for case in ("contig", "bcast", "transposed"):
            for op in (self.add, self.mul, self.div):
                op(case)
        for case in ("contig", "transposed"):
            for op in (self.exp, self.relu, self.gelu):
                op(case)
        return self.calls


def hip_backend():
    import maidenx_amd.lib as L
    lib = L.load()
    if L.device_count() < 1:
        sys.exit("bench.py needs one MI355X: no HIP device is visible")
    assert lib.hip_set_device(0) == 0

    def alloc(count, dtag, init):
        if init is None:
            buf = L.DeviceBuffer(count * ESZ[dtag])
        else:
            arr = f32_to_bf16(init) if dtag == "bf16" else np.ascontiguousarray(init, dtype={"f32": np.float32, "bool": np.uint8}[dtag])
            buf = L.DeviceBuffer.from_numpy(arr)
        return buf.ptr, buf
    return L, lib, alloc


def bind(lib, prefix):
    import maidenx_amd._signatures as S
    sig = dict(S.signatures())
    if prefix == "hip_":
        sig.update(S.extension_signatures())
    for name, args in sig.items():
        fn = getattr(lib, prefix + name, None)
        if fn is not None:
            fn.argtypes, fn.restype = args, None


def profile_traffic(path, key):
    """HBM bytes per launch of one kernel as a rocprofv3 --pmc run recorded them (FETCH_SIZE and WRITE_SIZE scaled by a
    copy kernel of known size): counters cannot be read from inside the timed process, so the figure is read from the
    committed summary, with the date of that measurement.  The line looked for is
    `traffic_bytes_per_launch[<key>] = <bytes> (measured <date>)`; (None, None) when the file or the line is missing."""
    import re
    try:
        with open(os.path.join(ROOT, path)) as f:
            for line in f:
                m = re.match(r"\s*traffic_bytes_per_launch\[(.+?)\]\s*=\s*(\d+)\s*\(measured (\S+)\)", line)
                if m and m.group(1) == key:
                    return float(m.group(2)), m.group(3)
    except OSError:
        pass
    return None, None


def per_call_times(lib, chains, passes=2):
    """One event pair around every call of `chains`, `passes` times over, outside any timed region.
    Returns {tag: [ms, ...]}."""
    out = {}
    ms = C.c_float()
    for _ in range(passes):
        evs = []
        for c in chains:
            a, b = C.c_void_p(), C.c_void_p()
            lib.hip_event_create(C.byref(a)); lib.hip_event_create(C.byref(b))
            lib.hip_event_record(a)
            c.fn(*c.args)
            lib.hip_event_record(b)
            evs.append((c.tag, a, b))
        lib.hip_synchronize()
        for tag, a, b in evs:
            lib.hip_event_elapsed_ms(a, b, C.byref(ms))
            out.setdefault(tag, []).append(ms.value)
            lib.hip_event_destroy(a); lib.hip_event_destroy(b)
    return out


def best_and_worst(chains, times, peak_per_ms, min_work, unit):
    """Of the calls that do at least `min_work` (bytes or flops), the one nearest to and the one furthest from the peak."""
    rows = []
    for tag, ms in times.items():
        work = next(c.bytes for c in chains if c.tag == tag)
        if work < min_work:
            continue
        avg = float(np.mean(ms))
        rows.append({"kernel": tag, "avg_launch_us": round(avg * 1e3, 1), "achieved": round(work / avg / peak_per_ms[1], 1), "unit": unit,
                     "frac": round(work / avg / peak_per_ms[0], 4)})
    rows.sort(key=lambda r: r["frac"])
    return (rows[-1], rows[0]) if rows else (None, None)


def timed_run(L, lib, chains, args, probe_tag):
    """W untimed passes, then K timed passes of `chains`; every launch tagged `probe_tag` in the timed
    passes is bracketed by events on the backend's stream.  Returns (seconds, [ms per probed launch])."""
    n_probe = sum(1 for c in chains if c.tag == probe_tag) * args.steps
    ev = [(C.c_void_p(), C.c_void_p()) for _ in range(min(n_probe, 4096))]
    for a, b in ev:
        lib.hip_event_create(C.byref(a)); lib.hip_event_create(C.byref(b))
    used = 0
    for _ in range(args.warmup):
        for c in chains:
            c.fn(*c.args)
    L.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        for c in chains:
            if c.tag == probe_tag and used < len(ev):
                a, b = ev[used]
                lib.hip_event_record(a)
                c.fn(*c.args)
                lib.hip_event_record(b)
                used += 1
            else:
                c.fn(*c.args)
    L.synchronize()
    dt_s = time.perf_counter() - t0
    L.check()
    ms = C.c_float()
    durs = []
    for a, b in ev[:used]:
        lib.hip_event_elapsed_ms(a, b, C.byref(ms))
        durs.append(ms.value)
        lib.hip_event_destroy(a); lib.hip_event_destroy(b)
    return dt_s, durs


def base_result(args, value, unit, dt_s, dtype, workload, extra_cfg):
    cfg = {"workload": workload}
    cfg.update(extra_cfg)
    return {"metric": "train steps/s; HBM GB/s elemwise/reduce; matmul TFLOP/s on 1 MI355X",
            "value": value, "unit": unit, "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
            "ms_per_step": round(dt_s / args.steps * 1e3, 3), "higher_is_better": True, "scaling": "weak",
            "vs_baseline": None, "dtype": dtype, "data": "synthetic", "config": cfg}


def hbm_roofline(kernel, nbytes, durs):
    avg_ms = float(np.mean(durs))
    achieved = nbytes / (avg_ms * 1e-3) / 1e9
    return {"bound": "hbm", "kernel": kernel, "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
            "frac": round(achieved / HBM_PEAK_GBS, 4), "avg_launch_us": round(avg_ms * 1e3, 2), "launches_timed": len(durs),
            "traffic": None}


def run_elementwise(args):
    L, lib, alloc = hip_backend()
    R = Cc = 8192
    chains, builders = [], []          # the builders own the device buffers: keep them alive
    for i, dt in enumerate(("f32", "bf16")):
        builders.append(ChainBuilder(lib, "hip_", alloc, dt, R, Cc, seed=0x5EED0002 + i))
        chains += builders[-1].build()
    step_bytes = sum(c.bytes for c in chains)
    probe_tag = "mul_f32/contig+contig"           # the most frequent kernel of the chain
    dt_s, durs = timed_run(L, lib, chains, args, probe_tag)
    probe_bytes = next(c.bytes for c in chains if c.tag == probe_tag)
    value = step_bytes * args.steps / dt_s / 1e9
    result = base_result(args, round(value, 1), "GB/s", dt_s, "f32+bf16",
                         "configs[1]: elementwise fwd+bwd (add,mul,div,exp,relu,gelu) on [8192,8192], f32+bf16, "
                         "contiguous / rhs [1,8192] broadcast / transposed lhs",
                         {"kernel_launches_per_step": len(chains), "algorithmic_GB_per_step": round(step_bytes / 1e9, 3)})
    result["roofline"] = hbm_roofline("ew_nd_kernel<OpMul<float>,4> (hip_mul_f32, contiguous [8192,8192]): the most frequent kernel of the chain",
                                      probe_bytes, durs)
    result["roofline"]["algorithmic_bytes"] = probe_bytes
    src = "profiles/elementwise_8192x8192_hbm_traffic.txt"
    result["roofline"]["traffic"], when = profile_traffic(src, "mul_f32/contig+contig")
    result["roofline"]["traffic_source"] = f"{src} (rocprofv3 --pmc, measured {when})" if when else None
    # every kernel of the chain on its own (launches that move at least 64 MB), and the chain as a whole
    best, worst = best_and_worst(chains, per_call_times(lib, chains), (HBM_PEAK_GBS * 1e6, 1e6), 64e6, "GB/s")
    result["roofline"]["best_of_chain"], result["roofline"]["worst_of_chain"] = best, worst
    result["roofline"]["whole_chain_frac"] = round(value / HBM_PEAK_GBS, 4)
    L.synchronize()
    del chains, builders
    result["cpu_baseline"] = None if args.no_cpu_baseline else cpu_baseline_elementwise(args)
    return result


def run_copy(args):
    """Counter calibration: nothing but contiguous copies of a [8192,8192] f32 tensor (268.4 MB read +
    268.4 MB written per launch), so that HBM byte counters can be scaled by a kernel of known traffic."""
    L, lib, alloc = hip_backend()
    N = 8192 * 8192
    src, dst = L.DeviceBuffer(N * 4), L.DeviceBuffer(N * 4)
    lib.hip_fill_f32(N, src.ptr, 1.0)
    md = u64([8192, 8192], [8192, 1], 0)
    chains = [Call(lib.hip_copy_strided_f32, (N, 2, md.ctypes.data, src.ptr, dst.ptr), 2 * N * 4, "copy_f32", md) for _ in range(8)]
    dt_s, durs = timed_run(L, lib, chains, args, "copy_f32")
    value = sum(c.bytes for c in chains) * args.steps / dt_s / 1e9
    result = base_result(args, round(value, 1), "GB/s", dt_s, "f32", "calibration: 8 contiguous copies of [8192,8192] f32 per step", {})
    result["roofline"] = hbm_roofline("ew_nd_kernel<OpCopy> (hip_copy_strided_f32, contiguous [8192,8192])", 2 * N * 4, durs)
    result["cpu_baseline"] = None
    return result


def reduce_calls(lib, prefix, ptr_in, ptr_out, ptr_tmp, shape, dt="f32"):
    """configs[2] on one input: sum/mean/max along every single axis and over all axes (the tensor layer
    chains single-axis calls from the last axis to the first, crates/maidenx_tensor/src/ops/reduction.rs:9-21).
    `ptr_in` may be a list of identical copies of the input: successive calls then read successive copies, so that no
    call finds its input in the last-level cache."""
    e = ESZ[dt]
    calls = []
    n = int(np.prod(shape))
    copies, turn = (list(ptr_in) if isinstance(ptr_in, (list, tuple)) else [ptr_in]), [0]

    def next_input():
        turn[0] += 1
        return copies[turn[0] % len(copies)]

    def one(op, dims, axis, src, dst):
        strides = [int(np.prod(dims[i + 1:])) for i in range(len(dims))]
        md = u64(dims, strides, dims[axis], strides[axis], 0)
        cnt = int(np.prod(dims))
        calls.append(Call(getattr(lib, f"{prefix}{op}_{dt}"), (cnt, len(dims), 1, md.ctypes.data, src, dst),
                          (cnt + cnt // dims[axis]) * e, f"{op}_{dt}/{'x'.join(map(str, dims))}/dim{axis}", md))
    for op in ("sum", "mean", "max"):
        for axis in range(len(shape)):
            one(op, list(shape), axis, next_input(), ptr_out)
        dims, src, k = list(shape), next_input(), 0    # all axes: last to first, ping-pong temporaries
        while dims:
            dst = (ptr_out, ptr_tmp)[k % 2]
            one(op, dims, len(dims) - 1, src, dst)
            dims, src, k = dims[:-1], dst, k + 1
    return calls


def run_reduce(args):
    L, lib, alloc = hip_backend()
    rng = np.random.default_rng(0x5EED0003)
    chains, keep = [], []
    for shape in ((8192, 8192), (64, 512, 1024)):
        n = int(np.prod(shape))
        host = rng.uniform(-1, 1, n).astype(np.float32)
        xs = [L.DeviceBuffer.from_numpy(host) for _ in range(4)]       # four copies in turn: 1 GB / 0.5 GB against a 256 MB cache
        out, tmp = L.DeviceBuffer(n * 4), L.DeviceBuffer(n * 4)
        keep += xs + [out, tmp]
        chains += reduce_calls(lib, "hip_", [x.ptr for x in xs], out.ptr, tmp.ptr, shape)
        if len(shape) == 3:
            md = u64(shape, [shape[1] * shape[2], shape[2], 1], [1, shape[1], 1], 0)
            chains.append(Call(lib.hip_sum_to_shape_f32, (n, 3, md.ctypes.data, xs[0].ptr, out.ptr), (n + shape[1]) * 4,
                               "sum_to_shape_f32/64x512x1024->1x512x1", md))
    step_bytes = sum(c.bytes for c in chains)
    probe_tag = "sum_f32/8192x8192/dim0"
    dt_s, durs = timed_run(L, lib, chains, args, probe_tag)
    value = step_bytes * args.steps / dt_s / 1e9
    result = base_result(args, round(value, 1), "GB/s", dt_s, "f32",
                         "configs[2]: sum/mean/max along dim 0, dim 1, all dims of [8192,8192] and [64,512,1024] f32, "
                         "plus sum_to_shape [64,512,1024]->[1,512,1]",
                         {"kernel_calls_per_step": len(chains), "algorithmic_GB_per_step": round(step_bytes / 1e9, 3)})
    probe_bytes = next(c.bytes for c in chains if c.tag == probe_tag)
    result["roofline"] = hbm_roofline("col_reduce_split_kernel<float,RSum> + fold (hip_sum_f32, [8192,8192] along dim 0)", probe_bytes, durs)
    result["roofline"]["algorithmic_bytes"] = probe_bytes
    src = "profiles/reduce_f32_kernel_trace.txt"
    result["roofline"]["traffic"], when = profile_traffic(src, "sum_f32/8192x8192/dim0")
    result["roofline"]["traffic_source"] = f"{src} (rocprofv3 --pmc, measured {when})" if when else None
    best, worst = best_and_worst(chains, per_call_times(lib, chains), (HBM_PEAK_GBS * 1e6, 1e6), 64e6, "GB/s")
    result["roofline"]["best_of_chain"], result["roofline"]["worst_of_chain"] = best, worst
    result["roofline"]["whole_chain_frac"] = round(value / HBM_PEAK_GBS, 4)
    result["cpu_baseline"] = None if args.no_cpu_baseline else cpu_baseline_reduce(args)
    return result


def cpu_baseline_reduce(args):
    """configs[2] on the CPU oracle, threaded, on a bounded sample: [512,8192] and [4,512,1024]."""
    from tests.helpers import ensure_oracle_built
    lib = C.CDLL(ensure_oracle_built())
    bind(lib, "oracle_")
    lib.oracle_set_num_threads.restype = C.c_int
    cores = lib.oracle_set_num_threads(0)
    rng = np.random.default_rng(0x5EED0003)
    chains, keep = [], []
    for shape in ((512, 8192), (4, 512, 1024)):
        n = int(np.prod(shape))
        x = rng.uniform(-1, 1, n).astype(np.float32)
        out, tmp = np.zeros(n, np.float32), np.zeros(n, np.float32)
        keep += [x, out, tmp]
        chains += reduce_calls(lib, "oracle_", x.ctypes.data, out.ctypes.data, tmp.ctypes.data, shape)
    nbytes = sum(c.bytes for c in chains)
    t0, reps = time.perf_counter(), 0
    while True:
        for c in chains:
            c.fn(*c.args)
        reps += 1
        if time.perf_counter() - t0 > 10.0 or reps >= 200:
            break
    el = time.perf_counter() - t0
    return {"value": round(nbytes * reps / el / 1e9, 2), "unit": "GB/s", "cores": cores, "kind": "port",
            "sample": f"same calls on [512,8192] and [4,512,1024] (1/16 of the rows / batches), {reps} passes, {el:.1f} s"}


def matmul_meta(batch, M, K, N):
    if batch:
        return u64(3, 3, 3, [batch, M, N], [batch, M, K], [batch, K, N], [M * K, K, 1], [K * N, N, 1], 0, 0)
    return u64(2, 2, 2, [M, N], [M, K], [K, N], [K, 1], [N, 1], 0, 0)


def matmul_calls(lib, prefix, new, dt, shapes, rng):
    """configs[3]: C = A.B, then matmul_backward giving dA = dC.B^T and dB = A^T.dC in one call."""
    calls, keep = [], []
    for batch, M, K, N in shapes:
        b = max(batch, 1)
        A = new(rng.standard_normal(b * M * K, dtype=np.float32), dt)
        B = new(rng.standard_normal(b * K * N, dtype=np.float32) * np.float32(0.02), dt)
        dC = new(rng.standard_normal(b * M * N, dtype=np.float32), dt)
        Cc, dA, dB = new(np.zeros(b * M * N, np.float32), dt), new(np.zeros(b * M * K, np.float32), dt), new(np.zeros(b * K * N, np.float32), dt)
        keep += [A, B, dC, Cc, dA, dB]
        md = matmul_meta(batch, M, K, N)
        flop = 2.0 * b * M * N * K
        name = f"{dt}/{'%dx' % batch if batch else ''}{M}x{K}x{N}"
        calls.append(Call(getattr(lib, f"{prefix}matmul_{dt}"), (b * M * N, md.ctypes.data, A[0], B[0], Cc[0]), flop, f"matmul_{name}", md))
        calls.append(Call(getattr(lib, f"{prefix}matmul_backward_{dt}"), (b * M * K, b * K * N, md.ctypes.data, dC[0], A[0], B[0], dA[0], dB[0]),
                          2 * flop, f"matmul_backward_{name}", md))
    return calls, keep


def run_matmul(args):
    L, lib, alloc = hip_backend()
    rng = np.random.default_rng(0x5EED0004)

    def new(arr, dt):
        buf = L.DeviceBuffer.from_numpy(f32_to_bf16(arr) if dt == "bf16" else arr)
        return buf.ptr, buf
    shapes = ((0, 4096, 4096, 4096), (32, 512, 1024, 1024))
    chains, keep = [], []
    for dt in ("bf16", "f32"):
        c, k = matmul_calls(lib, "hip_", new, dt, shapes, rng)
        chains += c; keep += k
    # the headline figure is the bf16 4096^3 forward + backward; f32 and the batched shape are reported beside it
    # A pass of the headline chain is 0.37 ms: the K timed passes are over before the card has left its idle clocks
    # unless the untimed part is long enough to raise them, so the warm-up is at least 200 passes (75 ms) here.
    args = argparse.Namespace(**{**vars(args), "warmup": max(args.warmup, 200)})
    def rate(tags):
        sel = [c for c in chains if c.tag in tags]
        a = argparse.Namespace(steps=args.steps, warmup=args.warmup)
        dt_s, _ = timed_run(L, lib, sel, a, None)
        return sum(c.bytes for c in sel) * args.steps / dt_s / 1e12, dt_s
    head = ("matmul_bf16/4096x4096x4096", "matmul_backward_bf16/4096x4096x4096")
    sel = [c for c in chains if c.tag in head]
    dt_s, durs = timed_run(L, lib, sel, args, head[0])
    value = sum(c.bytes for c in sel) * args.steps / dt_s / 1e12
    others = {}
    for dt in ("bf16", "f32"):
        for shp in ("4096x4096x4096", "32x512x1024x1024"):
            tags = (f"matmul_{dt}/{shp}", f"matmul_backward_{dt}/{shp}")
            others[f"{dt} {shp} fwd+bwd TFLOP/s"] = round(rate(tags)[0], 1)
    result = base_result(args, round(value, 1), "TFLOP/s", dt_s, "bf16",
                         "configs[3]: matmul forward + backward (dA = dC.B^T, dB = A^T.dC), [4096,4096]x[4096,4096] bf16; "
                         "f32 and the batched [32,512,1024]x[32,1024,1024] shape reported in `all`", {"all": others})
    fwd_flop = 2.0 * 4096 ** 3
    avg_ms = float(np.mean(durs))
    ach = fwd_flop / (avg_ms * 1e-3) / 1e12
    result["roofline"] = {"bound": "mfma", "kernel": "gemm_mfma_kernel<bf16, 256x256x64> (hip_matmul_bf16 4096^3 forward)",
                          "achieved": round(ach, 1), "peak": MFMA_PEAK_TFLOPS["bf16"], "unit": "TFLOP/s",
                          "frac": round(ach / MFMA_PEAK_TFLOPS["bf16"], 4), "avg_launch_us": round(avg_ms * 1e3, 2),
                          "launches_timed": len(durs), "algorithmic_flops": fwd_flop}
    # FETCH_SIZE + WRITE_SIZE of the forward kernel, scaled by the copy kernel (the algorithmic bytes are 100.7 MB; re-reads
    # of operand tiles are served by L2 and the last-level cache)
    src = "profiles/matmul_bf16_f32_kernel_trace_counters.txt"
    result["roofline"]["traffic"], when = profile_traffic(src, "matmul_bf16/4096x4096x4096")
    result["roofline"]["traffic_source"] = f"{src} (rocprofv3 --pmc, measured {when})" if when else None
    best, worst = best_and_worst(chains, per_call_times(lib, [c for c in chains if "bf16" in c.tag], passes=4),
                                 (MFMA_PEAK_TFLOPS["bf16"] * 1e9, 1e9), 1e9, "TFLOP/s")
    result["roofline"]["best_of_chain"], result["roofline"]["worst_of_chain"] = best, worst
    result["roofline"]["whole_chain_frac"] = round(value / MFMA_PEAK_TFLOPS["bf16"], 4)
    L.synchronize()
    if args.no_cpu_baseline:
        result["cpu_baseline"] = None
    else:
        result["cpu_baseline"] = cpu_baseline_matmul(args)
        result["cpu_baseline"]["bf16_distance"] = bf16_distance(L, lib)
    return result


def bf16_distance(L, lib):
    """Where the GPU's bf16 products and sums stand between the reference's arithmetic and the exact value: the
    reference accumulates in bf16 (crates/maidenx_cpu/src/ops/matmul.rs:74-86, reduction.rs:58), the GPU in f32 with one
    rounding at the end.  For a [64,4096]x[4096,64] product and 64 sums of 4096 terms on the same N(0,1) / N(0,0.02)
    inputs: the largest |error| against an f64 evaluation, over the largest sum of |terms|, for the GPU and for the CPU
    restatement, and the same measure between the two."""
    from tests.helpers import ensure_oracle_built
    orc = C.CDLL(ensure_oracle_built())
    bind(orc, "oracle_")
    orc.oracle_set_num_threads.restype = C.c_int
    orc.oracle_set_num_threads(1)
    rng = np.random.default_rng(0x5EED0044)
    M = N = 64
    K = 4096
    bf = lambda a: (f32_to_bf16(a).astype(np.uint32) << 16).view(np.float32)
    A = rng.standard_normal((M, K), dtype=np.float32)
    B = rng.standard_normal((K, N), dtype=np.float32) * np.float32(0.02)
    a16, b16 = f32_to_bf16(A).reshape(M, K), f32_to_bf16(B).reshape(K, N)
    Af, Bf = bf(A).reshape(M, K).astype(np.float64), bf(B).reshape(K, N).astype(np.float64)
    exact, scale = Af @ Bf, float((np.abs(Af) @ np.abs(Bf)).max())
    md = matmul_meta(0, M, K, N)
    out_o = np.zeros(M * N, np.uint16)
    orc.oracle_matmul_bf16(M * N, md.ctypes.data, a16.ctypes.data, b16.ctypes.data, out_o.ctypes.data)
    da, db, dc = L.DeviceBuffer.from_numpy(a16), L.DeviceBuffer.from_numpy(b16), L.DeviceBuffer(M * N * 2)
    lib.hip_matmul_bf16(M * N, md.ctypes.data, da.ptr, db.ptr, dc.ptr)
    out_g = dc.to_numpy(np.uint16)
    val = lambda u: (u.astype(np.uint32) << 16).view(np.float32).astype(np.float64).reshape(M, N)
    res = {"matmul [64,4096]x[4096,64]": {"gpu_vs_f64": float(np.abs(val(out_g) - exact).max() / scale),
                                          "cpu_vs_f64": float(np.abs(val(out_o) - exact).max() / scale),
                                          "gpu_vs_cpu": float(np.abs(val(out_g) - val(out_o)).max() / scale)}}
    # sums of 4096 terms along the contiguous axis
    mdr = u64([M, K], [K, 1], K, 1, 0)
    so = np.zeros(M, np.uint16)
    orc.oracle_sum_bf16(M * K, 2, 1, mdr.ctypes.data, a16.ctypes.data, so.ctypes.data)
    ds = L.DeviceBuffer(M * 2)
    lib.hip_sum_bf16(M * K, 2, 1, mdr.ctypes.data, da.ptr, ds.ptr)
    sg = ds.to_numpy(np.uint16)
    v1 = lambda u: (u.astype(np.uint32) << 16).view(np.float32).astype(np.float64)
    ex, sc = Af.sum(axis=1), float(np.abs(Af).sum(axis=1).max())
    res["sum of 4096 terms x 64 rows"] = {"gpu_vs_f64": float(np.abs(v1(sg) - ex).max() / sc), "cpu_vs_f64": float(np.abs(v1(so) - ex).max() / sc),
                                          "gpu_vs_cpu": float(np.abs(v1(sg) - v1(so)).max() / sc)}
    return res


def cpu_baseline_matmul(args):
    """The CPU oracle's matmul forward + backward, threaded, bf16, on a bounded sample: 512^3 (1/512 of the
    flops of 4096^3; the triple loop has no blocking, so its rate per flop does not improve with size)."""
    from tests.helpers import ensure_oracle_built
    lib = C.CDLL(ensure_oracle_built())
    bind(lib, "oracle_")
    lib.oracle_set_num_threads.restype = C.c_int
    cores = lib.oracle_set_num_threads(0)
    rng = np.random.default_rng(0x5EED0004)

    def new(arr, dt):
        a = f32_to_bf16(arr) if dt == "bf16" else np.ascontiguousarray(arr)
        return a.ctypes.data, a
    chains, keep = matmul_calls(lib, "oracle_", new, "bf16", ((0, 512, 512, 512),), rng)
    flop = sum(c.bytes for c in chains)
    t0, reps = time.perf_counter(), 0
    while True:
        for c in chains:
            c.fn(*c.args)
        reps += 1
        if time.perf_counter() - t0 > 10.0 or reps >= 50:
            break
    el = time.perf_counter() - t0
    return {"value": round(flop * reps / el / 1e12, 5), "unit": "TFLOP/s", "cores": cores, "kind": "port",
            "sample": f"bf16 [512,512]x[512,512] forward + backward, {reps} passes, {el:.1f} s"}


def cpu_baseline_elementwise(args):
    """The same chain on the CPU oracle (a restatement of maidenx_cpu, threaded like its rayon loops),
    on a bounded sample: [256,8192] instead of [8192,8192] (1/32 of the rows)."""
    from tests.helpers import ensure_oracle_built
    lib = C.CDLL(ensure_oracle_built())
    bind(lib, "oracle_")
    lib.oracle_set_num_threads.restype = C.c_int
    cores = lib.oracle_set_num_threads(0)
    R, Cc = 256, 8192

    def alloc(count, dtag, init):
        if init is None:
            arr = np.zeros(count, dtype={"f32": np.float32, "bf16": np.uint16, "bool": np.uint8}[dtag])
        else:
            arr = f32_to_bf16(init) if dtag == "bf16" else np.ascontiguousarray(init, dtype={"f32": np.float32, "bool": np.uint8}[dtag])
        return arr.ctypes.data, arr
    chains, builders = [], []          # the builders own the host arrays: keep them alive
    for i, dt in enumerate(("f32", "bf16")):
        b = ChainBuilder(lib, "oracle_", alloc, dt, R, Cc, seed=0x5EED0002 + i)
        builders.append(b)
        # the oracle has no device-side cast: the reference converts bool -> float on the host
        b.cast_bool = lambda a, out, b=b: b.calls.append(Call(lambda *x: None, (), 0, "host_cast", None))
        b.cast = lambda src, dst, a, out, b=b: b.calls.append(Call(lambda *x: None, (), 0, "host_cast", None))
        chains += b.build()
    nbytes = sum(c.bytes for c in chains)
    t0 = time.perf_counter()
    reps = 0
    while True:
        for c in chains:
            c.fn(*c.args)
        reps += 1
        if time.perf_counter() - t0 > 10.0 or reps >= 20:
            break
    el = time.perf_counter() - t0
    return {"value": round(nbytes * reps / el / 1e9, 2), "unit": "GB/s", "cores": cores, "kind": "port",
            "sample": f"same kernel chain on [{R},{Cc}] tensors (1/32 of the rows; the host-side dtype casts of the reference "
                      f"are left out, in the CPU's favour), {reps} passes, {el:.1f} s"}


def _mlp_setup(mx):
    i = np.arange(10000)
    x = np.stack([(i % 100) / 100.0, (i % 100 + 1) / 100.0, (i % 100 + 2) / 100.0], 1).astype(np.float32)
    y = ((i % 100) * 10 / 1000.0).astype(np.float32).reshape(-1, 1)
    lin = mx.Linear(in_features=3, out_features=1, with_bias=True, seed=0x5EED0000)
    return lin, mx.tensor(x).with_grad(), mx.tensor(y)


def empty_graph_floor(nodes_list=(3, 6, 13), replays=300):
    """Replay time of a captured sequence of N launches that compute nothing (a one-element fill each, fusion and
    programs switched off so that every launch stays a kernel node): what N dependent kernel nodes cost on this card
    before any work is done.  Microseconds per replay, by N."""
    import maidenx_amd.lib as L
    lib = L.load()
    buf = L.DeviceBuffer(256)
    was_f, was_p = lib.hip_graph_set_fusion(0), lib.hip_graph_set_programs(0)
    out = {}
    try:
        for n in nodes_list:
            assert lib.hip_graph_begin_capture() == 0
            for _ in range(n):
                lib.hip_fill_f32(1, buf.ptr, C.c_float(1.0))
            h = C.c_void_p()
            assert lib.hip_graph_end_capture(C.byref(h)) == 0
            for _ in range(20):
                lib.hip_graph_launch(h)
            L.synchronize()
            t0 = time.perf_counter()
            for _ in range(replays):
                lib.hip_graph_launch(h)
            L.synchronize()
            out[str(n)] = round((time.perf_counter() - t0) / replays * 1e6, 2)
            lib.hip_graph_destroy(h)
    finally:
        lib.hip_graph_set_fusion(was_f)
        lib.hip_graph_set_programs(was_p)
    return out


def run_mlp(args):
    """configs[0]: the loop of examples/device/cpu.rs (Linear(3->1) + MSELoss + SGD(0.01), 10000x3 input, full batch)
    through the host layer; a step is one epoch (forward, loss, backward, SGD step, zero_grad)."""
    hip_backend()
    from maidenx_amd.tensor import host
    mx = host()
    lin, x, y = _mlp_setup(mx)
    steps = max(args.steps, 1000)          # the example's own 1000 epochs: the eager epochs and the capture inside the call are part of the job
    # (40 untimed epochs: enough for the loop to record once, so that what a process sets up the first time it records -
    # the runtime's graph machinery and the chain kernel's first launch, 3.6 ms - is warm-up like every kernel's first launch)
    mx.train(lin, x, y, 0.01, max(args.warmup, 40))
    mx.synchronize()
    mx.reset_backend_calls()
    t0 = time.perf_counter()
    mx.train(lin, x, y, 0.01, steps)
    mx.synchronize()
    dt_s = time.perf_counter() - t0
    calls = mx.backend_calls() / steps
    a = argparse.Namespace(steps=steps, warmup=max(args.warmup, 40))
    result = base_result(a, round(steps / dt_s, 1), "steps/s", dt_s, "f32",
                         "configs[0]: README Linear(3->1, bias) + MSE + SGD(lr=0.01), f32, full batch 10000x3, 1000 epochs as in examples/device/cpu.rs",
                         {"backend_kernels_per_step": calls, "us_per_step": round(dt_s / steps * 1e6, 1)})
    result["roofline"] = None
    result["note"] = "launch-latency bound (about 200 KB touched per step): no roofline fraction applies"
    # the same loop on 1000 rows, where the recorded step is a resident step program (one work-group, tensors in LDS) by
    # default, against the same step as fused chains
    result["config"]["rows_1000_us_per_step"] = _small_mlp(mx, 1000)
    # (rocprofv3 has crashed inside hipGraphLaunch on this measurement's 900 replays when it follows the training graphs:
    # the profiles' command skips it)
    result["config"]["empty_graph_replay_us_by_nodes"] = None if args.no_graph_floor else empty_graph_floor()
    result["cpu_baseline"] = None if args.no_cpu_baseline else cpu_baseline_mlp(args)
    return result


def _small_mlp(mx, rows, epochs=2000):
    L, lib, _ = hip_backend()
    rng = np.random.default_rng(0x5EED0007)
    out = {}
    for mode, limit in (("resident_step_program", None), ("fused_chains", 0)):
        was = lib.hip_graph_set_resident(limit) if limit is not None else None
        try:
            x = mx.tensor(rng.standard_normal((rows, 3)).astype(np.float32)).with_grad()
            y = mx.tensor(rng.standard_normal((rows, 1)).astype(np.float32))
            lin = mx.Linear(in_features=3, out_features=1, with_bias=True, seed=3)
            mx.train(lin, x, y, 0.01, 100)
            mx.synchronize()
            t0 = time.perf_counter()
            mx.train(lin, x, y, 0.01, epochs)
            mx.synchronize()
            out[mode] = round((time.perf_counter() - t0) / epochs * 1e6, 1)
        finally:
            if was is not None:
                lib.hip_graph_set_resident(was)
    return out


def _oracle_host(threads):
    from tests.helpers import ensure_oracle_built, oracle_host
    lib = C.CDLL(ensure_oracle_built(), mode=C.RTLD_GLOBAL)
    lib.oracle_set_num_threads.restype = C.c_int
    cores = lib.oracle_set_num_threads(threads)
    mo = oracle_host()
    # the baseline is the reference's own sequence of backend calls: none of the host layer's shortcuts
    mo.set_autograd_shortcuts(False)
    mo.set_sum_all_in_one_pass(False)
    mo.set_conv_skip_unread_grad_cols(False)
    mo.set_conv_gathered_products(0)
    return mo, cores


def cpu_baseline_mlp(args):
    """The same loop with the host layer instantiated over the CPU oracle; the faster of the oracle's two modes
    (sequential, or threaded over all cores like the reference's rayon loops) is reported."""
    best = None
    for threads in (1, 0):
        mo, cores = _oracle_host(threads)
        lin, x, y = _mlp_setup(mo)
        mo.train(lin, x, y, 0.01, 5)
        t0, n = time.perf_counter(), 0
        while time.perf_counter() - t0 < 5.0:
            mo.train(lin, x, y, 0.01, 50)
            n += 50
        rate = n / (time.perf_counter() - t0)
        if best is None or rate > best[0]:
            best = (rate, cores, n)
    return {"value": round(best[0], 1), "unit": "steps/s", "cores": best[1], "kind": "port",
            "sample": f"same loop, {best[2]} steps on {best[1]} thread(s) (best of sequential and all-core modes)"}


def _conv_setup(mx, B, seed=0x5EED0004):
    rng = np.random.default_rng(seed)
    Cin = Cout = 64
    H = W = 56
    bound = 1.0 / np.sqrt(Cin * 9)
    x = mx.tensor(rng.standard_normal((B, Cin, H, W), dtype=np.float32)).with_grad()
    w = mx.tensor(rng.uniform(-bound, bound, (Cout, Cin, 3, 3)).astype(np.float32))
    b = mx.tensor(rng.uniform(-bound, bound, (Cout,)).astype(np.float32))
    target = mx.tensor(rng.standard_normal((B, Cout, H, W), dtype=np.float32))
    return mx.Conv2d(w, b, stride=(1, 1), padding=(1, 1)), x, target


def _conv_step(mx, conv, x, target):
    loss = mx.mse_loss(conv.forward(x), target)
    loss.backward()
    conv.zero_grad()
    return loss


def run_conv(args):
    """configs[4]: Conv2d(64->64, 3x3, stride 1, pad 1, bias) forward + MSE + backward on [32,64,56,56] f32 through
    the host layer (im2col -> GEMM -> bias add; backward: strided copy, GEMM, col2im, GEMM, bias sums)."""
    L, lib, alloc = hip_backend()
    from maidenx_amd.tensor import host
    mx = host()
    conv, x, target = _conv_setup(mx, 32)
    # (50 steps at least: the figure settles after about 20)
    args = argparse.Namespace(**{**vars(args), "steps": max(args.steps, 50)})
    for _ in range(max(args.warmup, 2)):
        _conv_step(mx, conv, x, target)
    mx.synchronize()
    mx.reset_backend_calls()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        _conv_step(mx, conv, x, target)
    mx.synchronize()
    dt_s = time.perf_counter() - t0
    calls = mx.backend_calls() / args.steps
    # the same steps with the product behind the input gradient made whole, as the reference makes it (col2im reads its
    # leading ninth only: nn/layers/conv.rs:391, crates/maidenx_cpu/src/nn/conv.rs:135)
    mx.set_conv_skip_unread_grad_cols(False)
    try:
        for _ in range(2):
            _conv_step(mx, conv, x, target)
        mx.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            _conv_step(mx, conv, x, target)
        mx.synchronize()
        whole_s = time.perf_counter() - t0
    finally:
        mx.set_conv_skip_unread_grad_cols(True)
    result = base_result(args, round(args.steps / dt_s, 2), "steps/s", dt_s, "f32",
                         "configs[4]: Conv2d 64->64 3x3 s1 p1 + bias, MSE loss, forward + backward, input [32,64,56,56] f32",
                         {"backend_kernels_per_step": calls,
                          "grad_cols_rows_computed": "11151 of 100352 (the rows col2im reads; same gradients as the whole product)",
                          "steps_per_s_with_whole_grad_cols": round(args.steps / whole_s, 2)})
    # the data-movement kernels of this config, each timed on its own through the C ABI (HIP events); the dominant
    # one, im2col, gives the roofline object
    Bn, Cc, H, W = 32, 64, 56, 56
    n_in, n_col, n_pad = Bn * Cc * H * W, Bn * H * W * Cc * 9, Bn * Cc * (H + 2) * (W + 2)
    # every launch works on the next of several buffer sets (16 for the 25 MB images, 4 for the 231 MB column matrix), so
    # that none finds its operands in the 256 MB last-level cache
    SETS = 16
    srcs, pads = [L.DeviceBuffer(n_in * 4) for _ in range(SETS)], [L.DeviceBuffer(n_pad * 4) for _ in range(SETS)]
    cols = [L.DeviceBuffer(n_col * 4) for _ in range(4)]
    for b in srcs:
        lib.hip_fill_f32(n_in, b.ptr, 1.0)
    for b in pads:
        lib.hip_fill_f32(n_pad, b.ptr, 1.0)
    for b in cols:
        lib.hip_fill_f32(n_col, b.ptr, 1.0)
    md = u64(Bn, Cc, H, W, 3, 3, H, W, 1, 1, 1, 1)
    mdp = u64([Bn, Cc, H, W], [Cc * H * W, H * W, W, 1], 0, [Bn, Cc, H + 2, W + 2], [0, 0, 0, 0, 1, 1, 1, 1])
    S, Cl, P = (lambda i: srcs[i % SETS].ptr), (lambda i: cols[i % 4].ptr), (lambda i: pads[i % SETS].ptr)
    solo = {
        "im2col": (lib.hip_conv2d_im2col_f32, lambda i: (n_col, md.ctypes.data, S(i), Cl(i)), (n_in + n_col) * 4),
        # the layer's call: num_els = B*C*H*W, so only the first 25.7 MB of the column matrix are read (nn/layers/conv.rs:393)
        "col2im (layer call)": (lib.hip_conv2d_col2im_f32, lambda i: (n_in, md.ctypes.data, Cl(i), S(i)), 2 * n_in * 4),
        "col2im (whole column matrix)": (lib.hip_conv2d_col2im_f32, lambda i: (n_col, md.ctypes.data, Cl(i), S(i)), (n_in + n_col) * 4),
        "pad_with_constant": (lib.hip_pad_with_constant_f32, lambda i: (n_in, n_pad, 4, mdp.ctypes.data, S(i), P(i), 0.0), (n_in + n_pad) * 4),
        "pad_with_constant_backward": (lib.hip_pad_with_constant_backward_f32, lambda i: (n_in, n_pad, 4, mdp.ctypes.data, P(i), S(i)), (n_in + n_pad) * 4),
    }
    kernels = {}
    ms = C.c_float()
    for name, (fn, fargs, nbytes) in solo.items():
        # one event pair around SETS back-to-back launches (the 10 us kernels here are shorter than the gap an event
        # pair of their own would add), three times over
        durs = []
        for rnd in range(4):
            a, b = C.c_void_p(), C.c_void_p()
            lib.hip_event_create(C.byref(a)); lib.hip_event_create(C.byref(b))
            lib.hip_event_record(a)
            for i in range(SETS):
                fn(*fargs(i))
            lib.hip_event_record(b)
            lib.hip_event_synchronize(b)
            lib.hip_event_elapsed_ms(a, b, C.byref(ms))
            lib.hip_event_destroy(a); lib.hip_event_destroy(b)
            if rnd:                      # the first round warms up
                durs.append(ms.value / SETS)
        L.check()
        kernels[name] = {"us": round(float(np.mean(durs)) * 1e3, 1), "GB/s": round(nbytes / float(np.mean(durs)) / 1e6, 1),
                         "hbm_frac": round(nbytes / float(np.mean(durs)) / 1e6 / HBM_PEAK_GBS, 4)}
        if name == "im2col":
            result["roofline"] = hbm_roofline("im2col_band_kernel<float> (hip_conv2d_im2col_f32, [32,64,56,56] 3x3), operands rotated", nbytes, durs)
            result["roofline"]["launches_timed"] = 3 * SETS
            result["roofline"]["algorithmic_bytes"] = nbytes
            src = "profiles/conv2d_32x64x56x56_kernel_trace.txt"
            result["roofline"]["traffic"], when = profile_traffic(src, "im2col_f32/32x64x56x56/3x3")
            result["roofline"]["traffic_source"] = f"{src} (rocprofv3 --pmc, measured {when})" if when else None
    result["config"]["kernels_alone"] = kernels
    worst = min(kernels, key=lambda k: kernels[k]["hbm_frac"])
    result["roofline"]["worst_of_chain"] = dict(kernel=worst, **kernels[worst])
    del srcs, pads, cols
    result["cpu_baseline"] = None if args.no_cpu_baseline else cpu_baseline_conv(args)
    return result


def cpu_baseline_conv(args):
    """The same step on the CPU oracle, threaded, on a bounded sample: batch 2 instead of 32 (the step is linear in
    the batch), scaled to full-size steps per second."""
    mo, cores = _oracle_host(0)
    conv, x, target = _conv_setup(mo, 2)
    _conv_step(mo, conv, x, target)
    t0, n = time.perf_counter(), 0
    while time.perf_counter() - t0 < 10.0:
        _conv_step(mo, conv, x, target)
        n += 1
    el = time.perf_counter() - t0
    return {"value": round(n / el / 16.0, 4), "unit": "steps/s", "cores": cores, "kind": "port",
            "sample": f"{n} steps at batch 2 in {el:.1f} s, divided by 16 for batch 32"}


def run_kernels(args):
    """Every kernel of the backend on its own, buffers rotated so that HBM serves them (maidenx_amd/kernel_bench.py).
    The table goes to stderr as it is measured and into config.kernels; value = the contiguous f32 multiply."""
    from maidenx_amd import kernel_bench
    t0 = time.perf_counter()
    rows = kernel_bench.run("", out=sys.stderr)
    dt_s = time.perf_counter() - t0
    mul = next(r for r in rows if r["kernel"] == "mul_f32/contig")
    res = base_result(args, mul["GB/s"], "GB/s", dt_s, "f32", "every backend kernel alone on the configs' shapes, operands rotated among 4 allocations (not cache-warm)",
                      {"kernels": rows})
    res["steps"], res["warmup"], res["ms_per_step"] = 1, 0, round(dt_s * 1e3, 1)
    res["roofline"] = {"bound": "hbm", "kernel": "ew_nd_kernel<OpMul<float>,4> (hip_mul_f32, contiguous [8192,8192])", "achieved": mul["GB/s"],
                       "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(mul["GB/s"] / HBM_PEAK_GBS, 4), "avg_launch_us": mul["us"],
                       "launches_timed": 20, "traffic": None}
    res["cpu_baseline"] = None
    return res


def run_all(args):
    """All five configurations in this process, one JSON line: the top level is configs[1] (the elementwise chain, which
    BASELINE's "HBM GB/s elemwise" is quoted on); config.results carries every configuration's own figures."""
    import gc
    res = run_elementwise(args)
    keys = ("value", "unit", "ms_per_step", "steps", "warmup", "dtype", "roofline", "cpu_baseline", "note")
    results = {"elementwise": {k: res[k] for k in keys if k in res}}
    results["elementwise"]["workload"] = res["config"]["workload"]
    for name, fn in (("reduce", run_reduce), ("matmul", run_matmul), ("mlp", run_mlp), ("conv", run_conv)):
        gc.collect()
        t0 = time.perf_counter()
        try:
            r = fn(args)
            results[name] = {k: r[k] for k in keys if k in r}
            results[name]["config"] = r["config"]
        except Exception as e:      # noqa: BLE001 - one configuration failing must not hide the others' figures
            results[name] = {"error": f"{type(e).__name__}: {e}"}
        results[name]["wall_s"] = round(time.perf_counter() - t0, 1)
    res["config"]["results"] = results
    res["config"]["workload"] = "all five configs in one run; top-level value/roofline/cpu_baseline = " + res["config"]["workload"]
    res["summary"] = {
        "train steps/s (configs[0] MLP)": results["mlp"].get("value"),
        "HBM GB/s elementwise chain (configs[1])": results["elementwise"]["value"],
        "HBM GB/s reduce chain (configs[2])": results["reduce"].get("value"),
        "matmul TFLOP/s bf16 4096^3 fwd+bwd (configs[3])": results["matmul"].get("value"),
        "conv2d steps/s (configs[4])": results["conv"].get("value"),
    }
    return res


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=10)
    ap.add_argument("--warmup", type=int, default=2)
    ap.add_argument("--workload", default="all")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-graph-floor", action="store_true", help="mlp: leave out the empty-graph replay measurement")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one MI355X; nothing in this backend uses a second GPU (--gpus must be 1)")
    runners = {"all": run_all, "elementwise": run_elementwise, "reduce": run_reduce, "matmul": run_matmul, "copy": run_copy, "mlp": run_mlp, "conv": run_conv, "kernels": run_kernels}
    if args.workload not in runners:
        sys.exit(f"unknown workload {args.workload}: choose from {sorted(runners)}")
    res = runners[args.workload](args)
    print(json.dumps(res))


if __name__ == "__main__":
    main()
