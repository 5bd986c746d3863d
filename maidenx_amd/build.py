"""Build libmaidenx_hip.so (the C-ABI backend) from the HIP sources in csrc/ for gfx950.

    python -m maidenx_amd.build [--force]

hipcc cross-compiles without a GPU.  Objects go to maidenx_amd/csrc/_obj/, the library to
maidenx_amd/libmaidenx_hip.so (in-tree, so that it travels with the source tree).
"""
import concurrent.futures
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(CSRC, "_obj")
LIB = os.path.join(HERE, "libmaidenx_hip.so")

# -ffp-contract=off : the reference never fuses a multiply-add, and f32 parity depends on it.
# -packed-fp32-ops off : keep the compiler from forming v_pk_*_f32.
HIPCC_FLAGS = [
    "-O3", "-std=c++17", "-fPIC", "--offload-arch=gfx950", "-ffp-contract=off",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function",
]


def _sources():
    return sorted(f for f in os.listdir(CSRC) if f.endswith(".hip"))


def _headers_mtime():
    return max(os.path.getmtime(os.path.join(CSRC, f)) for f in os.listdir(CSRC) if f.endswith(".hpp"))


def _compile(src, force):
    obj = os.path.join(OBJ, src[:-4] + ".o")
    path = os.path.join(CSRC, src)
    if not force and os.path.exists(obj) and os.path.getmtime(obj) > max(os.path.getmtime(path), _headers_mtime()):
        return obj, ""
    cmd = ["hipcc", "-c", *HIPCC_FLAGS, path, "-o", obj]
    p = subprocess.run(cmd, capture_output=True, text=True)
    log = "\n".join(l for l in (p.stdout + p.stderr).splitlines() if "packed-fp32-ops" not in l)
    if p.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src}:\n{log}")
    return obj, log


def build(force=False, verbose=False):
    os.makedirs(OBJ, exist_ok=True)
    srcs = _sources()
    with concurrent.futures.ThreadPoolExecutor(max_workers=min(8, len(srcs))) as ex:
        results = list(ex.map(lambda s: _compile(s, force), srcs))
    objs = [o for o, _ in results]
    if verbose:
        for _, log in results:
            if log.strip():
                print(log)
    if force or not os.path.exists(LIB) or any(os.path.getmtime(o) > os.path.getmtime(LIB) for o in objs):
        cmd = ["hipcc", "-shared", "-fPIC", "--offload-arch=gfx950", "-o", LIB, *objs]
        p = subprocess.run(cmd, capture_output=True, text=True)
        if p.returncode != 0:
            raise RuntimeError("link failed:\n" + p.stdout + p.stderr)
    build_host(force)
    return LIB


HOST_LIB = os.path.join(HERE, "libmaidenx_host.so")


def build_host(force=False):
    """libmaidenx_host.so: the C++ host layer (tensor / autograd / nn) above the C ABI.  Plain host code."""
    hdir = os.path.join(HERE, "host")
    srcs = [os.path.join(hdir, f) for f in os.listdir(hdir)] + [os.path.join(HERE, "..", "include", "maidenx_host.h"), LIB]
    if not force and os.path.exists(HOST_LIB) and os.path.getmtime(HOST_LIB) > max(os.path.getmtime(f) for f in srcs):
        return HOST_LIB
    # -fno-gnu-unique, -Bsymbolic: the layer's switches and counters are function-local statics of inline functions; as
    # GNU-unique symbols they would be ONE object for every build of the layer loaded into a process (this one and the
    # CPU oracle's), so that a switch set on one would set it on the other
    cmd = ["g++", "-O2", "-std=c++17", "-fPIC", "-shared", "-Wall", "-Wextra", "-fno-gnu-unique", os.path.join(hdir, "host_hip.cpp"), "-o", HOST_LIB,
           "-L" + HERE, "-lmaidenx_hip", "-Wl,-rpath,$ORIGIN", "-Wl,-Bsymbolic"]
    p = subprocess.run(cmd, capture_output=True, text=True)
    if p.returncode != 0:
        raise RuntimeError("host layer build failed:\n" + p.stdout + p.stderr)
    return HOST_LIB


if __name__ == "__main__":
    print(build(force="--force" in sys.argv, verbose=True))
