"""CPU: the C-ABI library loads without a GPU and exports every symbol include/maidenx_hip.h declares."""
import ctypes
import os
import re
import subprocess

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    out = subprocess.run(["gcc", "-E", "-P", os.path.join(ROOT, "include", "maidenx_hip.h")], check=True, capture_output=True, text=True).stdout
    return sorted(set(re.findall(r"\b(hip_[a-z0-9_]+)\s*\(", out)))


def test_header_is_valid_c_and_cxx():
    hdr = os.path.join(ROOT, "include", "maidenx_hip.h")
    for comp, lang in (("gcc", "c"), ("g++", "c++")):
        subprocess.run([comp, "-x", lang, "-fsyntax-only", "-Wall", "-Werror", hdr], check=True)


def test_library_exports_every_declared_symbol():
    import maidenx_amd.lib as L
    lib = ctypes.CDLL(L.LIB_PATH)
    names = declared_symbols()
    assert len(names) > 150
    missing = [n for n in names if not hasattr(lib, n)]
    assert not missing, missing


def test_python_binding_covers_the_header():
    import maidenx_amd._signatures as S
    bound = {"hip_" + n for n in {**S.signatures(), **S.binary_signatures(), **S.extension_signatures()}}
    runtime = {"hip_get_last_status", "hip_status_string", "hip_set_device", "hip_get_device", "hip_device_count", "hip_malloc",
               "hip_free", "hip_memcpy_h2d", "hip_memcpy_d2h", "hip_memcpy_d2d", "hip_stream_create", "hip_stream_destroy",
               "hip_stream_synchronize", "hip_set_stream", "hip_get_stream", "hip_synchronize", "hip_event_create",
               "hip_event_destroy", "hip_event_record", "hip_event_synchronize", "hip_event_elapsed_ms",
               "hip_graph_begin_capture", "hip_graph_end_capture", "hip_graph_launch", "hip_graph_destroy",
               "hip_graph_is_program", "hip_graph_set_programs", "hip_graph_fused_launches", "hip_graph_set_fusion",
               "hip_noalloc_prepare", "hip_scratch_allocations", "hip_graph_launch_n", "hip_graph_is_resident",
               "hip_graph_set_resident", "hip_buffer_discard", "hip_conv2d_forward_product_f32"}
    assert set(declared_symbols()) == bound | runtime


def host_symbols():
    out = subprocess.run(["gcc", "-E", "-P", os.path.join(ROOT, "include", "maidenx_host.h")], check=True, capture_output=True, text=True).stdout
    return sorted(set(re.findall(r"\b(mxt_[a-z0-9_]+)\s*\(", out)))


def test_host_header_is_valid_c_and_cxx():
    hdr = os.path.join(ROOT, "include", "maidenx_host.h")
    for comp, lang in (("gcc", "c"), ("g++", "c++")):
        subprocess.run([comp, "-x", lang, "-fsyntax-only", "-Wall", "-Werror", hdr], check=True)


def test_host_library_exports_every_declared_symbol():
    # loads without a GPU (no HIP call happens at load time); the oracle-backed build exports the same ABI
    from helpers import ORACLE_HOST_LIB, ensure_oracle_built
    from maidenx_amd.tensor import HOST_LIB_PATH
    ensure_oracle_built()
    names = host_symbols()
    assert len(names) >= 40
    for path in (HOST_LIB_PATH, ORACLE_HOST_LIB):
        lib = ctypes.CDLL(path)
        missing = [n for n in names if not hasattr(lib, n)]
        assert not missing, (path, missing)
