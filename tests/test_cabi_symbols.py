"""The C-ABI library loads on a CPU-only box and exports every declared symbol."""
import ctypes
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "guffin_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(guffin_hip_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_entry_point():
    path = os.path.join(ROOT, "guffin_amd", "libguffin_hip.so")
    assert os.path.exists(path), "build the library first: python -m guffin_amd.build"
    lib = ctypes.CDLL(path)
    names = declared_symbols()
    assert len(names) >= 8
    for name in names:
        assert hasattr(lib, name), name


def test_argument_errors_need_no_gpu():
    lib = ctypes.CDLL(os.path.join(ROOT, "guffin_amd", "libguffin_hip.so"))
    lib.guffin_hip_last_error.restype = ctypes.c_char_p
    assert lib.guffin_hip_arch is not None
    # null pointers and bad shapes are rejected before anything touches a device
    assert lib.guffin_hip_gemv(None, 1, None, None, None, 1, 256, 8) == -1
    buf = (ctypes.c_uint8 * 4096)()
    p = ctypes.addressof(buf)
    p16 = ctypes.c_void_p((p + 15) & ~15)
    assert lib.guffin_hip_gemv(None, 1, p16, p16, p16, 9, 256, 8) == -2
    assert lib.guffin_hip_gemv(None, 1, p16, p16, p16, 1, 100, 8) == -2
    assert lib.guffin_hip_gemv(None, 1, ctypes.c_void_p(p16.value + 2), p16, p16, 1, 256, 8) == -3
    assert lib.guffin_hip_gemv(None, 7, p16, p16, p16, 1, 256, 8) == -1
    assert b"gemv" in lib.guffin_hip_last_error()


def test_new_entry_points_reject_bad_arguments_without_a_gpu():
    lib = ctypes.CDLL(os.path.join(ROOT, "guffin_amd", "libguffin_hip.so"))
    buf = (ctypes.c_uint8 * 4096)()
    p = ctypes.c_void_p((ctypes.addressof(buf) + 255) & ~255)
    # ring-row copies: masks must be a power of two minus one, tokens must fit both sides
    assert lib.guffin_hip_kv_cache_copy(None, p, p, p, p, 0, 2, 5, 1, 256) == -1
    assert lib.guffin_hip_kv_cache_copy(None, p, p, p, p, 0, 3, 7, 1, 256) == -4
    assert lib.guffin_hip_kv_cache_copy(None, p, p, p, p, 0, 2, 7, 1, 12) == -2
    # drafter pre-pass: at most 64 history tokens, a positive penalty
    assert lib.guffin_hip_draft_process(None, p, 256, p, 65, ctypes.c_float(1.5), p) == -4
    assert lib.guffin_hip_draft_process(None, p, 256, p, 3, ctypes.c_float(0.0), p) == -1
    assert lib.guffin_hip_draft_process(None, p, 256, None, 3, ctypes.c_float(1.5), p) == -1


def test_bench_refuses_more_than_one_gpu():
    import subprocess
    import sys
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert r.returncode == 2 and "ONE GPU" in r.stderr and r.stdout == ""
