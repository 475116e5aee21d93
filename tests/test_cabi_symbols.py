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
