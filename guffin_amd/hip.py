"""ctypes binding of libguffin_hip.so over torch device tensors."""
import ctypes as C
import os

import torch

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libguffin_hip.so")

Q8_0, Q4_K, Q6_K = 0, 1, 2


class GuffinError(RuntimeError):
    def __init__(self, code, message):
        super().__init__("guffin_hip error %d: %s" % (code, message))
        self.code = code


_lib = None
_inited = set()


def lib():
    """Loads the built library; raises if it is missing (no fallback path exists)."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError(
                "%s is missing: build it with `python -m guffin_amd.build` "
                "(hipcc --offload-arch=gfx950); guffin_amd has no CPU fallback" % LIB_PATH)
        _lib = C.CDLL(LIB_PATH)
        _lib.guffin_hip_last_error.restype = C.c_char_p
        _lib.guffin_hip_arch.restype = C.c_char_p
    return _lib


def check(rc):
    if rc != 0:
        raise GuffinError(rc, lib().guffin_hip_last_error().decode())


def init(device=0):
    if device not in _inited:
        if not torch.cuda.is_available():
            raise RuntimeError("guffin_amd needs a gfx950 GPU; none is visible")
        check(lib().guffin_hip_init(device))
        _inited.add(device)


def _stream():
    return C.c_void_p(torch.cuda.current_stream().cuda_stream)


def _p(t):
    return C.c_void_p(t.data_ptr()) if t is not None else C.c_void_p(0)


def dequant(dtype, blocks, n_blocks):
    elems = 32 if dtype == Q8_0 else 256
    out = torch.empty(n_blocks * elems, dtype=torch.float32, device=blocks.device)
    check(lib().guffin_hip_dequant(_stream(), dtype, _p(blocks), C.c_uint64(n_blocks), _p(out)))
    return out


def gemv(dtype, w, x, N, out=None):
    rows, K = x.shape
    if out is None:
        out = torch.empty((rows, N), dtype=torch.float32, device=x.device)
    check(lib().guffin_hip_gemv(_stream(), dtype, _p(w), _p(x), _p(out), rows, K, N))
    return out
