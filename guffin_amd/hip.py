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


def packed_bytes(dtype, K, N):
    lib().guffin_hip_packed_bytes.restype = C.c_uint64
    return lib().guffin_hip_packed_bytes(dtype, K, N)


def repack(dtype, canonical, K, N):
    tiles = torch.empty_like(canonical)
    check(lib().guffin_hip_repack(_stream(), dtype, _p(canonical), _p(tiles), K, N))
    return tiles


def unpack(dtype, tiles, K, N):
    canonical = torch.empty_like(tiles)
    check(lib().guffin_hip_unpack(_stream(), dtype, _p(tiles), _p(canonical), K, N))
    return canonical


def group_sums(x, out=None):
    rows, K = x.shape
    if out is None:
        out = torch.empty((rows, K // 16 + K // 32), dtype=torch.float32, device=x.device)
    check(lib().guffin_hip_group_sums(_stream(), _p(x), _p(out), rows, K))
    return out


def gemv_packed_slices(dtype, K, N):
    lib().guffin_hip_gemv_packed_slices.restype = C.c_uint32
    return lib().guffin_hip_gemv_packed_slices(dtype, K, N)


def gemv_packed(dtype, tiles, x, xsums, N, partials=None, out=None, reduce=True):
    rows, K = x.shape
    S = gemv_packed_slices(dtype, K, N)
    if partials is None:
        partials = torch.empty((S, rows, N), dtype=torch.float32, device=x.device)
    if reduce and out is None:
        out = torch.empty((rows, N), dtype=torch.float32, device=x.device)
    check(lib().guffin_hip_gemv_packed(_stream(), dtype, _p(tiles), _p(x), _p(xsums), _p(partials),
                                       _p(out) if reduce else C.c_void_p(0), rows, K, N))
    return out if reduce else partials
