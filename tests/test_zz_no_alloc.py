"""guffin_hip_gemv_packed_static (the packed GEMV whose partial planes live in the library's static
device array, for callers that cannot allocate) against guffin_hip_gemv_packed on the same inputs:
bit-equal results on two calls in a row, the second with a smaller input, and with a launch that
needs no planes in between; sizes beyond the array are refused before anything is enqueued."""
import ctypes as C

import numpy as np
import pytest

from guffin_amd import synth


def test_static_entry_point_refuses_what_does_not_fit_without_a_gpu():
    from guffin_amd import hip   # imports torch first, so that one HIP runtime serves the whole process
    lib = hip.lib()
    lib.guffin_hip_gemv_packed_static_limit.restype = C.c_uint64
    lib.guffin_hip_gemv_packed_slices.restype = C.c_uint32
    lib.guffin_hip_last_error.restype = C.c_char_p
    limit = lib.guffin_hip_gemv_packed_static_limit()
    assert limit == 32768
    buf = (C.c_uint8 * 4096)()
    p = C.c_void_p((C.addressof(buf) + 255) & ~255)
    K, N = 3840, 12160   # Q4_K: 190 column tiles are cut into two planes, 2 * 2 * 12160 floats at two rows
    assert lib.guffin_hip_gemv_packed_slices(1, K, N) * 2 * N > limit
    assert lib.guffin_hip_gemv_packed_static(None, 1, p, p, p, p, 2, K, N) == -4
    assert b"static scratch" in lib.guffin_hip_last_error()
    assert lib.guffin_hip_gemv_packed_static(None, 1, None, p, p, p, 2, K, N) == -1
    assert lib.guffin_hip_gemv_packed_static(None, 1, p, p, p, p, 3, K, 64) == -2
    assert lib.guffin_hip_gemv_packed_static(None, 1, p, p, p, p, 1, 100, 64) == -2


@pytest.mark.gpu
def test_static_scratch_gemv_equals_the_workspace_entry_point():
    import torch
    from guffin_amd import hip
    hip.init(0)

    def dev(a):
        return torch.from_numpy(np.ascontiguousarray(a)).cuda()

    # the down projection (Q6_K, four planes at two rows), then a smaller Q4_K launch (four planes, one
    # row), a launch that fills the array to its last float, one that writes its result directly (a single
    # plane of 131072 floats: no planes, so no limit), the first shape again and a small one
    cases = [(2, 15360, 3840, 2), (1, 4096, 3840, 1), (0, 640, 4096, 2), (1, 3840, 65536, 2), (2, 15360, 3840, 2),
             (0, 1024, 640, 1)]
    for i, (dtype, K, N, rows) in enumerate(cases):
        print("static gemv case", i, dtype, K, N, rows, flush=True)
        w = synth.make_weight(dtype, K, N, seed=200 + i)
        x = dev(synth.make_activation(rows, K, seed=300 + i))
        tiles = hip.repack(dtype, dev(w), K, N)
        sums = hip.group_sums(x)
        want = hip.gemv_packed(dtype, tiles, x, sums, N)
        got = torch.full((rows, N), float("nan"), dtype=torch.float32, device="cuda")
        hip.gemv_packed_static(dtype, tiles, x, sums, N, got)
        torch.cuda.synchronize()
        planes = hip.gemv_packed_slices(dtype, K, N)
        assert planes == 1 or planes * rows * N <= 32768
        assert torch.equal(got.view(torch.int32), want.view(torch.int32)), (i, dtype, K, N, rows)
