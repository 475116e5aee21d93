"""GPU parity of the block decoders and dequant-GEMVs against the CPU oracle.

Bars: dequantised weights bit-exact; GEMV outputs within 1e-3 relative of the oracle's
sequential fp32 sums (relative to the row's RMS output, plus the operator bound
gamma*sum|x*w| the reference's own GPU tests use, tests/tensor/gemma3_metal_tests.cpp:454-470);
a row of a 2-row call bit-equal to the 1-row call on that row (:452-453, 1223-1224).
"""
import numpy as np
import pytest

from guffin_amd import synth
from bounds import assert_within_operator_bound

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def hip():
    import torch
    from guffin_amd import hip as module
    module.init(0)
    return module


def dev(a):
    import torch
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


@pytest.mark.parametrize("dtype", [0, 1, 2])
def test_dequant_bit_exact(hip, gfo, dtype):
    blocks = synth.make_blocks(dtype, 4096, seed=100 + dtype)
    got = hip.dequant(dtype, dev(blocks.reshape(-1)), 4096).cpu().numpy()
    want = gfo.dequant(dtype, blocks)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


def check_gemv(hip, gfo, dtype, K, N, rows, seed):
    w = synth.make_weight(dtype, K, N, seed)
    x = synth.make_activation(rows, K, seed + 1)
    y = hip.gemv(dtype, dev(w), dev(x), N).cpu().numpy()
    ref = gfo.gemv(dtype, w, x, N, threads=8)
    scale = np.sqrt((ref.astype(np.float64) ** 2).mean(axis=1, keepdims=True))
    err = np.abs(y.astype(np.float64) - ref)
    assert np.all(err <= 1e-3 * scale), (dtype, K, N, rows, float((err / scale).max()))
    # the reference's own bar for this operator: a few 1e-6 of sum|x*w| against a double dot product
    assert_within_operator_bound(gfo, dtype, w, x, y, K, N)
    return y


SHAPES = [
    (1, 3840, 4096), (1, 3840, 2048), (2, 3840, 2048), (1, 4096, 3840), (1, 3840, 1536),
    (1, 15360, 384), (2, 3840, 2048), (2, 15360, 3840), (0, 640, 1024), (0, 1024, 640),
    (0, 2048, 640), (0, 640, 2048), (1, 256, 8), (2, 256, 8), (1, 512, 7), (2, 768, 13), (0, 32, 5),
]


@pytest.mark.parametrize("dtype,K,N", SHAPES)
@pytest.mark.parametrize("rows", [1, 2])
def test_gemv_parity(hip, gfo, dtype, K, N, rows):
    check_gemv(hip, gfo, dtype, K, N, rows, seed=7)


@pytest.mark.parametrize("dtype,K,N", [(1, 3840, 2048), (2, 3840, 2048), (2, 15360, 512), (0, 640, 1024), (1, 15360, 256)])
def test_two_row_rows_equal_one_row_calls(hip, gfo, dtype, K, N):
    w = dev(synth.make_weight(dtype, K, N, 9))
    x = synth.make_activation(2, K, 10)
    both = hip.gemv(dtype, w, dev(x), N).cpu().numpy()
    for r in range(2):
        one = hip.gemv(dtype, w, dev(x[r:r + 1]), N).cpu().numpy()
        assert np.array_equal(one[0].view(np.uint32), both[r].view(np.uint32))
    again = hip.gemv(dtype, w, dev(x), N).cpu().numpy()
    assert np.array_equal(again.view(np.uint32), both.view(np.uint32))  # deterministic


@pytest.mark.parametrize("dtype", [0, 1, 2])
def test_gemv_three_and_five_rows(hip, gfo, dtype):
    K, N = (640, 96) if dtype == 0 else (512, 40)
    for rows in (3, 5):
        check_gemv(hip, gfo, dtype, K, N, rows, seed=20 + rows)


@pytest.mark.parametrize("dtype", [0, 1, 2])
def test_gemv_unit_vectors_recover_columns(hip, gfo, dtype):
    # y is linear in x: a unit vector returns the dequantised weights bit for bit
    K, N = 256, 24
    w = synth.make_weight(dtype, K, N, 30)
    dense = gfo.dequant(dtype, w).reshape(N, K)
    for k in (0, 17, 32, 100, 255):
        x = np.zeros((1, K), np.float32)
        x[0, k] = 1.0
        y = hip.gemv(dtype, dev(w), dev(x), N).cpu().numpy()[0]
        assert np.allclose(y, dense[:, k], rtol=2e-6, atol=1e-6), k


def test_gemv_cancellation_fixture(hip, gfo):
    # every weight is the small difference of two large terms d*sc*q - dmin*m
    # (tests/tensor/gemma3_metal_tests.cpp:1291-1365 builds the same kind of block)
    K, N = 1024, 16
    blocks = synth.make_blocks(1, N * 4, seed=40)
    for b in blocks:
        b[0:2] = np.array([np.float16(1.0)], np.float16).view(np.uint8)
        b[2:4] = np.array([np.float16(15.0)], np.float16).view(np.uint8)
        for g in range(8):
            synth.q4k_set_scale_min(b, g, 63, 63)
        b[16:144] = 0xFF  # q = 15 everywhere: 63*15 - 15*63 = 0 exactly, then perturb
        for e in range(0, 256, 5):
            synth.q4k_set_nibble(b, e, 14)
    w = blocks.reshape(-1)
    x = synth.make_activation(2, K, 41)
    y = hip.gemv(1, dev(w), dev(x), N).cpu().numpy()
    ref = gfo.gemv(1, w, x, N)
    dense = gfo.dequant(1, w).reshape(N, K).astype(np.float64)
    big = 63.0 * 15.0 * np.abs(x.astype(np.float64)).sum(axis=1, keepdims=True)
    # the factored sum carries the large terms: error scales with them, not with the result
    assert np.all(np.abs(y - ref) <= 4e-6 * big)
    assert np.all(np.abs(y - x.astype(np.float64) @ dense.T) <= 4e-6 * big)


def test_gemv_rejects_bad_arguments(hip):
    import torch
    w = torch.zeros(144 * 8, dtype=torch.uint8, device="cuda")
    x = torch.zeros((1, 256), dtype=torch.float32, device="cuda")
    with pytest.raises(hip.GuffinError):
        hip.gemv(1, w, torch.zeros((1, 100), dtype=torch.float32, device="cuda"), 8)
    with pytest.raises(hip.GuffinError):
        hip.gemv(1, w, torch.zeros((9, 256), dtype=torch.float32, device="cuda"), 8)
    with pytest.raises(hip.GuffinError):
        hip.gemv(5, w, x, 8)
