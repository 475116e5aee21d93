"""Pins the oracle's block decoders and sequential GEMV (CPU only).

Known-answer blocks restate tests/tensor/tensor_tests.cpp:474-503 (Q8_0), :539-559 and
:658-676 (Q4_K, built as tests/support/tensor_test_support.cpp:223-241 builds it),
:678-721 (Q6_K, tensor_test_support.cpp:243-262), and the all-groups Q4_K / signed-scale
Q6_K cases of tests/scripts/gemma3_target_reference_tests.py:40-69.
"""
import numpy as np
import pytest

from guffin_amd import synth


def f16bits(v):
    return np.array([v], np.float16).view(np.uint16)[0]


def q4k_reference_block():
    b = np.zeros(144, np.uint8)
    b[0:2] = np.array([0x3C00], np.uint16).view(np.uint8)
    b[2:4] = np.array([0x3800], np.uint16).view(np.uint8)
    synth.q4k_set_scale_min(b, 0, 2, 1)
    synth.q4k_set_scale_min(b, 1, 3, 2)
    synth.q4k_set_scale_min(b, 4, 6, 5)
    for e, v in ((0, 4), (31, 15), (32, 5), (63, 6), (128, 7)):
        synth.q4k_set_nibble(b, e, v)
    return b


def q6k_reference_block():
    b = np.zeros(210, np.uint8)
    b[208:210] = np.array([0x3800], np.uint16).view(np.uint8)
    for g, s in ((0, 2), (1, 3), (2, -3), (4, 4), (8, -2)):
        synth.q6k_set_scale(b, g, s)
    # a zeroed block holds q = -32 everywhere; set the named elements
    for e, v in ((0, -32), (31, 31), (32, -1), (64, 5), (128, 7)):
        synth.q6k_set_value(b, e, v)
    return b


def test_q8_0_known_block(gfo):
    b = np.array([0x00, 0x38, 0x00, 0x02, 0xFE, 0x7F, 0x80] + list(range(4, 0x3A, 2)), np.uint8)
    assert b.size == 34
    v = gfo.dequant(gfo.Q8_0, b)
    assert list(v[:5]) == [0.0, 1.0, -1.0, 63.5, -64.0]
    assert v[5] == 2.0 and v[31] == 28.0


def test_q4_k_known_block_and_dot(gfo):
    b = q4k_reference_block()
    v = gfo.dequant(gfo.Q4_K, b)
    assert v[0] == 7.5 and v[32] == 14.0 and v[128] == 39.5 and v[31] == 29.5 and v[63] == 17.0
    x = np.zeros((1, 256), np.float32)
    x[0, 0], x[0, 32], x[0, 128] = 1.0, 2.0, -1.0
    assert gfo.gemv(gfo.Q4_K, b, x, 1)[0, 0] == -4.0


def test_q6_k_known_block_and_dot(gfo):
    b = q6k_reference_block()
    v = gfo.dequant(gfo.Q6_K, b)
    assert v[0] == -32.0 and v[32] == 1.5 and v[64] == 10.0 and v[31] == 46.5 and v[128] == -7.0
    x = np.zeros((1, 256), np.float32)
    x[0, 0], x[0, 32], x[0, 64], x[0, 128] = 1.0, 2.0, -1.0, 3.0
    assert gfo.gemv(gfo.Q6_K, b, x, 1)[0, 0] == -60.0


def test_q4_k_all_groups_closed_form(gfo):
    # scales [0,1,15,16,31,32,47,63], mins reversed, negative dmin: value = d*sc*q - dmin*m
    scales = [0, 1, 15, 16, 31, 32, 47, 63]
    mins = scales[::-1]
    b = np.zeros(144, np.uint8)
    b[0:2] = np.array([f16bits(0.5)], np.uint16).view(np.uint8)
    b[2:4] = np.array([f16bits(-0.25)], np.uint16).view(np.uint8)
    for g in range(8):
        synth.q4k_set_scale_min(b, g, scales[g], mins[g])
    q = (np.arange(256) * 7 + 3) % 16
    for e in range(256):
        synth.q4k_set_nibble(b, e, int(q[e]))
    v = gfo.dequant(gfo.Q4_K, b)
    g = np.arange(256) // 32
    want = 0.5 * np.array(scales)[g] * q + 0.25 * np.array(mins)[g]
    assert np.array_equal(v, want.astype(np.float32))


def test_q6_k_all_bit_planes_closed_form(gfo):
    b = np.zeros(210, np.uint8)
    b[208:210] = np.array([f16bits(0.125)], np.uint16).view(np.uint8)
    scales = [(-128 + 17 * g) if g % 2 else (127 - 13 * g) for g in range(16)]
    for g in range(16):
        synth.q6k_set_scale(b, g, scales[g])
    q = ((np.arange(256) * 11 + 5) % 64) - 32
    for e in range(256):
        synth.q6k_set_value(b, e, int(q[e]))
    v = gfo.dequant(gfo.Q6_K, b)
    want = 0.125 * np.array(scales)[np.arange(256) // 16] * q
    assert np.array_equal(v, want.astype(np.float32))


@pytest.mark.parametrize("dtype", [0, 1, 2])
def test_dequant_matches_compiled_reference(gfo, ref, dtype):
    if ref is None:
        pytest.skip("oracle/_ref not built (no reference checkout)")
    blocks = synth.make_blocks(dtype, 64, seed=11 + dtype)
    a = gfo.dequant(dtype, blocks)
    b = gfo.dequant(dtype, blocks, which=ref)
    assert np.array_equal(a.view(np.uint32), b.view(np.uint32))


@pytest.mark.parametrize("dtype,K", [(0, 640), (1, 512), (2, 768)])
def test_gemv_matches_compiled_reference_bit_exact(gfo, ref, dtype, K):
    if ref is None:
        pytest.skip("oracle/_ref not built (no reference checkout)")
    N = 24
    w = synth.make_weight(dtype, K, N, seed=3)
    x = synth.make_activation(2, K, seed=4)
    a = gfo.gemv(dtype, w, x, N)
    b = gfo.gemv(dtype, w, x, N, which=ref)
    c = gfo.gemv(dtype, w, x, N, as_written=True)
    d = gfo.gemv(dtype, w, x, N, threads=3)
    assert np.array_equal(a.view(np.uint32), b.view(np.uint32))
    assert np.array_equal(a.view(np.uint32), c.view(np.uint32))
    assert np.array_equal(a.view(np.uint32), d.view(np.uint32))


@pytest.mark.parametrize("dtype", [0, 1, 2])
def test_gemv_unit_vectors_recover_dequantised_columns(gfo, dtype):
    K, N = 256, 5
    w = synth.make_weight(dtype, K, N, seed=21)
    dense = gfo.dequant(dtype, w).reshape(N, K)
    for k in (0, 31, 32, 127, 255):
        x = np.zeros((1, K), np.float32)
        x[0, k] = 1.0
        y = gfo.gemv(dtype, w, x, N)[0]
        assert np.array_equal(y, dense[:, k] + np.float32(0.0))


@pytest.mark.parametrize("dtype", [0, 1, 2])
def test_gemv_against_double_dot_with_operator_bound(gfo, dtype):
    # |err| <= gamma_K/(1-gamma_K) * sum|x*w| for a sequential fp32 sum (plus the product rounding)
    K, N = 1024, 16
    w = synth.make_weight(dtype, K, N, seed=5)
    x = synth.make_activation(2, K, seed=6)
    dense = gfo.dequant(dtype, w).reshape(N, K).astype(np.float64)
    y = gfo.gemv(dtype, w, x, N).astype(np.float64)
    exact = x.astype(np.float64) @ dense.T
    gamma = (K + 1) * 2.0 ** -24
    bound = gamma / (1 - gamma) * (np.abs(x.astype(np.float64)) @ np.abs(dense).T)
    assert np.all(np.abs(y - exact) <= bound + 1e-30)


def test_f16_decode_all_bit_patterns(gfo, ref):
    bits = np.arange(65536, dtype=np.uint16)
    want = bits.view(np.float16).astype(np.float32)
    # NaN payloads do not survive the float -> Python double -> float32 trip: compare NaN-ness
    got = np.array([gfo.lib().gfo_f16_to_f32(int(b)) for b in bits[::7]], np.float32)
    nan = np.isnan(want[::7])
    assert np.array_equal(np.isnan(got), nan)
    assert np.array_equal(got[~nan].view(np.uint32), want[::7][~nan].view(np.uint32))
    if ref is not None:
        r = np.array([ref.gfr_f16_to_f32(int(b)) for b in bits[::7]], np.float32)
        assert np.array_equal(got[~nan].view(np.uint32), r[~nan].view(np.uint32))
