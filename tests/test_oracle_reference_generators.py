"""The restated generators against the formats' decoders: every scale, offset and quant a generator asks for comes
back out of the oracle's dequantisation (which the reference's KATs and its compiled code pin elsewhere)."""
import numpy as np

import reference_generators as rg


def test_stress_matrices_decode_to_their_formulas(gfo):
    shared, columns, seed = 3840, 7, 137
    nblk = shared // 256
    column = np.repeat(np.arange(columns), nblk)[:, None]
    block = np.tile(np.arange(nblk), columns)[:, None]
    e = np.arange(256)[None, :]
    # Q6_K: d s (q - 32)
    raw = (seed + 11 * column + 7 * block + 13 * (e // 16)) % 63 - 31
    scale = np.where(raw == 0, -17, raw)
    want = (np.float32(0.03125) * scale.astype(np.float32)) * ((seed + 5 * column + 3 * block + 17 * e) % 64 - 32).astype(np.float32)
    got = gfo.dequant(2, rg.q6k_stress(shared, columns, seed)).reshape(-1, 256)
    assert np.array_equal(got, want.astype(np.float32))
    # Q4_K: d sc q - dmin m
    sc = 1 + (seed + 17 * column + 11 * block + 9 * (e // 32)) % 63
    mn = 1 + (seed + 13 * column + 7 * block + 15 * (e // 32)) % 63
    q = (seed + 3 * column + 5 * block + 7 * e) % 16
    want = (np.float32(0.125) * sc.astype(np.float32)) * q.astype(np.float32) - np.float32(0.03125) * mn.astype(np.float32)
    got = gfo.dequant(1, rg.q4k_stress(shared, columns, seed)).reshape(-1, 256)
    assert np.array_equal(got, want.astype(np.float32))


def test_plain_matrices_and_patterns(gfo):
    got = gfo.dequant(1, rg.q4k_plain(512, 3, 5)).reshape(3, 512)
    assert got.min() >= 0 and got.max() <= 5 * 15 and np.all(got == np.round(got))
    got = gfo.dequant(2, rg.q6k_plain(512, 3, 5)).reshape(3, 512)
    assert np.abs(got).max() <= 0.5 * 3 * 15 and np.all(got * 2 == np.round(got * 2))
    v = rg.projection_values(2, 11)
    assert v[0, 0] == -0.25 and set(np.unique(v * 8)) <= set(range(-5, 6))
    p = rg.pattern(10, 0.03)
    assert abs(p[0] - 0.03 * 0.37) < 1e-7 and np.abs(p).max() < 0.03 * 1.37 + 1e-6


def test_q8_0_quantiser_restated(gfo):
    """The Q8_0 quantiser of the reference's tests: a block's largest element maps to +-127, every decoded value is
    within half a step of its source, the scale is the half nearest max / 127, and a zero block stays zero."""
    shared, columns = 128, 5
    values = (((np.arange(shared * columns) % 31).astype(np.float32) - 15) / np.float32(37.0)).reshape(shared, columns)
    values[32:64, 2] = 0.0
    stream = rg.q8_0_from_values(values)
    blocks = stream.reshape(columns, shared // 32, 34)
    quants = blocks[:, :, 2:].view(np.int8)
    scales = np.ascontiguousarray(blocks[:, :, 0:2]).view(np.float16).reshape(columns, shared // 32).astype(np.float32)
    source = values.astype(np.float16).astype(np.float32).T.reshape(columns, shared // 32, 32)
    peak = np.abs(source).max(2)
    assert np.array_equal(scales, (peak / np.float32(127.0)).astype(np.float16).astype(np.float32))
    assert np.all(np.abs(quants).max(2)[peak > 0] == 127) and np.all(quants[2, 1] == 0) and scales[2, 1] == 0
    decoded = gfo.dequant(0, stream).reshape(columns, shared // 32, 32)
    step = (peak / 127.0)[:, :, None]
    assert np.all(np.abs(decoded - source) <= 0.5 * step * (1 + 2.0 ** -10) + 1e-12)
