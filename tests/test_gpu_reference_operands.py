"""Decode GEMV, output head and embedding on the reference's own deterministic operands (tests/reference_generators.py)
with the reference's own criteria:
  tests/tensor/gemma3_metal_tests.cpp:426-470   stress Q4_K / Q6_K matrices against pattern() rows: rows of a two-row
                                                call bit-equal to one-row calls, each within gamma / (1 - gamma) sum|x w|
                                                + 1e-6 of a double dot, gamma = (K / 32 + 32) eps
  tests/tensor/gemma3_metal_tests.cpp:511-548   the tied Q6_K matrix as embedding (2e-6 of the decoded value times
                                                sqrt(hidden)) and as head (3e-5 of a double dot)
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
