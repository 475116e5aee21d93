"""Decode GEMV, output head and embedding on the reference's own deterministic operands (tests/reference_generators.py)
with the reference's own criteria:
  tests/tensor/gemma3_metal_tests.cpp:426-470   stress Q4_K / Q6_K matrices against pattern() rows: rows of a two-row
                                                call bit-equal to one-row calls, each within gamma / (1 - gamma) sum|x w|
                                                + 1e-6 of a double dot, gamma = (K / 32 + 32) eps
  tests/tensor/gemma3_metal_tests.cpp:511-548   the tied Q6_K matrix as embedding (2e-6 of the decoded value times
                                                sqrt(hidden)) and as head (3e-5 of a double dot)
  tests/tensor/gemma3_metal_tests.cpp:1290-1365  Q4_K weights that are the difference of two terms 1365 times larger,
                                                against signed activations, within the same gamma bound on the SMALL
                                                weights: both the canonical-layout GEMV and the packed GEMV (which keeps
                                                d sc sum(q x) and dmin m sum(x) apart until the end of a group) meet it
                                                (measured: 0.45 and 0.28 of it at K = 3840, 0.13 and 0.06 at K = 15360)
  tests/tensor/tensor_backend_tests.cpp:964-1158 the 17 small-batch / tile-boundary cases and the 17 parallel-projection
                                                cases (12B block counts, odd column counts, a head that starts inside the
                                                input), activations with a 512-fold range inside every 32-group
  tests/tensor/tensor_backend_tests.cpp:1352-1472 one-row decode at the reference's block and column counts; the Q8_0
                                                output projection on weights through the reference's quantiser
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
    worst = {"packed": 0.0, "canonical": 0.0, "matrix": 0.0}
    xall = dev(x)
    matrix_rows = hip.prefill_gemm(1, tiles, hip.prefill_pack(xall), rows, width, 64).cpu().numpy()[:, :columns]
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
        worst["matrix"] = max(worst["matrix"], float((np.abs(matrix_rows[row] - reference) / bound).max()))
    print("cancellation fixture, K = %d: packed %.2f, canonical %.2f, matrix path %.2f of the reference's bound"
          % (width, worst["packed"], worst["canonical"], worst["matrix"]), flush=True)
    assert worst["canonical"] <= 1.0
    assert worst["packed"] <= 1.0
    # the fixture is the reference's for its one-to-five-row verify matmul; the prefill GEMM, whose B operand is
    # the pattern sc q (13 here: seven leading zeros below bit 10), is reported beside it and held to four times
    # the bound (measured 2.5 at K = 3840, 1.1 at K = 15360)
    assert worst["matrix"] <= 4.0


# tests/tensor/tensor_backend_tests.cpp:964-1067: the reference's 17 (rows, 256-blocks of K, columns) cases around its
# small-batch / tile boundaries, production block counts and the 64-column boundary, on the stress matrices, with
# every 17th activation 16 times and every 13th 1/32 of its pattern value.
PROJECTION_CASES = [(2, 1, 1), (2, 14, 3), (2, 16, 4), (2, 56, 5), (3, 2, 2), (4, 14, 3), (5, 16, 4), (6, 56, 5), (7, 1, 63),
                    (8, 2, 64), (9, 14, 65), (15, 16, 5), (16, 56, 4), (17, 1, 3), (31, 2, 2), (32, 14, 1), (33, 16, 5)]


@pytest.mark.parametrize("dtype", [1, 2])
@pytest.mark.parametrize("rows,blocks,columns", PROJECTION_CASES)
def test_small_batch_and_tiled_projection_cases(hip, gfo, dtype, rows, blocks, columns):
    """The reference holds its backend to 0.05-2.0 absolute + 1e-5..2e-2 relative of a float reference here and,
    up to 8 rows, to bit-equality with one-row calls.  Here every row of the matrix path is held to the operator
    bound gamma / (1 - gamma) sum|x w| + 1e-6 of a double dot, and the decode path (one- and two-row calls) is
    bit-equal row by row and within 2e-5 of the row RMS of the matrix path."""
    K = blocks * 256
    x = rg.projection_values(rows, K).reshape(-1)
    i = np.arange(x.size)
    x = np.where(i % 17 == 0, x * np.float32(16.0), np.where(i % 13 == 0, x * np.float32(0.03125), x)).astype(np.float32)
    x = x.reshape(rows, K)
    w = rg.q4k_stress(K, columns, rows) if dtype == 1 else rg.q6k_stress(K, columns, rows)
    N = (columns + 63) // 64 * 64
    dense = gfo.dequant(dtype, w).reshape(columns, K).astype(np.float64)
    tiles = hip.repack(dtype, dev(padded(w, dtype, K, columns, N)), K, N)
    xd = dev(x)
    y = hip.prefill_gemm(dtype, tiles, hip.prefill_pack(xd), rows, K, N).cpu().numpy()
    assert np.all(y[:, columns:] == 0)
    gamma = (K // 32 + 32) * np.finfo(np.float32).eps
    products = np.abs(dense)[None, :, :] * np.abs(x.astype(np.float64))[:, None, :]
    bound = gamma / (1.0 - gamma) * products.sum(2) + 1e-6
    exact = x.astype(np.float64) @ dense.T
    worst = float((np.abs(y[:, :columns] - exact) / bound).max())
    assert worst <= 1.0, worst
    rms = np.sqrt((exact ** 2).mean(1)) + 1e-30
    for r in (0, 1, rows - 1):
        one = dev(x[r:r + 1])
        single = hip.gemv_packed(dtype, tiles, one, hip.group_sums(one), N).cpu().numpy()[0]
        assert float((np.abs(single[:columns] - exact[r]) / bound[r]).max()) <= 1.0
        assert np.all(np.abs(single[:columns].astype(np.float64) - y[r, :columns]) <= 2e-5 * rms[r])
        if r + 1 < rows:
            two = dev(x[r:r + 2])
            both = hip.gemv_packed(dtype, tiles, two, hip.group_sums(two), N).cpu().numpy()
            assert np.array_equal(both[0].view(np.uint32), single.view(np.uint32)), "one-row and two-row calls differ"
    print("rows %d blocks %d columns %d dtype %d: matrix path at %.3f of the bound" % (rows, blocks, columns, dtype, worst), flush=True)


# tests/tensor/tensor_backend_tests.cpp:1069-1158: the 12B model's K dimensions (15, 16 and 60 blocks) with odd column
# counts, batches of 1-8 rows and a head that starts `head_offset` rows into the input.
PARALLEL_CASES = [(2, 1, 1, 1), (1, 15, 3, 0), (2, 15, 5, 1), (3, 15, 7, 3), (4, 15, 33, 4), (5, 15, 65, 5), (1, 16, 5, 1),
                  (2, 16, 67, 3), (3, 16, 3, 4), (4, 16, 4, 5), (5, 16, 7, 1), (1, 60, 3, 3), (2, 60, 4, 4), (3, 60, 5, 5),
                  (4, 60, 5, 1), (5, 60, 7, 3), (8, 60, 3, 1)]


@pytest.mark.parametrize("dtype", [1, 2])
@pytest.mark.parametrize("rows,blocks,columns,head_offset", PARALLEL_CASES)
def test_parallel_projection_keeps_scalar_bits(hip, gfo, dtype, rows, blocks, columns, head_offset):
    """A batch of verify rows (here: calls of at most two rows, the width of a verify pass) and a head over rows
    that start `head_offset` into the input give, row by row, the bits of one-row calls; every value is finite and
    within the reference's 0.05 (Q4_K) / 0.1 (Q6_K) + 1e-5 |e| of a double dot; the row after the batch in the
    output keeps its NaN pattern.  (The reference compares with a sequential fp32 sum; here the comparison is with
    a double dot, and the oracle's sequential sum's own error on these operands -- up to 3e-2 at 60 blocks -- is
    printed beside the kernel's.)"""
    import torch
    K = blocks * 256
    input_rows = rows + head_offset
    i = np.arange(input_rows * K)
    x = rg.projection_values(input_rows, K).reshape(-1)
    x = (x * np.where(i % 17 == 0, np.float32(16.0), np.where(i % 13 == 0, np.float32(0.03125), np.float32(1.0))).astype(np.float32)
         + np.float32(0.00037) * (i % 11).astype(np.float32)).astype(np.float32).reshape(input_rows, K)
    w = rg.q4k_stress(K, columns, rows) if dtype == 1 else rg.q6k_stress(K, columns, rows)
    N = (columns + 63) // 64 * 64
    tiles = hip.repack(dtype, dev(padded(w, dtype, K, columns, N)), K, N)
    sequential = gfo.gemv(dtype, padded(w, dtype, K, columns, N), x, N, threads=4)[:, :columns]
    dense = gfo.dequant(dtype, w).reshape(columns, K).astype(np.float64)
    expected = x.astype(np.float64) @ dense.T
    xd = dev(x)
    worst = 0.0

    def one(r):
        xr = xd[r:r + 1].contiguous()
        return hip.gemv_packed(dtype, tiles, xr, hip.group_sums(xr), N).cpu().numpy()[0]

    scalar = [one(r) for r in range(input_rows)]
    for first in (0, head_offset):
        out = torch.full((rows + 1, N), float("nan"), dtype=torch.float32, device="cuda")
        out.view(torch.int32)[...] = 0x7fc00000
        for r in range(0, rows, 2):
            n = min(2, rows - r)
            xr = xd[first + r:first + r + n].contiguous()
            hip.gemv_packed(dtype, tiles, xr, hip.group_sums(xr), N, out=out[r:r + n])
        got = out.cpu().numpy()
        assert np.all(got[rows].view(np.uint32) == 0x7fc00000), "the row after the batch was written"
        for r in range(rows):
            assert np.all(np.isfinite(got[r]))
            assert np.array_equal(got[r].view(np.uint32), scalar[first + r].view(np.uint32)), (first, r)
            e = expected[first + r]
            tol = (0.05 if dtype == 1 else 0.1) + 1e-5 * np.abs(e)
            assert np.all(np.abs(got[r, :columns] - e) <= tol), float(np.abs(got[r, :columns] - e).max())
            worst = max(worst, float(np.abs(got[r, :columns] - e).max()))
    print("rows %d blocks %d columns %d dtype %d: worst error %.2e, the sequential fp32 sum's %.2e"
          % (rows, blocks, columns, dtype, worst, float(np.abs(sequential - expected).max())), flush=True)


@pytest.mark.parametrize("dtype,width", [(0, 640), (0, 2048), (1, 256), (1, 3840), (1, 15360), (2, 3840), (2, 15360)])
def test_range_inside_a_group_costs_no_precision(hip, gfo, dtype, width):
    """Activations whose magnitudes span 2^9 inside every 32-group and use all their mantissa bits: the packed GEMV
    and the prefill GEMM stay within 2 eps sum|x w| of a double dot (the canonical-layout GEMV: 0.1-0.5).  The
    quants enter the matrix instruction as fp16 bit patterns below 2048, which it does not normalise: with the
    pattern's leading zeros in place (a nibble in bits 0-3) every product loses that many bits once a sum's
    products are aligned, and these operands came out 70 times worse than the canonical kernel (up to 200 eps
    on a single group); the quants therefore sit near the top of the 11-bit window (bits 4-7 for Q4_K, 4-9
    for Q6_K, 3-10 for the biased Q8_0 byte; the prefill GEMM's scaled quants reach it by themselves)."""
    from guffin_amd import synth
    columns, rows = 64, 4
    i = np.arange(rows * width)
    x = rg.projection_values(rows, width).reshape(-1)
    x = (x * np.where(i % 17 == 0, np.float32(16.0), np.where(i % 13 == 0, np.float32(0.03125), np.float32(1.0))).astype(np.float32)
         + np.float32(0.00037) * (i % 11).astype(np.float32)).astype(np.float32).reshape(rows, width)
    w = (synth.make_weight(0, width, columns, 3) if dtype == 0 else
         rg.q4k_stress(width, columns, 2) if dtype == 1 else rg.q6k_stress(width, columns, 2))
    dense = gfo.dequant(dtype, w).reshape(columns, width).astype(np.float64)
    stream = dev(w)
    tiles = hip.repack(dtype, stream, width, columns)
    xd = dev(x)
    exact = x.astype(np.float64) @ dense.T
    unit = np.finfo(np.float32).eps * (np.abs(x.astype(np.float64)) @ np.abs(dense).T)
    two = xd[:2].contiguous()
    packed = hip.gemv_packed(dtype, tiles, two, hip.group_sums(two), columns).cpu().numpy()
    canonical = hip.gemv(dtype, stream, two, columns).cpu().numpy()
    matrix = hip.prefill_gemm(dtype, tiles, hip.prefill_pack(xd), rows, width, columns).cpu().numpy()
    worst = [float((np.abs(packed - exact[:2]) / unit[:2]).max()), float((np.abs(matrix - exact) / unit).max()),
             float((np.abs(canonical - exact[:2]) / unit[:2]).max())]
    print("dtype %d K %d: packed %.2f, matrix path %.2f, canonical %.2f eps sum|x w|" % (dtype, width, *worst), flush=True)
    assert worst[0] <= 2.0 and worst[1] <= 2.0, worst


@pytest.mark.parametrize("dtype", [1, 2])
@pytest.mark.parametrize("blocks", [1, 2, 14, 16, 56])
def test_decode_boundary_cases(hip, gfo, dtype, blocks):
    """tests/tensor/tensor_backend_tests.cpp:1352-1392: one row against 1-7 columns of the stress matrices at the
    reference's block counts, every 17th activation times -8 and every 11th times 1/8; the reference's tolerance
    (0.1 for Q4_K, 0.25 for Q6_K, + 1e-5 |e|), here against a double dot."""
    K = blocks * 256
    x = rg.projection_values(1, K).reshape(-1)
    i = np.arange(K)
    x = np.where(i % 17 == 0, x * np.float32(-8.0), np.where(i % 11 == 0, x * np.float32(0.125), x)).astype(np.float32).reshape(1, K)
    xd = dev(x)
    receipt = hip.group_sums(xd)
    for columns in (1, 2, 3, 4, 5, 7):
        w = rg.q4k_stress(K, columns, blocks) if dtype == 1 else rg.q6k_stress(K, columns, blocks)
        dense = gfo.dequant(dtype, w).reshape(columns, K).astype(np.float64)
        tiles = hip.repack(dtype, dev(padded(w, dtype, K, columns)), K, 64)
        y = hip.gemv_packed(dtype, tiles, xd, receipt, 64).cpu().numpy()[0]
        exact = dense @ x[0].astype(np.float64)
        assert np.all(y[columns:] == 0)
        assert np.all(np.abs(y[:columns] - exact) <= (0.1 if dtype == 1 else 0.25) + 1e-5 * np.abs(exact))


@pytest.mark.parametrize("shared", [64, 3584])
def test_q8_0_output_projection(hip, gfo, shared):
    """tests/tensor/tensor_backend_tests.cpp:1423-1472: weights ((i % 31) - 15) / 37 through the reference's Q8_0
    quantiser, activations ((i % 17) - 8) / 9, one and two rows within 2e-4 of the CPU path (here the oracle's
    sequential GEMV); rows of the two-row call equal the one-row calls (bit for bit here, 2e-4 there)."""
    columns = 5
    a = ((np.arange(2 * shared) % 17).astype(np.float32) - 8) / np.float32(9.0)
    wv = (((np.arange(shared * columns) % 31).astype(np.float32) - 15) / np.float32(37.0)).reshape(shared, columns)
    w = rg.q8_0_from_values(wv)
    stream = np.concatenate([w, np.zeros((64 - columns) * (shared // 32) * 34, np.uint8)])
    dense = gfo.dequant(0, w).reshape(columns, shared)
    assert np.abs(dense - wv.T).max() <= np.abs(wv).max() / 127.0        # the quantiser restated: half a step at most
    tiles = hip.repack(0, dev(stream), shared, 64)
    x = a.reshape(2, shared).astype(np.float32)
    both = None
    for rows in (1, 2):
        xd = dev(x[:rows])
        got = hip.gemv_packed(0, tiles, xd, hip.group_sums(xd), 64).cpu().numpy()
        cpu = gfo.gemv(0, stream, x[:rows], 64, threads=1)
        assert np.all(np.abs(got[:, :columns] - cpu[:, :columns]) <= 2e-4)
        if rows == 2:
            both = got
    for row in range(2):
        xr = dev(x[row:row + 1])
        single = hip.gemv_packed(0, tiles, xr, hip.group_sums(xr), 64).cpu().numpy()[0]
        assert np.array_equal(single.view(np.uint32), both[row].view(np.uint32))
