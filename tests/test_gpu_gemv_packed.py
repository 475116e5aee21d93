"""GPU parity of the wave-tile repack and the packed GEMV.

Bars: repack -> unpack restores every byte (the reference pins its own repack the same
way, tests/tensor/tensor_tests.cpp:3193-3283); packed GEMV within 1e-3 relative of the
oracle's sequential fp32 sums; rows of a 2-row call bit-equal to 1-row calls; the packed
and canonical-layout kernels agree to fp32 rounding.
"""
import numpy as np
import pytest

from guffin_amd import synth
from bounds import assert_within_operator_bound

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def hip():
    from guffin_amd import hip as module
    module.init(0)
    return module


def dev(a):
    import torch
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


@pytest.mark.parametrize("dtype,K,N", [(0, 640, 128), (1, 768, 192), (2, 512, 64), (1, 3840, 2048), (2, 3840, 256)])
def test_repack_round_trip_is_lossless(hip, dtype, K, N):
    w = synth.make_weight(dtype, K, N, seed=50 + dtype)
    wd = dev(w)
    tiles = hip.repack(dtype, wd, K, N)
    assert hip.packed_bytes(dtype, K, N) == w.size
    back = hip.unpack(dtype, tiles, K, N).cpu().numpy()
    assert np.array_equal(back, w)
    t = tiles.cpu().numpy()
    assert not np.array_equal(t, w)
    # spot-check the documented tile layouts
    bb = synth.BLOCK_BYTES[dtype]
    nblk = K // synth.BLOCK_ELEMS[dtype]
    col, b = 70 % N, nblk - 1
    tile = t[((col // 64) * nblk + b) * 64 * bb:][:64 * bb]
    blk = w[(col * nblk + b) * bb:][:bb]
    lane = col % 64
    if dtype == 1:
        # matrix-core tile: header = piece 8 of the column's lane; quant chunk ch, k-slice s of
        # column 16*cg + j = bytes (ch % 2)*8.. of piece 2*cg + ch/2, lane 16*s + j
        assert np.array_equal(tile[8 * 1024 + lane * 16:][:16], blk[0:16])
        cg, j, ch, sl = lane // 16, lane % 16, 1, 2
        assert np.array_equal(tile[(2 * cg + ch // 2) * 1024 + (16 * sl + j) * 16 + (ch % 2) * 8:][:8],
                              blk[16 + 32 * ch + 8 * sl:][:8])
    elif dtype == 2:
        # ql byte (half n, run m, k-slice s): piece 2*cg + n, lane 16*s + j, byte 8*m; qh (half n,
        # k-slice s): piece 8 + cg, byte 8*n; scales piece 12 and d behind the pieces, by column
        cg, j, n, m, sl = lane // 16, lane % 16, 1, 1, 3
        assert np.array_equal(tile[(2 * cg + n) * 1024 + (16 * sl + j) * 16 + 8 * m:][:8],
                              blk[64 * n + 32 * m + 8 * sl:][:8])
        assert np.array_equal(tile[(8 + cg) * 1024 + (16 * sl + j) * 16 + 8 * n:][:8], blk[128 + 32 * n + 8 * sl:][:8])
        assert np.array_equal(tile[12288 + lane * 16:][:16], blk[192:208])
        assert np.array_equal(tile[13312 + lane * 2:][:2], blk[208:210])
    else:
        # quant k-slice s: piece cg/2, lane 16*s + j, byte 8*(cg % 2); d behind the pieces
        cg, j, sl = lane // 16, lane % 16, 2
        assert np.array_equal(tile[(cg // 2) * 1024 + (16 * sl + j) * 16 + 8 * (cg % 2):][:8], blk[2 + 8 * sl:][:8])
        assert np.array_equal(tile[2048 + lane * 2:][:2], blk[0:2])


def test_group_sums(hip):
    x = synth.make_activation(2, 3840, seed=60)
    s = hip.group_sums(dev(x)).cpu().numpy()
    want16 = x.reshape(2, -1, 16).astype(np.float64).sum(-1)
    want32 = x.reshape(2, -1, 32).astype(np.float64).sum(-1)
    assert s.shape == (2, 240 + 120)
    assert np.allclose(s[:, :240], want16, rtol=0, atol=2e-5)
    assert np.allclose(s[:, 240:], want32, rtol=0, atol=3e-5)


SHAPES = [
    (1, 3840, 4096), (1, 3840, 2048), (2, 3840, 2048), (1, 4096, 3840), (1, 3840, 15360),
    (2, 15360, 3840), (1, 15360, 3840), (0, 640, 1024), (0, 1024, 640), (0, 2048, 640),
    (0, 640, 2048), (1, 256, 64), (2, 256, 64), (0, 32, 64), (2, 768, 128),
]


@pytest.mark.parametrize("dtype,K,N", SHAPES)
@pytest.mark.parametrize("rows", [1, 2])
def test_packed_gemv_parity(hip, gfo, dtype, K, N, rows):
    w = synth.make_weight(dtype, K, N, seed=7)
    x = synth.make_activation(rows, K, seed=8)
    wd, xd = dev(w), dev(x)
    tiles = hip.repack(dtype, wd, K, N)
    y = hip.gemv_packed(dtype, tiles, xd, hip.group_sums(xd), N).cpu().numpy()
    ref = gfo.gemv(dtype, w, x, N, threads=8)
    scale = np.sqrt((ref.astype(np.float64) ** 2).mean(axis=1, keepdims=True))
    err = np.abs(y.astype(np.float64) - ref)
    assert np.all(err <= 1e-3 * scale), float((err / scale).max())
    # the reference's operator bound against a double dot product (a dropped low half of the operand
    # or a wrong multiplier on one 32-group is orders of magnitude outside it)
    assert_within_operator_bound(gfo, dtype, w, x, y, K, N)
    # and against the canonical-layout kernel: both are fp32 sums of the same products
    yc = hip.gemv(dtype, wd, xd, N).cpu().numpy()
    assert np.all(np.abs(y.astype(np.float64) - yc) <= 2e-5 * scale)


@pytest.mark.parametrize("dtype,K,N", [(1, 3840, 2048), (2, 3840, 2048), (2, 15360, 512), (0, 640, 1024), (1, 15360, 256)])
def test_packed_two_row_rows_equal_one_row_calls(hip, dtype, K, N):
    w = hip.repack(dtype, dev(synth.make_weight(dtype, K, N, 9)), K, N)
    x = synth.make_activation(2, K, 10)
    xd = dev(x)
    both = hip.gemv_packed(dtype, w, xd, hip.group_sums(xd), N).cpu().numpy()
    for r in range(2):
        xr = dev(x[r:r + 1])
        one = hip.gemv_packed(dtype, w, xr, hip.group_sums(xr), N).cpu().numpy()
        assert np.array_equal(one[0].view(np.uint32), both[r].view(np.uint32))
    again = hip.gemv_packed(dtype, w, xd, hip.group_sums(xd), N).cpu().numpy()
    assert np.array_equal(again.view(np.uint32), both.view(np.uint32))


@pytest.mark.parametrize("dtype", [0, 1, 2])
def test_packed_unit_vectors_recover_columns(hip, gfo, dtype):
    K, N = 256, 64
    w = synth.make_weight(dtype, K, N, 30)
    dense = gfo.dequant(dtype, w).reshape(N, K)
    tiles = hip.repack(dtype, dev(w), K, N)
    for k in (0, 17, 33, 100, 255):
        x = np.zeros((1, K), np.float32)
        x[0, k] = 1.0
        xd = dev(x)
        y = hip.gemv_packed(dtype, tiles, xd, hip.group_sums(xd), N).cpu().numpy()[0]
        assert np.allclose(y, dense[:, k], rtol=2e-6, atol=2e-6), k


def f32_information_case(dtype, rows, width, columns):
    """tests/tensor/gemma3_metal_tests.cpp:1419-1499: one non-zero per row, 1 + (row + 1) 2^-20, which a half
    cannot hold, against weights whose first block scale is the half 0x3555 (about 1/3, not a power of two), so
    that neither operand survives narrowing to 16 bits; returns (weights, activations, inner index per row)."""
    w = synth.make_weight(dtype, width, columns, seed=51 if dtype == 1 else 71)
    bb, scale_offset = (144, 0) if dtype == 1 else (210, 208)
    for column in range(columns):
        at = column * (width // 256) * bb + scale_offset
        w[at], w[at + 1] = 0x55, 0x35
    x = np.zeros((rows, width), np.float32)
    inner = [(row % 8) * 33 for row in range(rows)]
    for row in range(rows):
        x[row, inner[row]] = np.float32(1.0 + (row + 1) * 2.0 ** -20)
    return w, x, inner


def assert_f32_information(gfo, dtype, w, x, inner, y, width, columns):
    """The reference's bound is 4 eps |x w| + 1e-6.  Q4_K meets it as written.  For Q6_K the kernels form
    d s (sum q x - 32 sum x) with q the stored 0..63 (the matrix core takes unsigned quants), not d s sum (q - 32) x:
    both terms are exact to fp32, but their difference carries their rounding, so the bound here is 4 eps on the
    two terms, |x w| + 32 |d s x| — wider than the reference's by at most (q + 32) / |q - 32|, still far below what
    a half-staged operand loses (2^-11)."""
    dense = gfo.dequant(dtype, w).reshape(columns, width)
    discriminates = False
    d_half = np.float32(np.array([0x3555], np.uint16).view(np.float16)[0])
    for row, k in enumerate(inner):
        expected = (x[row, k] * dense[:, k]).astype(np.float32)
        terms = np.abs(expected)
        if dtype == 2:
            scales = np.array([np.int8(w[c * (width // 256) * 210 + 192 + k // 16]) for c in range(columns)], np.float32)
            terms = terms + 32.0 * np.abs(d_half * scales * x[row, k])
        bound = 4.0 * np.finfo(np.float32).eps * terms + 1e-6
        assert np.all(np.abs(y[row] - expected) <= bound), (row, float(np.max(np.abs(y[row] - expected) / bound)))
        narrowed = np.float32(np.float16(x[row, k])) * dense[:, k].astype(np.float16).astype(np.float32)
        discriminates |= bool(np.any(np.abs(expected - narrowed) > 16.0 * bound))
    assert discriminates          # the fixture must be able to tell half operands from fp32 ones


@pytest.mark.parametrize("dtype", [1, 2])
def test_packed_gemv_keeps_all_f32_operand_information(hip, gfo, dtype):
    width, columns = 3840, 64
    w, x, inner = f32_information_case(dtype, 33, width, columns)
    tiles = hip.repack(dtype, dev(w), width, columns)
    got = np.zeros((33, columns), np.float32)
    for r0 in range(0, 33, 2):                       # rows in pairs (and one single row), as a verify pass sees them
        xr = dev(x[r0:r0 + 2])
        got[r0:r0 + 2] = hip.gemv_packed(dtype, tiles, xr, hip.group_sums(xr), columns).cpu().numpy()
    assert_f32_information(gfo, dtype, w, x, inner, got, width, columns)


def test_packed_partials_sum_in_slice_order(hip):
    dtype, K, N = 1, 3840, 1024
    w = hip.repack(dtype, dev(synth.make_weight(dtype, K, N, 11)), K, N)
    xd = dev(synth.make_activation(2, K, 12))
    xs = hip.group_sums(xd)
    S = hip.gemv_packed_slices(dtype, K, N)
    assert 1 <= S <= K // 256
    parts = hip.gemv_packed(dtype, w, xd, xs, N, reduce=False).cpu().numpy()
    y = hip.gemv_packed(dtype, w, xd, xs, N).cpu().numpy()
    total = parts[0].copy()
    for s in range(1, S):
        total = total + parts[s]
    assert np.array_equal(total.view(np.uint32), y.view(np.uint32))


MULTI = [
    ((1, 1, 2), 3840, (4096, 2048, 2048)),   # 12B q/k/v with a Q6_K value projection
    ((1, 1, 1), 3840, (4096, 2048, 2048)),
    ((1, 1), 3840, (15360, 15360)),          # 12B gate/up
    ((2, 2), 768, (128, 64)),
    ((0, 0, 0), 640, (1024, 256, 256)),      # 270M q/k/v
    ((0, 0), 640, (2048, 2048)),
]


@pytest.mark.parametrize("dtypes,K,Ns", MULTI)
@pytest.mark.parametrize("rows", [1, 2])
def test_packed_multi_matches_single_launches(hip, gfo, dtypes, K, Ns, rows):
    x = synth.make_activation(rows, K, seed=40)
    xd = dev(x)
    xs = hip.group_sums(xd)
    ws = [synth.make_weight(dt, K, N, seed=41 + i) for i, (dt, N) in enumerate(zip(dtypes, Ns))]
    tiles = [hip.repack(dt, dev(w), K, N) for dt, w, N in zip(dtypes, ws, Ns)]
    parts = hip.gemv_packed_multi(dtypes, tiles, xd, xs, Ns)
    assert len({p.shape[0] for p in parts}) == 1            # one slice count per launch
    for dt, w, t, N, p in zip(dtypes, ws, tiles, Ns, parts):
        assert p.shape[1:] == (rows, N)
        y = p.cpu().numpy().astype(np.float64).sum(axis=0)
        ref = gfo.gemv(dt, w, x, N, threads=8)
        scale = np.sqrt((ref.astype(np.float64) ** 2).mean(axis=1, keepdims=True))
        assert np.all(np.abs(y - ref) <= 1e-3 * scale)
        single = hip.gemv_packed(dt, t, xd, xs, N).cpu().numpy()
        assert np.all(np.abs(y - single) <= 2e-5 * scale)


def test_packed_multi_rejects_mixed_block_lengths(hip):
    import torch
    x = torch.zeros((1, 256), dtype=torch.float32, device="cuda")
    xs = hip.group_sums(x)
    t = torch.zeros(144 * 64, dtype=torch.uint8, device="cuda")
    with pytest.raises(hip.GuffinError):
        hip.gemv_packed_multi((1, 0), [t, t], x, xs, (64, 64))


@pytest.mark.parametrize("dtype,K,F,rows,bit_equal", [(1, 3840, 15360, 2, True), (1, 3840, 15360, 1, True),
                                                     (0, 640, 2048, 1, False), (1, 512, 128, 2, False)])
def test_fused_gate_up_geglu_equals_the_three_launches(hip, dtype, K, F, rows, bit_equal):
    import torch
    x = synth.make_activation(rows, K, seed=80)
    xd = dev(x)
    xs = hip.group_sums(xd)
    gate = hip.repack(dtype, dev(synth.make_weight(dtype, K, F, seed=81)), K, F)
    up = hip.repack(dtype, dev(synth.make_weight(dtype, K, F, seed=82)), K, F)
    pg, pu = hip.gemv_packed_multi((dtype, dtype), [gate, up], xd, xs, (F, F))
    want, want_sums = hip.geglu(pg, pu, planes=pg.shape[0], want_sums=True)
    h, sums = hip.gateup_geglu(dtype, gate, up, xd, xs, F)
    if bit_equal:   # same k-split as the unfused launch: identical arithmetic
        assert torch.equal(h.view(torch.int32), want.view(torch.int32))
    scale = float(want.abs().max())
    assert float((h - want).abs().max()) <= 3e-6 * scale
    assert float((sums - want_sums).abs().max()) <= 1e-4 * scale
    mult, image = hip.receipt_parts(sums, rows, F)
    mult_w, image_w = hip.receipt_parts(want_sums, rows, F)
    if bit_equal:
        assert torch.equal(mult, mult_w) and torch.equal(image.view(torch.int16), image_w.view(torch.int16))
    with pytest.raises(hip.GuffinError):
        hip.gateup_geglu(2, gate, up, xd, xs, F)


def test_packed_rejects_bad_arguments(hip):
    import torch
    w = torch.zeros(144 * 64, dtype=torch.uint8, device="cuda")
    x = torch.zeros((1, 256), dtype=torch.float32, device="cuda")
    with pytest.raises(hip.GuffinError):
        hip.repack(1, w, 256, 60)          # N not a multiple of 64
    with pytest.raises(hip.GuffinError):
        hip.gemv_packed(1, w, torch.zeros((3, 256), dtype=torch.float32, device="cuda"),
                        torch.zeros((3, 24), dtype=torch.float32, device="cuda"), 64)
    with pytest.raises(hip.GuffinError):
        hip.gemv_packed(1, w[8:], x, torch.zeros((1, 24), dtype=torch.float32, device="cuda"), 64)
