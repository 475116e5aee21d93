"""GPU parity of the chunked-prefill path: matrix-core GEMM, causal attention, whole block graph.

Bars: GEMM rows within 1e-3 relative of the oracle's sequential fp32 row dots and within fp32
rounding of the packed GEMV on the same rows; attention within 2e-6 of a double softmax;
the ingested run's hidden rows within 1e-3 (relative to the row RMS) of the oracle's forward of
the same rows, and the published ring rows equal to the oracle's fp16 K/V up to rare rounding ties.
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


@pytest.mark.parametrize("dtype,K,N", [(1, 3840, 256), (2, 3840, 128), (0, 640, 256), (1, 256, 64), (2, 512, 192),
                                       (1, 768, 320), (1, 512, 384), (1, 256, 448), (2, 256, 320)])
@pytest.mark.parametrize("M", [1, 7, 33, 130])
def test_prefill_gemm_parity(hip, gfo, dtype, K, N, M):
    w = synth.make_weight(dtype, K, N, seed=70 + dtype)
    x = synth.make_activation(M, K, seed=71)
    x[M // 2] *= 300.0          # rows of very different magnitude share nothing
    x[0, ::7] *= 1e-3
    tiles = hip.repack(dtype, dev(w), K, N)
    xd = dev(x)
    y = hip.prefill_gemm(dtype, tiles, hip.prefill_pack(xd), M, K, N).cpu().numpy()
    ref = gfo.gemv(dtype, w, x, N, threads=8)
    scale = np.sqrt((ref.astype(np.float64) ** 2).mean(axis=1, keepdims=True))
    assert np.all(np.abs(y.astype(np.float64) - ref) <= 1e-3 * scale)
    assert_within_operator_bound(gfo, dtype, w, x, y, K, N, matrix_path=True)   # the reference's bound for its matrix path
    # the decode GEMV on the same rows computes the same exact products
    for r in (0, M - 1):
        xr = xd[r:r + 1].contiguous()
        one = hip.gemv_packed(dtype, tiles, xr, hip.group_sums(xr), N).cpu().numpy()[0]
        assert np.all(np.abs(one.astype(np.float64) - y[r]) <= 2e-5 * scale[r])


@pytest.mark.parametrize("dtype", [1, 2])
def test_prefill_gemm_keeps_all_f32_operand_information(hip, gfo, dtype):
    """tests/tensor/gemma3_metal_tests.cpp:1419-1499 on the matrix path: 33 rows (a ragged row group), operands
    that a half cannot hold."""
    from test_gpu_gemv_packed import assert_f32_information, f32_information_case
    width, columns = 3840, 64
    w, x, inner = f32_information_case(dtype, 33, width, columns)
    tiles = hip.repack(dtype, dev(w), width, columns)
    y = hip.prefill_gemm(dtype, tiles, hip.prefill_pack(dev(x)), 33, width, columns).cpu().numpy()
    assert_f32_information(gfo, dtype, w, x, inner, y, width, columns)


def test_prefill_gemm_down_projection_shape(hip, gfo):
    """Q6_K at the down projection's K = 15360 (60 blocks per column, the longest chain of LDS
    stages and weight prefetches) with an odd number of column tiles and rows in every row group."""
    dtype, K, N, M = 2, 15360, 192, 37
    w = synth.make_weight(dtype, K, N, seed=81)
    x = synth.make_activation(M, K, seed=82)
    x[5] *= 1e3
    tiles = hip.repack(dtype, dev(w), K, N)
    xd = dev(x)
    y = hip.prefill_gemm(dtype, tiles, hip.prefill_pack(xd), M, K, N).cpu().numpy()
    ref = gfo.gemv(dtype, w, x, N, threads=8)
    scale = np.sqrt((ref.astype(np.float64) ** 2).mean(axis=1, keepdims=True))
    assert np.all(np.abs(y.astype(np.float64) - ref) <= 1e-3 * scale)
    assert_within_operator_bound(gfo, dtype, w, x, y, K, N, matrix_path=True)
    for r in (0, 5, 24, M - 1):
        xr = xd[r:r + 1].contiguous()
        one = hip.gemv_packed(dtype, tiles, xr, hip.group_sums(xr), N).cpu().numpy()[0]
        assert np.all(np.abs(one.astype(np.float64) - y[r]) <= 2e-5 * scale[r])


@pytest.mark.parametrize("dtype,K,N", [(1, 3840, 15360), (2, 15360, 3840)])
def test_prefill_gemm_at_2048_rows(hip, gfo, dtype, K, N):
    """The benchmark's prompt length on the gate (Q4_K) and down (Q6_K) shapes: 64 row chunks x every
    column-tile group of the launch.  Rows sampled from the first, last and neighbouring chunks agree
    with the decode GEMV on the same row to fp32 rounding, and with a double dot product within the
    reference's bound for its matrix path (tests/tensor/gemma3_metal_tests.cpp:1280-1285)."""
    import torch
    M = 2048
    w = synth.make_weight(dtype, K, N, seed=90 + dtype)
    tiles = hip.repack(dtype, dev(w), K, N)
    gen = torch.Generator(device="cuda")
    gen.manual_seed(91)
    xd = torch.randn((M, K), device="cuda", generator=gen)
    xd[777] *= 300.0
    y = hip.prefill_gemm(dtype, tiles, hip.prefill_pack(xd), M, K, N)
    torch.cuda.synchronize()
    assert bool(torch.isfinite(y).all())
    rows = sorted(set([0, 1, 31, 32, 33, 63, 64, 127, 128, 1023, 1024, 1055, 1056, 2015, 2016, 2046, 2047]
                      + list(np.random.default_rng(3).integers(0, M, 23))))
    ys = y[rows].cpu().numpy().astype(np.float64)
    scale = np.sqrt((ys ** 2).mean(axis=1, keepdims=True))
    for i, r in enumerate(rows):
        xr = xd[r:r + 1].contiguous()
        one = hip.gemv_packed(dtype, tiles, xr, hip.group_sums(xr), N).cpu().numpy()[0]
        assert np.all(np.abs(one.astype(np.float64) - ys[i]) <= 2e-5 * scale[i]), r
    check = [0, 33, 1024, 1055, 2016, 2047, 777, rows[5]]
    x_host = xd[check].cpu().numpy()
    assert_within_operator_bound(gfo, dtype, w, x_host, y[check].cpu().numpy(), K, N, matrix_path=True)


def test_prefill_rows_at_2048_rows_against_the_oracle_on_the_last_chunk(hip, gfo):
    """2048 prompt tokens through two blocks of the 12B widths whose attention windows are 32 tokens: the
    last 32 rows depend on the last 94 only, so the oracle's forward pass of those 94 rows (empty rings)
    gives the expected rows 2016..2047 and their K/V (bars of tests/engine/gemma3_target_runtime_tests.cpp:
    310-327).  The row chunks, the run-row indexing and the ring publication at 2048 rows are all in play."""
    import torch
    from dataclasses import replace
    from guffin_amd import model
    rows, window = 2048, 32
    shape = replace(model.GEMMA3_12B, layers=2, vocab=2048, ring_global=2048, ring_local=64, sliding_window=window,
                    global_period=3)   # both blocks local
    host = model.HostModel(shape, seed=14, position=0)
    devm = model.DeviceModel.from_host(host)
    tokens = np.random.default_rng(10).integers(0, shape.vocab, rows).astype(np.uint32)
    hidden, status = devm.prefill(dev(tokens), 0)
    torch.cuda.synchronize()
    assert int(status.item()) == 0
    got = hidden.cpu().numpy().astype(np.float64)
    assert np.isfinite(got).all()
    start = rows - 1 - 3 * (window - 1)    # block 0 rows are right from start + 31 on, block 1 rows from start + 62 on
    want, wk, wv = gfo.forward(host, tokens[start:], start, threads=8)
    tail = np.arange(rows - window, rows)
    scale = np.sqrt((want[tail - start].astype(np.float64) ** 2).mean(axis=-1, keepdims=True)) + 1e-30
    assert np.max(np.abs(got[tail] - want[tail - start]) / scale) <= 1e-3
    for l in range(shape.layers):
        rk = devm.ring_k[l].view(torch.int16).cpu().numpy().view(np.uint16)
        rv = devm.ring_v[l].view(torch.int16).cpu().numpy().view(np.uint16)
        for r in tail:
            assert np.mean(rk[r & (shape.ring_local - 1)] == wk[l, r - start]) >= 0.95, (l, r)
            assert np.mean(rv[r & (shape.ring_local - 1)] == wv[l, r - start]) >= 0.95, (l, r)


def test_prefill_rows_at_2048_rows_agree_with_the_decode_path(hip, gfo):
    """The benchmark's prompt through one sliding-window block (window 1024) and one global block of the
    12B widths.  The first rows are checked against the oracle; rows sampled from every part of the run
    (chunk boundaries included) against the decode pass of the same token at the same position, which
    reads the K/V the run published: hidden rows to fp32 rounding, the row's own K/V against the ring rows."""
    import torch
    from dataclasses import replace
    from guffin_amd import model
    rows = 2048
    shape = replace(model.GEMMA3_12B, layers=2, vocab=2048, ring_global=2048, ring_local=2048, global_period=2)
    host = model.HostModel(shape, seed=15, position=0)
    devm = model.DeviceModel.from_host(host)
    tokens = np.random.default_rng(11).integers(0, shape.vocab, rows).astype(np.uint32)
    td = dev(tokens.view(np.int32))
    hidden, status = devm.prefill(td, 0)
    torch.cuda.synchronize()
    assert int(status.item()) == 0
    got = hidden.cpu().numpy().astype(np.float64)
    assert np.isfinite(got).all()
    head = 24
    want, wk, wv = gfo.forward(host, tokens[:head], 0, threads=8)
    scale = np.sqrt((want.astype(np.float64) ** 2).mean(axis=-1, keepdims=True)) + 1e-30
    assert np.max(np.abs(got[:head] - want) / scale) <= 1e-3
    sample = sorted(set([31, 32, 33, 127, 128, 1023, 1024, 1025, 1055, 1056, 2015, 2016, 2046, 2047]
                        + list(np.random.default_rng(4).integers(40, rows, 18))))
    rk = [t.view(torch.int16).cpu().numpy().view(np.uint16) for t in devm.ring_k]
    rv = [t.view(torch.int16).cpu().numpy().view(np.uint16) for t in devm.ring_v]
    for r in sample:
        one, _, pk, pv, st = devm.forward(td[r:r + 1].contiguous(), int(r))
        assert int(st.item()) == 0
        row = one.cpu().numpy().astype(np.float64)[0]
        assert np.max(np.abs(got[r] - row)) <= 2e-4 * np.sqrt((row ** 2).mean()), r
        pk = pk.view(torch.int16).cpu().numpy().view(np.uint16)
        pv = pv.view(torch.int16).cpu().numpy().view(np.uint16)
        for l in range(shape.layers):
            assert np.mean(rk[l][r] == pk[l, 0]) >= 0.95 and np.mean(rv[l][r] == pv[l, 0]) >= 0.95, (r, l)


@pytest.mark.parametrize("matrix_core", [True, False])
@pytest.mark.parametrize("q_heads,kv_heads,rows,position,window,cap", [
    (16, 8, 40, 100, 0, 256), (16, 8, 21, 300, 64, 128), (4, 1, 33, 0, 0, 64), (4, 1, 50, 17, 32, 64), (2, 2, 5, 3, 0, 16),
    (16, 8, 200, 1000, 1024, 1024), (4, 2, 130, 0, 0, 16), (2, 2, 64, 95, 48, 64)])
def test_prefill_attention_matches_double_softmax(hip, q_heads, kv_heads, rows, position, window, cap, matrix_core):
    import torch
    rng = np.random.default_rng(5)
    hd = 256
    q = rng.normal(0, 1, (rows, q_heads * hd)).astype(np.float32)
    ring_k = rng.normal(0, 1, (cap, kv_heads * hd)).astype(np.float16)
    ring_v = rng.normal(0, 1, (cap, kv_heads * hd)).astype(np.float16)
    run_k = rng.normal(0, 1, (rows, kv_heads * hd)).astype(np.float16)
    run_v = rng.normal(0, 1, (rows, kv_heads * hd)).astype(np.float16)
    out = hip.prefill_attention(dev(q), dev(ring_k), dev(ring_v), dev(run_k), dev(run_v), position, window, cap - 1,
                                q_heads, kv_heads, hd, 0.0625, matrix_core=matrix_core).cpu().numpy()
    group = q_heads // kv_heads
    want = np.zeros_like(out, dtype=np.float64)
    for r in range(rows):
        pos = position + r
        first = max(0, pos + 1 - window) if window else 0
        ks, vs = [], []
        for p in range(first, pos + 1):
            src_k, src_v, i = (run_k, run_v, p - position) if p >= position else (ring_k, ring_v, p & (cap - 1))
            ks.append(src_k[i]); vs.append(src_v[i])
        ks = np.array(ks, np.float64).reshape(len(ks), kv_heads, hd)
        vs = np.array(vs, np.float64).reshape(len(vs), kv_heads, hd)
        for h in range(q_heads):
            s = ks[:, h // group] @ q[r, h * hd:(h + 1) * hd].astype(np.float64) * 0.0625
            p = np.exp(s - s.max()); p /= p.sum()
            want[r, h * hd:(h + 1) * hd] = p @ vs[:, h // group]
    assert np.max(np.abs(out - want)) <= 2e-6 * max(1.0, np.abs(want).max())


REFERENCE_ATTENTION_CASES = (
    [(rows, 0, rows, 256, 4, 2, False, False) for rows in (8, 9, 31, 32, 33, 127, 128)]
    + [(rows, 141, 8, 32, 4, 2, False, False) for rows in (8, 9, 31, 32, 33, 127, 128)]
    + [(9, 1021, 1024, 1024, 16, 8, False, False), (33, 257, 290, 512, 16, 8, False, False),
       (9, 141, 32, 32, 16, 8, True, False), (8, 0, 8, 16, 4, 2, False, True)])


@pytest.mark.parametrize("matrix_core", [True, False])
@pytest.mark.parametrize("rows,origin,window,capacity,q_heads,kv_heads,large_scores,sensitive_query", REFERENCE_ATTENTION_CASES)
def test_prefill_attention_reference_cases(hip, rows, origin, window, capacity, q_heads, kv_heads, large_scores,
                                           sensitive_query, matrix_core):
    """tests/tensor/gemma3_metal_tests.cpp:940-1077: dyadic key / value / query patterns, NaN in every ring slot
    and beyond every row that must not be read, causal tails of 8..128 rows from an empty cache and behind an
    unaligned origin whose chunk wraps the ring, the target's head geometry, large scores, and a query whose
    information is lost if it is rounded to fp16 (row 1's two scores then cancel and the output is 0 instead of
    about 0.0016).  Bar: the reference's 4e-4 against a double softmax."""
    hd = 256
    width = kv_heads * hd
    end = origin + rows
    first = origin + 1 - window if origin + 1 > window else 0
    pos = np.arange(end)[:, None, None]
    head = np.arange(kv_heads)[None, :, None]
    col = np.arange(hd)[None, None, :]
    if sensitive_query:
        logical_k = np.where(pos == 0, 1.0, -1.0) * np.ones((1, kv_heads, hd))
        logical_v = logical_k.copy()
    else:
        logical_k = (((pos * 97 + head * 19 + col * 37) % 251) - 125) / 64.0
        logical_v = (((pos * 41 + head * 29 + col * 11) % 127) - 63) / 64.0
    logical_k = logical_k.astype(np.float32).reshape(end, width)
    logical_v = logical_v.astype(np.float32).reshape(end, width)
    r = np.arange(rows)[:, None, None]
    h = np.arange(q_heads)[None, :, None]
    if sensitive_query:
        q = np.where(col < 128, np.float32(1.0002), np.float32(-1.0)) * np.ones((rows, q_heads, 1), np.float32)
    else:
        q = ((((r * 43 + h * 23 + col * 17) % 257) - 128).astype(np.float32) * np.float32(0.500173 if large_scores else 0.0078173)
             + (h % 3).astype(np.float32) * np.float32(0.000173))
    q = q.astype(np.float32).reshape(rows, q_heads * hd)
    ring_k = np.full((capacity, width), np.nan, np.float16)
    ring_v = np.full((capacity, width), np.nan, np.float16)
    for p in range(first, origin):
        ring_k[p & (capacity - 1)], ring_v[p & (capacity - 1)] = logical_k[p], logical_v[p]
    run_k, run_v = logical_k[origin:end].astype(np.float16), logical_v[origin:end].astype(np.float16)
    out = hip.prefill_attention(dev(q), dev(ring_k), dev(ring_v), dev(run_k), dev(run_v), origin, window, capacity - 1,
                                q_heads, kv_heads, hd, 0.0625, matrix_core=matrix_core).cpu().numpy()
    group = q_heads // kv_heads
    worst = 0.0
    for row in range(rows):
        position = origin + row
        start = position + 1 - window if position + 1 > window else 0
        K = logical_k[start:position + 1].astype(np.float64).reshape(-1, kv_heads, hd)
        V = logical_v[start:position + 1].astype(np.float64).reshape(-1, kv_heads, hd)
        for hq in range(q_heads):
            scores = K[:, hq // group] @ q[row, hq * hd:(hq + 1) * hd].astype(np.float64) / 16.0
            w = np.exp(scores - scores.max())
            expected = (w / w.sum()) @ V[:, hq // group]
            worst = max(worst, float(np.abs(out[row, hq * hd:(hq + 1) * hd] - expected).max()))
    assert np.all(np.isfinite(out)) and worst <= 4e-4, worst
    if sensitive_query:
        assert abs(float(out[1, 0]) ) > 1e-3       # the retained fp32 query decides row 1


def test_publish_run_keeps_the_newest_rows(hip):
    import torch
    rows, width, cap, position = 40, 256, 16, 9
    rk = torch.arange(rows * width, dtype=torch.float32, device="cuda").reshape(rows, width).to(torch.float16)
    rv = -rk
    ring_k = torch.zeros((cap, width), dtype=torch.float16, device="cuda")
    ring_v = torch.zeros_like(ring_k)
    hip.publish_run(rk, rv, ring_k, ring_v, position, cap - 1)
    for row in range(rows - cap, rows):
        slot = (position + row) & (cap - 1)
        assert torch.equal(ring_k[slot], rk[row]) and torch.equal(ring_v[slot], rv[row])


@pytest.mark.parametrize("kind,rows,position", [("target", 37, 20), ("drafter", 70, 0)])
def test_prefill_rows_match_oracle_forward(hip, gfo, kind, rows, position):
    import torch
    from dataclasses import replace
    from guffin_amd import model
    if kind == "drafter":
        shape = replace(model.GEMMA3_270M, layers=6, vocab=4096, ring_global=256, ring_local=128, sliding_window=48)
    else:
        shape = replace(model.GEMMA3_12B, layers=6, vocab=2048, ring_global=256, ring_local=128, sliding_window=32)
    host = model.HostModel(shape, seed=4, position=position)
    devm = model.DeviceModel.from_host(host)
    tokens = np.random.default_rng(9).integers(0, shape.vocab, rows).astype(np.uint32)
    want, wk, wv = gfo.forward(host, tokens, position, threads=8)
    hidden, status = devm.prefill(dev(tokens), position)
    assert int(status.item()) == 0
    got = hidden.cpu().numpy().astype(np.float64)
    scale = np.sqrt((want.astype(np.float64) ** 2).mean(axis=-1, keepdims=True)) + 1e-30
    assert np.max(np.abs(got - want) / scale) <= 1e-3
    # the rings now hold the run: compare the last layer's published rows with the oracle's K/V
    for l in (0, shape.layers - 1):
        cap = shape.ring_local if shape.is_local(l) else shape.ring_global
        rk = devm.ring_k[l].view(torch.int16).cpu().numpy().view(np.uint16)
        for row in range(max(0, rows - cap), rows):
            g = rk[(position + row) & (cap - 1)]
            w = wk[l, row]
            assert np.mean(g == w) >= 0.95
            d = np.abs(g.view(np.float16).astype(np.float32) - w.view(np.float16).astype(np.float32))
            assert d.max() <= 2.0 ** -9 * np.abs(w.view(np.float16).astype(np.float32)).max() + 1e-6
