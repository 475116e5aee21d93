"""Pins the oracle's small operators (CPU only): compiled reference where it links,
closed forms and library routines elsewhere."""
import ctypes as C

import numpy as np
import pytest

# the reference's binary16 round-to-nearest-even contract,
# tests/tensor/gemma3_metal_tests.cpp:93-109 (inputs and expected bits, data only)
F16_CASES = [
    (0.0, 0x0000), (-0.0, 0x8000), (1.0, 0x3C00), (-1.0, 0xBC00),
    (1.0 + 2.0 ** -11, 0x3C00), (-1.0 - 2.0 ** -11, 0xBC00),
    (1.0 + 1.5 * 2.0 ** -10, 0x3C02), (-1.0 - 1.5 * 2.0 ** -10, 0xBC02),
    (float(np.nextafter(np.float32(1.0 + 2.0 ** -11), np.float32(0.0))), 0x3C00),
    (float(np.nextafter(np.float32(1.0 + 2.0 ** -11), np.float32(2.0))), 0x3C01),
    (2.0 ** -24, 0x0001), (-2.0 ** -24, 0x8001), (2.0 ** -25, 0x0000), (-2.0 ** -25, 0x8000),
    (1.5 * 2.0 ** -24, 0x0002), (-1.5 * 2.0 ** -24, 0x8002),
    (2.0 ** -14 - 2.0 ** -24, 0x03FF), (2.0 ** -14 - 2.0 ** -25, 0x0400),
    (2.0 ** -14, 0x0400), (-2.0 ** -14, 0x8400),
    (65504.0, 0x7BFF), (-65504.0, 0xFBFF), (65519.0, 0x7BFF), (-65519.0, 0xFBFF),
    (65520.0, 0x7C00), (-65520.0, 0xFC00), (65536.0, 0x7C00), (-65536.0, 0xFC00),
]


def test_f16_rne_reference_bit_cases(gfo):
    assert len(F16_CASES) == 28
    for value, bits in F16_CASES:
        assert gfo.lib().gfo_f32_to_f16_rne(C.c_float(value)) == bits, (value, hex(bits))


def test_f16_rne_matches_numpy_on_random_and_edge_values(gfo):
    rng = np.random.default_rng(0)
    vals = np.concatenate([
        rng.normal(0, 1, 4000), rng.normal(0, 1e-5, 2000), rng.normal(0, 3e4, 2000),
        rng.uniform(-7e-8, 7e-8, 2000), [np.inf, -np.inf, 70000.0, 1e-8],
    ]).astype(np.float32)
    with np.errstate(over="ignore"):
        want = vals.astype(np.float16).view(np.uint16)
    got = np.array([gfo.lib().gfo_f32_to_f16_rne(C.c_float(float(v))) for v in vals], np.uint16)
    assert np.array_equal(got, want)


def test_rms_norm_matches_compiled_reference(gfo, ref):
    if ref is None:
        pytest.skip("oracle/_ref not built")
    rng = np.random.default_rng(1)
    x = rng.normal(0, 3, (3, 640)).astype(np.float32)
    g = rng.normal(1, 0.2, 640).astype(np.float32)
    y = gfo.rms_norm(x, g, 1e-6)
    r = np.empty_like(x)
    assert ref.gfr_rms_norm(x.ctypes, g.ctypes, r.ctypes, 3, 640, C.c_float(1e-6)) == 0
    assert np.array_equal(y.view(np.uint32), r.view(np.uint32))
    # head norm = the same operator over rows*heads rows of head_dim
    yh = np.empty_like(x)
    gh = g[:128].copy()
    gfo.lib().gfo_head_rms_norm(x.ctypes, gh.ctypes, yh.ctypes, 3, 5, 128, C.c_float(1e-6))
    rh = np.empty_like(x)
    ref.gfr_rms_norm(x.ctypes, gh.ctypes, rh.ctypes, 15, 128, C.c_float(1e-6))
    assert np.array_equal(yh.view(np.uint32), rh.view(np.uint32))


def test_rms_norm_against_double_and_residual_add(gfo):
    rng = np.random.default_rng(2)
    x = rng.normal(0, 2, (2, 3840)).astype(np.float32)
    g = rng.normal(1, 0.1, 3840).astype(np.float32)
    res = rng.normal(0, 1, (2, 3840)).astype(np.float32)
    x64 = x.astype(np.float64)
    want = x64 / np.sqrt((x64 ** 2).mean(-1, keepdims=True) + 1e-6) * g
    y = gfo.rms_norm(x, g, 1e-6)
    assert np.max(np.abs(y - want)) < 6e-7 * np.max(np.abs(want)) + 1e-6
    ya = gfo.rms_norm(x, g, 1e-6, residual=res)
    assert np.array_equal(ya, y + res)


def test_rope_matches_compiled_reference_and_closed_form(gfo, ref):
    rng = np.random.default_rng(3)
    heads, hd = 4, 256
    x = rng.normal(0, 1, (3, heads * hd)).astype(np.float32)
    for base, start in ((1e4, 0), (1e4, 1024), (1e6, 32769), (1e6, 131071)):
        pos = np.arange(start, start + 3, dtype=np.uint32)
        y = gfo.rope_neox(x, pos, heads, hd, hd, base, 1.0)
        if ref is not None:
            r = np.empty_like(x)
            assert ref.gfr_rope_neox(x.ctypes, r.ctypes, C.c_uint64(start), 3, heads, hd, hd,
                                     C.c_float(base)) == 0
            assert np.array_equal(y.view(np.uint32), r.view(np.uint32))
        # closed form in double, pair (i, i+128), theta = pos / base^(2i/256)
        xr = x.reshape(3, heads, hd).astype(np.float64)
        i = np.arange(hd // 2)
        theta = pos[:, None].astype(np.float64) / np.float64(np.float32(base)) ** (2.0 * i / hd)
        c, s = np.cos(theta)[:, None, :], np.sin(theta)[:, None, :]
        a, b = xr[..., :hd // 2], xr[..., hd // 2:]
        want = np.concatenate([a * c - b * s, a * s + b * c], -1).reshape(3, -1)
        tol = 4 * 2.0 ** -23 * (np.abs(a) + np.abs(b)).max() + 2e-6
        assert np.max(np.abs(y - want)) < tol


def test_rope_frequency_scale_is_a_position_scale(gfo):
    rng = np.random.default_rng(4)
    x = rng.normal(0, 1, (1, 256)).astype(np.float32)
    y8 = gfo.rope_neox(x, [4096], 1, 256, 256, 1e6, 0.125)
    y1 = gfo.rope_neox(x, [512], 1, 256, 256, 1e6, 1.0)
    assert np.allclose(y8, y1, atol=1e-6)


def test_kv_store_rotates_then_narrows(gfo):
    rng = np.random.default_rng(5)
    k = rng.normal(0, 1, (2, 512)).astype(np.float32)
    v = rng.normal(0, 100, (2, 512)).astype(np.float32)
    pos = np.array([7, 8], np.uint32)
    hk, hv = gfo.kv_store_f16(k, v, pos, 2, 256, 256, 1e4, 1.0)
    rot = gfo.rope_neox(k, pos, 2, 256, 256, 1e4, 1.0)
    assert np.array_equal(hk, rot.astype(np.float16).view(np.uint16))
    assert np.array_equal(hv, v.astype(np.float16).view(np.uint16))
    # rope_dim 0 isolates the narrowing (the reference's rounding test does this)
    hk0, _ = gfo.kv_store_f16(k, v, pos, 2, 256, 0, 1e4, 1.0)
    assert np.array_equal(hk0, k.astype(np.float16).view(np.uint16))


def test_geglu_matches_compiled_reference(gfo, ref):
    rng = np.random.default_rng(6)
    g = np.concatenate([rng.normal(0, 3, 5000), [0.0, -0.0, 20.0, -20.0, 1e-20]]).astype(np.float32)
    u = rng.normal(0, 2, g.size).astype(np.float32)
    y = gfo.geglu(g, u)
    if ref is not None:
        r = np.empty_like(g)
        assert ref.gfr_gelu_mul(g.ctypes, u.ctypes, r.ctypes, C.c_uint64(g.size)) == 0
        assert np.array_equal(y.view(np.uint32), r.view(np.uint32))
    g64 = g.astype(np.float64)
    want = 0.5 * g64 * (1 + np.tanh(0.7978845608028654 * (g64 + 0.044715 * g64 ** 3))) * u
    # 1 + tanh cancels for negative gates: the fp32 error scales with |g*u|, not with |result|
    assert np.all(np.abs(y - want) <= 3e-7 * np.abs(g64 * u) + 1e-30)


def _ring_case(rng, tokens, kv_heads, hd, cap):
    k = rng.normal(0, 1, (cap, kv_heads * hd)).astype(np.float16)
    v = rng.normal(0, 1, (cap, kv_heads * hd)).astype(np.float16)
    return k, v


def test_attention_matches_compiled_reference_composition(gfo, ref):
    if ref is None:
        pytest.skip("oracle/_ref not built")
    rng = np.random.default_rng(7)
    q_heads, kv_heads, hd = 4, 2, 64
    position, rows, window = 37, 2, 16
    total = position + rows
    kf = rng.normal(0, 1, (total, kv_heads * hd)).astype(np.float16)
    vf = rng.normal(0, 1, (total, kv_heads * hd)).astype(np.float16)
    q = rng.normal(0, 1, (rows, q_heads * hd)).astype(np.float32)
    # reference: contiguous fp32 K/V rows, causal, last `window` positions
    r = np.empty_like(q)
    k32, v32 = kf.astype(np.float32), vf.astype(np.float32)
    assert ref.gfr_attention(q.ctypes, k32.ctypes, v32.ctypes, r.ctypes, C.c_uint64(position), rows,
                             total, q_heads, kv_heads, hd, window, C.c_float(0.125),
                             C.c_float(2.0 ** 100)) == 0
    # oracle: ring (capacity 64 > position) for the prefix, private rows for the new ones
    cap = 64
    ring_k = np.zeros((cap, kv_heads * hd), np.float16)
    ring_v = np.zeros((cap, kv_heads * hd), np.float16)
    ring_k[:position], ring_v[:position] = kf[:position], vf[:position]
    sched = []
    for row in range(rows):
        p = position + row
        ws = p + 1 - window
        base_start = min(position, ws)
        private_start = max(ws - position, 0)
        sched.append([base_start, position - base_start, private_start, row + 1 - private_start])
    out = gfo.attention(q, ring_k.view(np.uint16), ring_v.view(np.uint16),
                        kf[position:].copy().view(np.uint16), vf[position:].copy().view(np.uint16),
                        np.array(sched, np.uint32), np.arange(rows, dtype=np.uint32), cap - 1,
                        q_heads, kv_heads, hd, 0.125)
    assert np.array_equal(out.view(np.uint32), r.view(np.uint32))


def test_attention_closed_forms_and_wrapped_ring(gfo):
    rng = np.random.default_rng(8)
    q_heads, kv_heads, hd, cap = 4, 2, 32, 8
    q = rng.normal(0, 1, (1, q_heads * hd)).astype(np.float32)
    # uniform K => output = mean of V over the attended tokens (ring wraps: slots 6,7,0,1,2)
    ring_k = np.ones((cap, kv_heads * hd), np.float16)
    ring_v = rng.normal(0, 1, (cap, kv_heads * hd)).astype(np.float16)
    pk = np.ones((1, kv_heads * hd), np.float16)
    pv = rng.normal(0, 1, (1, kv_heads * hd)).astype(np.float16)
    sched = np.array([[14, 5, 0, 1]], np.uint32)
    out = gfo.attention(q, ring_k.view(np.uint16), ring_v.view(np.uint16), pk.view(np.uint16),
                        pv.view(np.uint16), sched, np.array([0], np.uint32), cap - 1, q_heads,
                        kv_heads, hd, 0.25)
    slots = [(14 + t) & 7 for t in range(5)]
    vals = np.concatenate([ring_v[slots], pv]).astype(np.float64).mean(0).reshape(kv_heads, hd)
    want = np.repeat(vals, q_heads // kv_heads, axis=0).reshape(1, -1)
    assert np.max(np.abs(out - want)) < 5e-7
    # a single attended token => output = its V exactly
    sched1 = np.array([[0, 0, 0, 1]], np.uint32)
    out1 = gfo.attention(q, ring_k.view(np.uint16), ring_v.view(np.uint16), pk.view(np.uint16),
                         pv.view(np.uint16), sched1, np.array([0], np.uint32), cap - 1, q_heads,
                         kv_heads, hd, 0.25)
    want1 = np.repeat(pv.astype(np.float32).reshape(kv_heads, hd), 2, axis=0).reshape(1, -1)
    assert np.array_equal(out1, want1)


def test_argmax_and_selection_order(gfo, ref):
    # tests/tensor/gemma3_metal_tests.cpp:1112-1142: ties prefer the lower id; history appended
    logits = np.full(1025, -2.0, np.float32)
    logits[1000] = logits[1001] = 101.0
    logits[1010] = 100.0
    logits[7] = -99.75
    c = gfo.select_candidates(logits, 3, history=[7])
    assert list(c["token"]) == [1000, 1001, 1010, 7]
    assert list(c["logit"]) == [101.0, 101.0, 100.0, -99.75]
    assert gfo.lib().gfo_argmax(logits.ctypes, 1025) == 1000
    if ref is not None:
        assert ref.gfr_argmax(logits.ctypes, 1025) == 1000
    rng = np.random.default_rng(9)
    big = rng.normal(0, 2, 50000).astype(np.float32)
    big[rng.integers(0, 50000, 500)] = big[17]  # force ties
    c = gfo.select_candidates(big, 64)
    order = np.lexsort((np.arange(big.size), -big.astype(np.float64)))[:64]
    assert np.array_equal(c["token"], order.astype(np.uint32))
    assert gfo.lib().gfo_argmax(big.ctypes, big.size) == order[0]
    with pytest.raises(ValueError):
        bad = big.copy()
        bad[3] = np.inf
        gfo.select_candidates(bad, 4)


def test_embedding_is_scaled_dequantised_row(gfo):
    from guffin_amd import synth
    for dtype, width in ((0, 640), (2, 768)):
        w = synth.make_weight(dtype, width, 10, seed=31)
        dense = gfo.dequant(dtype, w).reshape(10, width)
        scale = np.sqrt(np.float32(width))
        out = gfo.embed(dtype, w, [3, 9], width, scale)
        assert np.array_equal(out, dense[[3, 9]] * scale)
