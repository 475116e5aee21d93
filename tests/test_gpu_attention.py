"""GPU parity of the GQA decode/verify attention against the CPU oracle and closed forms.

The reference checks its kernel against a double-precision softmax at 2e-7 on a
tree + wrapped-ring case (tests/tensor/gemma3_metal_tests.cpp:746-833); the oracle here
follows the CPU operators (fp32 dots, double exp), so the bar is a few fp32 ulps of the
value scale.
"""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def hip():
    from guffin_amd import hip as module
    module.init(0)
    return module


def dev(a):
    import torch
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def contiguous_schedule(position, rows, window):
    sched = []
    for row in range(rows):
        p = position + row
        ws = p + 1 - window if (window and p >= window) else 0
        base_start = min(position, ws)
        private_start = max(ws - position, 0) if ws > position else 0
        sched.append([base_start, position - base_start, private_start, row + 1 - private_start])
    return np.array(sched, np.uint32)


def run_case(hip, gfo, rows, q_heads, kv_heads, cap, position, window, seed, sigma_v=1.0):
    hd = 256
    rng = np.random.default_rng(seed)
    ring_k = rng.normal(0, 1, (cap, kv_heads * hd)).astype(np.float16)
    ring_v = rng.normal(0, sigma_v, (cap, kv_heads * hd)).astype(np.float16)
    pk = rng.normal(0, 1, (rows, kv_heads * hd)).astype(np.float16)
    pv = rng.normal(0, sigma_v, (rows, kv_heads * hd)).astype(np.float16)
    q = rng.normal(0, 1, (rows, q_heads * hd)).astype(np.float32)
    sched = contiguous_schedule(position, rows, window)
    anc = np.arange(rows, dtype=np.uint32)
    want = gfo.attention(q, ring_k.view(np.uint16), ring_v.view(np.uint16), pk.view(np.uint16),
                         pv.view(np.uint16), sched, anc, cap - 1, q_heads, kv_heads, hd, 0.0625)
    union = int(max(s[0] + s[1] for s in sched) - min(s[0] for s in sched if s[1]) if any(s[1] for s in sched) else 0)
    out, sums = hip.attention_decode(dev(q), dev(ring_k), dev(ring_v), dev(pk), dev(pv), dev(sched), dev(anc),
                                     union + rows, cap - 1, q_heads, kv_heads, hd, 0.0625, want_sums=True)
    out = out.cpu().numpy()
    err = np.max(np.abs(out - want))
    assert err <= 3e-6 * sigma_v * 4, err
    o64 = out.astype(np.float64)
    ref_sums = np.concatenate([o64.reshape(rows, -1, 16).sum(-1), o64.reshape(rows, -1, 32).sum(-1)], axis=1)
    assert np.allclose(sums.cpu().numpy(), ref_sums, rtol=0, atol=1e-4 * sigma_v)
    return out


@pytest.mark.parametrize("rows,q_heads,kv_heads,cap,position,window", [
    (2, 16, 8, 1024, 8190, 1024),   # target local layer: wrapped ring, window drops the oldest token for row 1
    (2, 16, 8, 8192, 8190, 0),      # target global layer
    (1, 16, 8, 1024, 500, 1024),    # single row, ring not yet wrapped
    (1, 4, 1, 512, 4096, 512),      # drafter local
    (1, 4, 1, 8192, 4096, 0),       # drafter global
    (2, 4, 2, 64, 5, 0),            # tiny: one partition, mostly masked
    (2, 2, 2, 64, 0, 0),            # empty prefix: only the private rows
])
def test_attention_matches_oracle(hip, gfo, rows, q_heads, kv_heads, cap, position, window):
    run_case(hip, gfo, rows, q_heads, kv_heads, cap, position, window, seed=rows * 100 + q_heads)


def test_attention_large_values_keep_relative_accuracy(hip, gfo):
    run_case(hip, gfo, 2, 16, 8, 1024, 3000, 1024, seed=77, sigma_v=200.0)


def test_attention_closed_forms(hip):
    import torch
    hd, cap, q_heads, kv_heads = 256, 64, 4, 2
    rng = np.random.default_rng(3)
    q = rng.normal(0, 1, (1, q_heads * hd)).astype(np.float32)
    ring_k = np.ones((cap, kv_heads * hd), np.float16)            # uniform keys -> uniform weights
    ring_v = rng.normal(0, 1, (cap, kv_heads * hd)).astype(np.float16)
    pk = np.ones((1, kv_heads * hd), np.float16)
    pv = rng.normal(0, 1, (1, kv_heads * hd)).astype(np.float16)
    sched = np.array([[60, 9, 0, 1]], np.uint32)                   # ring slots 60..63, 0..4 then self
    out = hip.attention_decode(dev(q), dev(ring_k), dev(ring_v), dev(pk), dev(pv), dev(sched),
                               dev(np.array([0], np.uint32)), 10, cap - 1, q_heads, kv_heads, hd, 0.0625).cpu().numpy()
    slots = [(60 + t) & 63 for t in range(9)]
    mean = np.concatenate([ring_v[slots], pv]).astype(np.float64).mean(0).reshape(kv_heads, hd)
    want = np.repeat(mean, 2, axis=0).reshape(1, -1)
    assert np.max(np.abs(out - want)) < 1e-6
    # a single attended token returns its value row exactly
    sched1 = np.array([[0, 0, 0, 1]], np.uint32)
    out1 = hip.attention_decode(dev(q), dev(ring_k), dev(ring_v), dev(pk), dev(pv), dev(sched1),
                                dev(np.array([0], np.uint32)), 1, cap - 1, q_heads, kv_heads, hd, 0.0625).cpu().numpy()
    want1 = np.repeat(pv.astype(np.float32).reshape(kv_heads, hd), 2, axis=0).reshape(1, -1)
    assert np.array_equal(out1, want1)


def test_attention_extreme_finite_scores(hip):
    """tests/tensor/gemma3_metal_tests.cpp:882-936: scores of exactly +-1024 and +-2048 against fp16 values of
    +-65504.  A stable fp32 softmax discards the losing exponentials, maxima of different partitions stay finite,
    and every output element is exact: the winning private row's 65504 / -65504, or the plain mean of 256 equal
    value rows."""
    rows, heads, kv_heads, width, capacity = 2, 16, 8, 256, 512
    q = np.zeros((rows, heads, width), np.float32)
    q[:, 0::2, 0], q[:, 1::2, 0] = 1024.0, -1024.0
    pk = np.zeros((rows, kv_heads, width), np.float16)
    pk[0, :, 0], pk[1, :, 0] = 32.0, -32.0
    pv = np.zeros((rows, kv_heads, width), np.float16)
    pv[0], pv[1] = 65504.0, -65504.0
    k = np.zeros((capacity, kv_heads, width), np.float16)
    k[0::2, :, 0], k[1::2, :, 0] = 16.0, -16.0
    v = np.zeros((capacity, kv_heads, width), np.float16)
    v[:] = (np.arange(kv_heads, dtype=np.float32)[:, None] + np.arange(width, dtype=np.float32)[None, :] * 0.25)[None]
    sched = np.array([[0, capacity, 0, 1], [0, capacity, 1, 2]], np.uint32)
    ancestors = np.array([0, 0, 1], np.uint32)
    flat = lambda a: dev(a.reshape(a.shape[0], -1))
    for want_sums in (False, True):
        got = hip.attention_decode(flat(q), flat(k), flat(v), flat(pk), flat(pv), dev(sched), dev(ancestors), capacity + rows,
                                   capacity - 1, heads, kv_heads, width, 1.0 / 16.0, want_sums=want_sums)
        out = (got[0] if want_sums else got).cpu().numpy().reshape(rows, heads, width)
        for row in range(rows):
            for head in range(heads):
                if head % 2 == 0:
                    expected = np.full(width, 65504.0, np.float32)
                elif row == 1:
                    expected = np.full(width, -65504.0, np.float32)
                else:
                    expected = (head // 2 + np.arange(width) * 0.25).astype(np.float32)
                assert np.array_equal(out[row, head], expected), (row, head, out[row, head][:4], expected[:4])


def test_attention_rejects_bad_shapes(hip):
    import torch
    z = torch.zeros(4096, dtype=torch.float32, device="cuda")
    h = torch.zeros((4, 512), dtype=torch.float16, device="cuda")
    s = torch.zeros(8, dtype=torch.int32, device="cuda")
    with pytest.raises(hip.GuffinError):   # head_dim 128 unsupported
        hip.attention_decode(z[:256].view(1, 256), h, h, h[:1], h[:1], s, s, 4, 3, 2, 2, 128, 0.1)
    with pytest.raises(hip.GuffinError):   # ring capacity not a power of two
        hip.attention_decode(z[:1024].view(1, 1024), h, h, h[:1], h[:1], s, s, 4, 2, 4, 2, 256, 0.1)


@pytest.mark.parametrize("rows,q_heads,kv_heads,cap,position,window,planes", [
    (2, 16, 8, 1024, 8190, 1024, 2),   # target local block: private rows straddle the last partition
    (2, 16, 8, 8192, 8190, 0, 2),      # target global block
    (1, 4, 1, 512, 4096, 512, 4),      # drafter local block
    (1, 4, 1, 8192, 4095, 0, 1),       # drafter global block, a single plane
    (2, 4, 2, 64, 31, 0, 3),           # private rows fall into two different partitions
    (2, 2, 2, 64, 0, 0, 1),            # empty prefix
])
def test_attention_from_projection_planes_equals_the_separate_passes(hip, rows, q_heads, kv_heads, cap, position,
                                                                     window, planes):
    """One launch that prepares q, k, v itself gives bit for bit what qkv_post + attention give."""
    import torch
    hd = 256
    rng = np.random.default_rng(position * 7 + rows)
    ring_k = dev(rng.normal(0, 1, (cap, kv_heads * hd)).astype(np.float16))
    ring_v = dev(rng.normal(0, 1, (cap, kv_heads * hd)).astype(np.float16))
    q_raw = dev(rng.normal(0, 1, (planes, rows, q_heads * hd)).astype(np.float32))
    k_raw = dev(rng.normal(0, 1, (planes, rows, kv_heads * hd)).astype(np.float32))
    v_raw = dev(rng.normal(0, 1, (planes, rows, kv_heads * hd)).astype(np.float32))
    q_norm = dev(rng.normal(1, 0.1, hd).astype(np.float32))
    k_norm = dev(rng.normal(1, 0.1, hd).astype(np.float32))
    positions = dev(np.arange(position, position + rows, dtype=np.uint32))
    table = hip.rope_table(positions, hd, 10000.0)
    sched = contiguous_schedule(position, rows, window)
    anc = dev(np.arange(rows, dtype=np.uint32))
    union = int(max(s[0] + s[1] for s in sched) - min(s[0] for s in sched if s[1]) if any(s[1] for s in sched) else 0)
    status = torch.zeros(1, dtype=torch.int32, device="cuda")
    q, pk, pv = hip.qkv_post(q_raw, k_raw, v_raw, q_norm, k_norm, positions, rows, q_heads, kv_heads, hd, hd, 10000.0,
                             planes=planes, table=table)
    want, want_sums = hip.attention_decode(q, ring_k, ring_v, pk, pv, dev(sched), anc, union + rows, cap - 1,
                                           q_heads, kv_heads, hd, 0.0625, want_sums=True)
    got, got_sums, gk, gv = hip.qkv_attention(q_raw, k_raw, v_raw, q_norm, k_norm, table, ring_k, ring_v, dev(sched),
                                              anc, union + rows, cap - 1, q_heads, kv_heads, hd, 0.0625, status=status)
    torch.cuda.synchronize()
    assert int(status[0]) == 0
    assert torch.equal(gk.view(torch.int16), pk.view(torch.int16)) and torch.equal(gv.view(torch.int16), pv.view(torch.int16))
    assert torch.equal(got.view(torch.int32), want.view(torch.int32))
    assert torch.equal(got_sums.view(torch.int32), want_sums.view(torch.int32))


@pytest.mark.parametrize("offset_bytes", [4, 12])
def test_kv_views_at_any_word_offset(hip, offset_bytes):
    """K/V buffers may be views that start at any 4-byte offset of their allocation (the reference's case uses a
    12-byte one, tests/tensor/gemma3_metal_tests.cpp:765-774): the same bits as from 16-byte aligned rows, through
    the separate pass and through the pass that prepares q/k/v itself."""
    import torch
    rows, q_heads, kv_heads, hd, cap, position = 2, 16, 8, 256, 2048, 1500
    rng = np.random.default_rng(77)
    ring_k = rng.normal(0, 1, (cap, kv_heads * hd)).astype(np.float16)
    ring_v = rng.normal(0, 1, (cap, kv_heads * hd)).astype(np.float16)
    pk = rng.normal(0, 1, (rows, kv_heads * hd)).astype(np.float16)
    pv = rng.normal(0, 1, (rows, kv_heads * hd)).astype(np.float16)
    q = dev(rng.normal(0, 1, (rows, q_heads * hd)).astype(np.float32))
    sched = dev(contiguous_schedule(position, rows, 1024))
    anc = dev(np.arange(rows, dtype=np.uint32))

    def shifted(a):
        pad = offset_bytes // 2
        parent = torch.zeros(a.size + pad + 8, dtype=torch.float16, device="cuda")
        view = parent[pad:pad + a.size].view(a.shape)
        view.copy_(dev(a))
        assert view.data_ptr() % 16 == offset_bytes % 16
        return view

    args = (1023 + rows, cap - 1, q_heads, kv_heads, hd, 0.0625)
    want = hip.attention_decode(q, dev(ring_k), dev(ring_v), dev(pk), dev(pv), sched, anc, *args)
    got = hip.attention_decode(q, shifted(ring_k), shifted(ring_v), shifted(pk), shifted(pv), sched, anc, *args)
    torch.cuda.synchronize()
    assert torch.equal(got, want)
