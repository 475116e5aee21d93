"""GPU parity of the per-layer operators against the CPU oracle.

Tolerances follow the reference's own GPU tests: head RMS 6e-7 relative to the row scale
(tests/tensor/gemma3_metal_tests.cpp:604-612), RoPE 4 eps |theta| (|a|+|b|) + 2e-6 (:568-629),
fp16 narrowing bit-exact (:87-128), embedding 2e-6 (:511-552).
"""
import numpy as np
import pytest

from guffin_amd import synth
from test_oracle_ops import F16_CASES

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def hip():
    from guffin_amd import hip as module
    module.init(0)
    return module


def dev(a):
    import torch
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def group_sums_ref(y):
    rows, w = y.shape
    y64 = y.astype(np.float64)
    return np.concatenate([y64.reshape(rows, -1, 16).sum(-1), y64.reshape(rows, -1, 32).sum(-1)], axis=1)


@pytest.mark.parametrize("rows,width", [(1, 640), (2, 3840), (2, 15360), (3, 96)])
def test_rms_norm_and_residual(hip, gfo, rows, width):
    rng = np.random.default_rng(1)
    x = rng.normal(0, 3, (rows, width)).astype(np.float32)
    g = rng.normal(1, 0.2, width).astype(np.float32)
    res = rng.normal(0, 1, (rows, width)).astype(np.float32)
    want = gfo.rms_norm(x, g, 1e-6)
    if rows <= 2:   # receipts exist for the 1- and 2-row passes only
        y, sums = hip.rms_norm(dev(x), dev(g), want_sums=True)
    else:
        y, sums = hip.rms_norm(dev(x), dev(g)), None
    y = y.cpu().numpy()
    # against the exact operator (double) the reference's 6e-7 bound holds; the oracle's own
    # sequential fp32 sum of `width` squares carries an extra ~sqrt(width) eps
    x64 = x.astype(np.float64)
    exact = x64 / np.sqrt((x64 ** 2).mean(-1, keepdims=True) + 1e-6) * g
    assert np.max(np.abs(y - exact)) <= 6e-7 * np.abs(exact).max() + 1e-7
    tol = (6e-7 + 2.4e-7 * np.sqrt(width)) * np.abs(want).max() + 1e-7
    assert np.max(np.abs(y - want)) <= tol
    if sums is not None:
        assert np.allclose(sums.cpu().numpy(), group_sums_ref(y), rtol=0, atol=3e-5 * np.abs(y).max())
        # the matrix-core image: (hi + lo) * mult * 2^-24 restores every activation to 22 bits
        mult, image = hip.receipt_parts(sums, rows, width)
        img = image.cpu().numpy().astype(np.float64).reshape(width // 32, 4, 4, 8)
        order = [0, 2, 1, 3, 4, 6, 5, 7]
        m = mult.cpu().numpy().astype(np.float64)
        for r in range(rows):
            back = np.empty((width // 32, 4, 8))
            back[:, :, order] = img[:, 2 * r] + img[:, 2 * r + 1]
            back = back.reshape(width // 32, 32) * (m[r][:, None] / 2.0 ** 24)
            assert np.max(np.abs(back.reshape(-1) - y[r])) <= 2.0 ** -21 * np.abs(y[r]).max()
        if rows == 1:
            assert not img[:, 2:].any()
    ya = hip.rms_norm(dev(x), dev(g), residual=dev(res)).cpu().numpy()
    assert np.max(np.abs(ya - gfo.rms_norm(x, g, 1e-6, residual=res))) <= tol + 1e-6


def test_rms_norm_sums_partial_planes_in_order(hip, gfo):
    rng = np.random.default_rng(2)
    planes = rng.normal(0, 1, (5, 2, 3840)).astype(np.float32)
    g = rng.normal(1, 0.1, 3840).astype(np.float32)
    total = planes[0].copy()
    for s in range(1, 5):
        total = total + planes[s]
    want = gfo.rms_norm(total, g, 1e-6)
    y = hip.rms_norm(dev(planes), dev(g), planes=5).cpu().numpy()
    assert np.max(np.abs(y - want)) <= 2e-5 * np.abs(want).max() + 1e-7


def test_rms_norm_add_norm_joint(hip, gfo):
    rng = np.random.default_rng(3)
    x = rng.normal(0, 50, (2, 3840)).astype(np.float32)
    res = rng.normal(0, 2, (2, 3840)).astype(np.float32)
    g1 = rng.normal(1, 0.1, 3840).astype(np.float32)
    g2 = rng.normal(1, 0.1, 3840).astype(np.float32)
    want_res = gfo.rms_norm(x, g1, 1e-6, residual=res)
    want_norm = gfo.rms_norm(want_res, g2, 1e-6)
    out_res, out_norm, sums = hip.rms_norm_add_norm(dev(x), dev(g1), dev(res), dev(g2), want_sums=True)
    assert np.max(np.abs(out_res.cpu().numpy() - want_res)) <= 2e-5 * np.abs(want_res).max()
    assert np.max(np.abs(out_norm.cpu().numpy() - want_norm)) <= 4e-5 * np.abs(want_norm).max()
    assert np.allclose(sums.cpu().numpy(), group_sums_ref(out_norm.cpu().numpy()), rtol=0, atol=1e-4)


@pytest.mark.parametrize("rows,width,planes", [(2, 3840, 4), (1, 3840, 1), (2, 640, 2), (1, 8192, 3), (2, 3840, 5), (2, 96, 4)])
def test_rms_norm_add_norm_over_planes(hip, gfo, rows, width, planes):
    """Both kernels behind the entry point (registers for up to four planes, staged rows beyond) against the
    oracle on the plane sum taken in plane order; image and multipliers of the receipt rebuild the normed rows."""
    rng = np.random.default_rng(31)
    parts = rng.normal(0, 10, (planes, rows, width)).astype(np.float32)
    res = rng.normal(0, 2, (rows, width)).astype(np.float32)
    g1 = rng.normal(1, 0.1, width).astype(np.float32)
    g2 = rng.normal(1, 0.1, width).astype(np.float32)
    total = parts[0].copy()
    for s in range(1, planes):
        total = total + parts[s]
    want_res = gfo.rms_norm(total, g1, 1e-6, residual=res)
    want_norm = gfo.rms_norm(want_res, g2, 1e-6)
    status = hip.new_status()
    out_res, out_norm, sums = hip.rms_norm_add_norm(dev(parts), dev(g1), dev(res), dev(g2), planes=planes, want_sums=True,
                                                    status=status)
    y = out_norm.cpu().numpy()
    assert int(status[0]) == 0
    assert np.max(np.abs(out_res.cpu().numpy() - want_res)) <= 2e-5 * np.abs(want_res).max()
    assert np.max(np.abs(y - want_norm)) <= 4e-5 * np.abs(want_norm).max()
    assert np.allclose(sums.cpu().numpy(), group_sums_ref(y), rtol=0, atol=1e-4)
    mult, image = hip.receipt_parts(sums, rows, width)
    m, img = mult.cpu().numpy().astype(np.float64), image.cpu().numpy().astype(np.float64)
    order = [0, 2, 1, 3, 4, 6, 5, 7]
    img = img.reshape(width // 32, 4, 4, 8)
    for r in range(rows):
        back = np.empty((width // 32, 4, 8))
        back[:, :, order] = img[:, 2 * r] + img[:, 2 * r + 1]
        back = back.reshape(width // 32, 32) * (m[r][:, None] / 2.0 ** 24)
        assert np.max(np.abs(back.reshape(-1) - y[r])) <= 2.0 ** -21 * np.abs(y[r]).max()
    parts[0, rows - 1, width - 1] = np.inf
    hip.rms_norm_add_norm(dev(parts), dev(g1), dev(res), dev(g2), planes=planes, status=status)
    assert int(status[0]) == 2


def test_head_rms_norm(hip, gfo):
    rng = np.random.default_rng(4)
    x = rng.normal(0, 4, (2, 16 * 256)).astype(np.float32)
    g = rng.normal(1, 0.2, 256).astype(np.float32)
    import ctypes as C
    want = np.empty_like(x)
    gfo.lib().gfo_head_rms_norm(x.ctypes, g.ctypes, want.ctypes, 2, 16, 256, C.c_float(1e-6))
    y = hip.head_rms_norm(dev(x), dev(g), 16, 256).cpu().numpy()
    assert np.max(np.abs(y - want)) <= 6e-7 * np.abs(want).max() + 1e-7


@pytest.mark.parametrize("base,scale,start", [(1e4, 1.0, 1), (1e4, 1.0, 1024), (1e6, 0.125, 32769), (1e6, 0.125, 131071), (1e6, 1.0, 8190)])
def test_rope_by_positions(hip, gfo, base, scale, start):
    rng = np.random.default_rng(5)
    x = rng.normal(0, 1, (2, 8 * 256)).astype(np.float32)
    pos = np.array([start, start + 1], np.uint32)
    want = gfo.rope_neox(x, pos, 8, 256, 256, base, scale)
    y = hip.rope_neox(dev(x), dev(pos), 8, 256, 256, base, scale).cpu().numpy()
    theta = float(start + 1) * scale
    tol = 4 * 2.0 ** -23 * theta * 2 * np.abs(x).max() + 2e-6
    assert np.max(np.abs(y - want)) <= tol
    # the double-precision angle makes the device agree with the CPU operator far inside that bound
    assert np.max(np.abs(y - want)) <= 4e-7 * np.abs(x).max() * 2


def test_kv_store_rounding_contract_and_status(hip, gfo):
    import torch
    vals = np.array([c[0] for c in F16_CASES] * 10, np.float32)[:256].reshape(1, 256)
    bits = np.array([c[1] for c in F16_CASES] * 10, np.uint16)[:256]
    pos = dev(np.array([0], np.uint32))
    k, v = hip.kv_store_f16(dev(vals), dev(vals), pos, 1, 256, 0, 1e4)  # rope_dim 0 isolates the narrowing
    assert np.array_equal(k.view(torch.int16).cpu().numpy().view(np.uint16)[0], bits)
    assert np.array_equal(v.view(torch.int16).cpu().numpy().view(np.uint16)[0], bits)
    rng = np.random.default_rng(6)
    rk = rng.normal(0, 1, (2, 2048)).astype(np.float32)
    rv = rng.normal(0, 200, (2, 2048)).astype(np.float32)
    p2 = np.array([8190, 8191], np.uint32)
    status = hip.new_status()
    k, v = hip.kv_store_f16(dev(rk), dev(rv), dev(p2), 8, 256, 256, 1e6, 0.125, status=status)
    wk, wv = gfo.kv_store_f16(rk, rv, p2, 8, 256, 256, 1e6, 0.125)
    gk = k.view(torch.int16).cpu().numpy().view(np.uint16)
    gv = v.view(torch.int16).cpu().numpy().view(np.uint16)
    assert np.array_equal(gv, wv)
    # K: rotation agrees to ~1e-7, so at most a last-place fp16 difference on rare ties
    diff = np.abs(gk.view(np.float16).astype(np.float32) - wk.view(np.float16).astype(np.float32))
    assert np.mean(gk == wk) > 0.999 and diff.max() <= 2.0 ** -10 * np.abs(rk).max() * 2
    assert int(status.item()) == 0
    rv[1, 5] = 1e6  # overflows fp16 -> inf -> status bit 8
    hip.kv_store_f16(dev(rk), dev(rv), dev(p2), 8, 256, 256, 1e6, 0.125, status=status)
    assert int(status.item()) == 8


def test_qkv_post_fuses_headnorm_rope_and_narrowing(hip, gfo):
    import ctypes as C
    import torch
    rng = np.random.default_rng(7)
    rows, qh, kvh, hd = 2, 16, 8, 256
    planes = 3
    qp = rng.normal(0, 2, (planes, rows, qh * hd)).astype(np.float32)
    kp = rng.normal(0, 2, (planes, rows, kvh * hd)).astype(np.float32)
    vp = rng.normal(0, 30, (planes, rows, kvh * hd)).astype(np.float32)
    qn = rng.normal(1, 0.1, hd).astype(np.float32)
    kn = rng.normal(1, 0.1, hd).astype(np.float32)
    pos = np.array([777, 778], np.uint32)
    qs, ks, vs = qp[0] + qp[1] + qp[2], kp[0] + kp[1] + kp[2], vp[0] + vp[1] + vp[2]
    qh_n, kh_n = np.empty_like(qs), np.empty_like(ks)
    gfo.lib().gfo_head_rms_norm(qs.ctypes, qn.ctypes, qh_n.ctypes, rows, qh, hd, C.c_float(1e-6))
    gfo.lib().gfo_head_rms_norm(ks.ctypes, kn.ctypes, kh_n.ctypes, rows, kvh, hd, C.c_float(1e-6))
    want_q = gfo.rope_neox(qh_n, pos, qh, hd, hd, 1e4, 1.0)
    want_k, want_v = gfo.kv_store_f16(kh_n, vs, pos, kvh, hd, hd, 1e4, 1.0)
    q, k, v = hip.qkv_post(dev(qp), dev(kp), dev(vp), dev(qn), dev(kn), dev(pos), rows, qh, kvh, hd, hd, 1e4,
                           planes=planes)
    assert np.max(np.abs(q.cpu().numpy() - want_q)) <= 2e-6 * np.abs(want_q).max()
    gk = k.view(torch.int16).cpu().numpy().view(np.uint16)
    gv = v.view(torch.int16).cpu().numpy().view(np.uint16)
    assert np.array_equal(gv, want_v)
    assert np.mean(gk == want_k) > 0.995
    d = np.abs(gk.view(np.float16).astype(np.float32) - want_k.view(np.float16).astype(np.float32))
    assert d.max() <= 2.0 ** -9 * np.abs(want_q).max()
    # a precomputed angle table gives the same bits as angles formed in the kernel
    table = hip.rope_table(dev(pos), hd, 1e4, 1.0)
    q2, k2, v2 = hip.qkv_post(dev(qp), dev(kp), dev(vp), dev(qn), dev(kn), None, rows, qh, kvh, hd, hd, 1e4,
                              planes=planes, table=table)
    assert torch.equal(q2.view(torch.int32), q.view(torch.int32))
    assert torch.equal(k2.view(torch.int16), k.view(torch.int16)) and torch.equal(v2.view(torch.int16), v.view(torch.int16))
    tb = table.cpu().numpy().astype(np.float64)
    ang = pos[:, None].astype(np.float64) / 1e4 ** (2.0 * np.arange(hd // 2) / hd)
    assert np.max(np.abs(tb[..., 0] - np.cos(ang))) <= 6e-8 and np.max(np.abs(tb[..., 1] - np.sin(ang))) <= 6e-8


@pytest.mark.parametrize("rows,width", [(1, 2048), (2, 15360)])
def test_geglu(hip, gfo, rows, width):
    rng = np.random.default_rng(8)
    g = rng.normal(0, 3, (rows, width)).astype(np.float32)
    u = rng.normal(0, 2, (rows, width)).astype(np.float32)
    want = gfo.geglu(g, u)
    y, sums = hip.geglu(dev(g), dev(u), want_sums=True)
    y = y.cpu().numpy()
    assert np.all(np.abs(y - want) <= 4e-7 * np.abs(g.astype(np.float64) * u) + 1e-30)
    assert np.allclose(sums.cpu().numpy(), group_sums_ref(y), rtol=0, atol=2e-4)
    planes = np.stack([g * 0.25, g * 0.75]), np.stack([u * 0.5, u * 0.5])
    y2 = hip.geglu(dev(planes[0]), dev(planes[1]), planes=2).cpu().numpy()
    assert np.all(np.abs(y2 - want) <= 8e-7 * np.abs(g.astype(np.float64) * u) + 1e-30)


@pytest.mark.parametrize("dtype,width", [(0, 640), (2, 3840), (1, 512)])
def test_embedding(hip, gfo, dtype, width):
    vocab = 300
    w = synth.make_weight(dtype, width, vocab, seed=31)
    toks = np.array([3, 299, 0], np.uint32)
    scale = float(np.sqrt(np.float32(width)))
    want = gfo.embed(dtype, w, toks, width, scale)
    status = hip.new_status()
    y = hip.embed(dtype, dev(w), dev(toks), width, scale, vocab, status=status).cpu().numpy()
    assert np.array_equal(y.view(np.uint32), want.view(np.uint32))
    assert int(status.item()) == 0
    hip.embed(dtype, dev(w), dev(np.array([300], np.uint32)), width, scale, vocab, status=status)
    assert int(status.item()) & 1


def test_kv_scatter_publishes_selected_rows(hip):
    import torch
    rng = np.random.default_rng(9)
    cap, width = 8, 512
    ring_k = torch.zeros((cap, width), dtype=torch.float16, device="cuda")
    ring_v = torch.zeros((cap, width), dtype=torch.float16, device="cuda")
    pk = dev(rng.normal(0, 1, (3, width)).astype(np.float16))
    pv = dev(rng.normal(0, 1, (3, width)).astype(np.float16))
    sel = dev(np.array([2, 0], np.uint32))
    hip.kv_scatter(pk, pv, sel, ring_k, ring_v, 7, width, cap - 1)
    assert torch.equal(ring_k[7], pk[2]) and torch.equal(ring_k[0], pk[0])
    assert torch.equal(ring_v[7], pv[2]) and torch.equal(ring_v[0], pv[0])
    assert float(ring_k[1:7].abs().sum()) == 0.0


def test_kv_cache_copy_backs_ring_rows_up_and_restores_them(hip):
    """encode_gemma2_kv_cache_copy with both row masks (metal_command_context.hpp:170), used as the reference's
    verify pass uses it (gemma_target_runtime.cpp:473-479, gemma2_runtime.cpp:756-765): the two rows a verify
    pair will overwrite are saved from a ring that wraps, overwritten, and the rejected suffix is put back."""
    import torch
    rng = np.random.default_rng(10)
    cap, width, position = 8, 2048, 7        # rows 7 and 8 -> ring slots 7 and 0
    ring_k = dev(rng.normal(0, 1, (cap, width)).astype(np.float16))
    ring_v = dev(rng.normal(0, 1, (cap, width)).astype(np.float16))
    before_k, before_v = ring_k.clone(), ring_v.clone()
    backup_k = torch.zeros((2, width), dtype=torch.float16, device="cuda")
    backup_v = torch.zeros((2, width), dtype=torch.float16, device="cuda")
    hip.kv_cache_copy(ring_k, ring_v, backup_k, backup_v, position, 2, cap - 1, 1)
    # a backup of capacity 2 keeps row p in slot p & 1
    assert torch.equal(backup_k[1], before_k[7]) and torch.equal(backup_k[0], before_k[0])
    assert torch.equal(backup_v[1], before_v[7]) and torch.equal(backup_v[0], before_v[0])
    new_k = dev(rng.normal(0, 1, (2, width)).astype(np.float16))
    new_v = dev(rng.normal(0, 1, (2, width)).astype(np.float16))
    hip.publish_run(new_k, new_v, ring_k, ring_v, position, cap - 1)
    assert torch.equal(ring_k[7], new_k[0]) and torch.equal(ring_k[0], new_k[1])
    # the proposal was rejected: row 0 stays, the suffix (row position + 1) returns
    hip.kv_cache_copy(backup_k, backup_v, ring_k, ring_v, position + 1, 1, 1, cap - 1)
    assert torch.equal(ring_k[0], before_k[0]) and torch.equal(ring_v[0], before_v[0])
    assert torch.equal(ring_k[7], new_k[0]) and torch.equal(ring_v[7], new_v[0])
    assert torch.equal(ring_k[1:7], before_k[1:7]) and torch.equal(ring_v[1:7], before_v[1:7])
    with pytest.raises(hip.GuffinError):
        hip.kv_cache_copy(ring_k, ring_v, backup_k, backup_v, position, 3, cap - 1, 1)   # three tokens, two rows
    with pytest.raises(hip.GuffinError):
        hip.kv_cache_copy(ring_k, ring_v, backup_k, backup_v, position, 2, 5, 1)         # not a row mask


@pytest.mark.parametrize("offset_bytes", [4, 12])
def test_kv_rows_move_between_views_at_any_word_offset(hip, offset_bytes):
    """The reference's K/V caches may be views that start at any word of their allocation
    (tests/tensor/gemma3_metal_tests.cpp:765-774 uses 12 bytes): copies and publications between such views give
    the bytes the aligned calls give, and touch nothing outside the views; half a word off is refused."""
    import torch
    rng = np.random.default_rng(12)
    cap, width, position = 8, 2048, 6
    pad = offset_bytes // 2

    def view(rows, fill):
        parent = torch.full((rows * width + 16,), fill, dtype=torch.float16, device="cuda")
        return parent, parent[pad:pad + rows * width].view(rows, width)

    ring = rng.normal(0, 1, (2, cap, width)).astype(np.float16)
    run = rng.normal(0, 1, (2, 3, width)).astype(np.float16)
    pk, ring_k = view(cap, 7.0)
    pv, ring_v = view(cap, 7.0)
    ring_k.copy_(dev(ring[0])); ring_v.copy_(dev(ring[1]))
    assert ring_k.data_ptr() % 16 == offset_bytes % 16
    pbk, backup_k = view(4, 5.0)
    pbv, backup_v = view(4, 5.0)
    hip.kv_cache_copy(ring_k, ring_v, backup_k, backup_v, position, 3, cap - 1, 3)        # rows 6, 7, 8 -> slots 2, 3, 0
    _, run_k = view(3, 0.0)
    _, run_v = view(3, 0.0)
    run_k.copy_(dev(run[0])); run_v.copy_(dev(run[1]))
    hip.publish_run(run_k, run_v, ring_k, ring_v, position, cap - 1)
    # the same on aligned tensors
    a_ring_k, a_ring_v = dev(ring[0]), dev(ring[1])
    a_backup_k, a_backup_v = torch.full((4, width), 5.0, dtype=torch.float16, device="cuda"), torch.full((4, width), 5.0, dtype=torch.float16, device="cuda")
    hip.kv_cache_copy(a_ring_k, a_ring_v, a_backup_k, a_backup_v, position, 3, cap - 1, 3)
    hip.publish_run(dev(run[0]), dev(run[1]), a_ring_k, a_ring_v, position, cap - 1)
    torch.cuda.synchronize()
    assert torch.equal(ring_k, a_ring_k) and torch.equal(ring_v, a_ring_v)
    assert torch.equal(backup_k, a_backup_k) and torch.equal(backup_v, a_backup_v)
    assert torch.equal(ring_k[6], dev(run[0][0])) and torch.equal(ring_k[0], dev(run[0][2]))
    for parent, fill, rows in ((pk, 7.0, cap), (pv, 7.0, cap), (pbk, 5.0, 4), (pbv, 5.0, 4)):
        assert float((parent[:pad] - fill).abs().sum()) == 0.0 and float((parent[pad + rows * width:] - fill).abs().sum()) == 0.0
    half_word = pk[1:1 + cap * width].view(cap, width)
    with pytest.raises(hip.GuffinError):
        hip.kv_cache_copy(half_word, ring_v, backup_k, backup_v, position, 2, cap - 1, 3)
    with pytest.raises(hip.GuffinError):
        hip.publish_run(run_k, run_v, half_word, ring_v, position, cap - 1)
