"""Replays the committed golden vectors (tests/golden/*.npz, written by tests/golden/make_golden.py
from the compiled reference sources) through the oracle restatement.  CPU only; needs no
reference tree, so it pins the oracle wherever the suite runs."""
import ctypes as C
import os

import numpy as np

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def test_prepare_token_distribution_golden(gfo):
    g = np.load(os.path.join(GOLD, "prepare.npz"))
    ok = 0
    for i in range(g["n"].size):
        n, hn = int(g["n"][i]), int(g["hist_n"][i])
        c = np.zeros(n, gfo.token_logit)
        c["token"], c["logit"] = g["tokens"][i, :n], g["logits"][i, :n]
        t, k, p, m, r = g["options"][i]
        rc, out = gfo.prepare(c, gfo.SamplerOptions(float(t), int(k), float(p), float(m), float(r)), g["tokens"][i, :hn])
        assert (rc == 0) == (int(g["rc"][i]) == 0), i
        if rc:
            continue
        ok += 1
        cnt = int(g["count"][i])
        assert out.count == cnt and out.total_sampling_weight == g["total"][i]
        assert np.array_equal(np.ctypeslib.as_array(out.token)[:cnt], g["out_token"][i, :cnt])
        assert np.array_equal(np.ctypeslib.as_array(out.probability)[:cnt], g["out_prob"][i, :cnt])
        assert np.array_equal(np.ctypeslib.as_array(out.sampling_weight)[:cnt], g["out_weight"][i, :cnt])
    assert ok > 100


def test_speculative_accept_golden(gfo):
    g = np.load(os.path.join(GOLD, "accept.npz"))
    opt = gfo.SamplerOptions(1.0, 64, 0.95, 0.0, 1.0)
    accepted = 0
    for i in range(g["proposal"].size):
        rows = []
        for r in range(2):
            c = np.zeros(64, gfo.token_logit)
            c["token"], c["logit"] = g["row_tokens"][i, r], g["row_logits"][i, r]
            rows.append(c)
        law = gfo.DraftLaw()
        law.count = int(g["law_count"][i])
        for j in range(law.count):
            law.ids[j] = int(g["law_ids"][i, j])
        for j in range(law.count + 1):
            law.cdf[j] = int(g["law_cdf"][i, j])
        ua, ur, un = g["draws"][i]
        rc, out = gfo.spec_accept(rows[0], rows[1], law, int(g["proposal"][i]), opt, float(ua), float(ur), float(un))
        assert rc == 0
        assert (out.accepted, out.token, out.next_root) == (int(g["accepted"][i]), int(g["token"][i]), int(g["next_root"][i])), i
        assert out.acceptance_probability == g["acceptance"][i]
        assert out.residual_total == g["residual_total"][i] and out.residual_count == int(g["residual_count"][i])
        accepted += out.accepted
    assert 0 < accepted < g["proposal"].size


def test_row_dots_and_dequant_golden(gfo):
    g = np.load(os.path.join(GOLD, "rowdot.npz"))
    for dtype, name in ((0, "q8_0"), (1, "q4_k"), (2, "q6_k")):
        for K in (256, 1024):
            w, x = g["%s_%d_w" % (name, K)], g["%s_%d_x" % (name, K)]
            dense = gfo.dequant(dtype, w)
            assert np.array_equal(dense.view(np.uint32), g["%s_%d_dense" % (name, K)].view(np.uint32))
            y = gfo.gemv(dtype, w, x, 24)
            assert np.array_equal(y.view(np.uint32), g["%s_%d_y" % (name, K)].view(np.uint32))
