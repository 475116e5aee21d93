#!/usr/bin/env python3
"""Writes golden vectors from the compiled reference (oracle/_ref, built by oracle/Makefile from
the reference's own sampling.cpp / quantization.cpp) for the functions only a compile can pin:

  prepare.npz   prepare_token_distribution (src/engine/sampling.cpp:394-499) on random
                candidate lists: tokens, probabilities and sampling weights bit for bit
  accept.npz    prepare_speculative_distribution + sample_speculative_token
                (sampling.cpp:561-656) on seeded target rows, proposal laws and injected draws
  rowdot.npz    dot_q4_k_row_f32 / dot_q6_k_row_f32 (src/tensor/quantization.cpp:706-713,
                826-833) and the Q8_0 row sum on seeded blocks, K = 256..1024

Run here (needs /root/reference):  python tests/golden/make_golden.py
The vectors are inputs and expected outputs only; tests/test_golden.py replays them through the
oracle restatement, so the CPU suite pins it where the reference tree is absent.
"""
import ctypes as C
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from guffin_amd import synth  # noqa: E402
from oracle import gfo  # noqa: E402


def main():
    gfo.build()
    ref = gfo.ref()
    if ref is None:
        raise SystemExit("oracle/_ref is not built (needs /root/reference)")
    rng = np.random.default_rng(2024)

    # ---- prepare_token_distribution ------------------------------------------------------
    cases = 160
    P = dict(n=np.zeros(cases, np.uint32), tokens=np.zeros((cases, 130), np.uint32),
             logits=np.zeros((cases, 130), np.float32), options=np.zeros((cases, 5), np.float64),
             hist_n=np.zeros(cases, np.uint32), rc=np.zeros(cases, np.int32), count=np.zeros(cases, np.uint32),
             total=np.zeros(cases, np.float64), out_token=np.zeros((cases, 256), np.uint32),
             out_prob=np.zeros((cases, 256), np.float64), out_weight=np.zeros((cases, 256), np.float64))
    for i in range(cases):
        n = int(rng.integers(64, 130))
        toks = rng.choice(262144, n, replace=False).astype(np.uint32)
        logit = rng.normal(0, rng.choice([0.5, 2.0, 6.0]), n).astype(np.float32)
        if i % 7 == 0:
            logit[: n // 2] = logit[0]  # ties
        opt = (float(rng.choice([0.0, 0.7, 1.0, 1.3])), int(rng.choice([1, 40, 64])),
               float(rng.choice([0.5, 0.9, 0.95, 1.0])), float(rng.choice([0.0, 0.05])),
               float(rng.choice([1.0, 1.1])))
        hn = int(rng.integers(0, 5))
        c = np.zeros(n, gfo.token_logit)
        c["token"], c["logit"] = toks, logit
        rc, out = gfo.prepare(c, gfo.SamplerOptions(*opt), toks[:hn], which=ref)
        P["n"][i], P["hist_n"][i], P["rc"][i] = n, hn, rc
        P["tokens"][i, :n], P["logits"][i, :n], P["options"][i] = toks, logit, opt
        if rc == 0:
            P["count"][i], P["total"][i] = out.count, out.total_sampling_weight
            P["out_token"][i] = np.ctypeslib.as_array(out.token)
            P["out_prob"][i] = np.ctypeslib.as_array(out.probability)
            P["out_weight"][i] = np.ctypeslib.as_array(out.sampling_weight)
    np.savez_compressed(os.path.join(HERE, "prepare.npz"), **P)

    # ---- accept / residual -----------------------------------------------------------------
    cases, vocab = 200, 2048
    A = dict(row_tokens=np.zeros((cases, 2, 64), np.uint32), row_logits=np.zeros((cases, 2, 64), np.float32), law_count=np.zeros(cases, np.uint32),
             law_ids=np.zeros((cases, 256), np.uint32), law_cdf=np.zeros((cases, 257), np.uint64),
             proposal=np.zeros(cases, np.uint32), draws=np.zeros((cases, 3), np.float64),
             accepted=np.zeros(cases, np.uint32), token=np.zeros(cases, np.uint32),
             next_root=np.zeros(cases, np.uint32), acceptance=np.zeros(cases, np.float64),
             residual_total=np.zeros(cases, np.float64), residual_count=np.zeros(cases, np.uint32))
    opt = gfo.SamplerOptions(1.0, 64, 0.95, 0.0, 1.0)
    for i in range(cases):
        p = rng.normal(0, 3, (2, vocab)).astype(np.float32)
        # the proposal law is an input here: random integer masses over a random support inside p's top tokens
        top = np.argsort(-p[0])[:80]
        support = np.sort(rng.choice(top, int(rng.integers(1, 60)), replace=False)).astype(np.uint32)
        cuts = np.sort(rng.choice(np.arange(1, 1 << 32, dtype=np.uint64), support.size - 1, replace=False)) \
            if support.size > 1 else np.zeros(0, np.uint64)
        cdf = np.concatenate([[0], cuts, [1 << 32]]).astype(np.uint64)
        law = gfo.DraftLaw()
        law.count = support.size
        for j, t in enumerate(support):
            law.ids[j] = int(t)
        for j, e in enumerate(cdf):
            law.cdf[j] = int(e)
        word, ua, ur, un = gfo.step_draws(77, i)
        masses = np.diff(cdf).astype(np.uint64)
        st = C.c_int(0)
        ref.gfr_select_draft_token.restype = C.c_uint32
        proposal = ref.gfr_select_draft_token(support.ctypes, masses.ctypes, C.c_uint32(support.size),
                                              C.c_uint32(word), C.byref(st))
        assert st.value == 0
        r0 = gfo.select_candidates(p[0], 64)
        r1 = gfo.select_candidates(p[1], 64)
        rc, out = gfo.spec_accept(r0, r1, law, proposal, opt, ua, ur, un, which=ref)
        assert rc == 0
        A["row_tokens"][i, 0], A["row_logits"][i, 0] = r0["token"], r0["logit"]
        A["row_tokens"][i, 1], A["row_logits"][i, 1] = r1["token"], r1["logit"]
        A["law_count"][i] = support.size
        A["law_ids"][i, :support.size], A["law_cdf"][i, :cdf.size] = support, cdf
        A["proposal"][i], A["draws"][i] = proposal, (ua, ur, un)
        A["accepted"][i], A["token"][i], A["next_root"][i] = out.accepted, out.token, out.next_root
        A["acceptance"][i], A["residual_total"][i] = out.acceptance_probability, out.residual_total
        A["residual_count"][i] = out.residual_count
    np.savez_compressed(os.path.join(HERE, "accept.npz"), **A)

    # ---- quantised row dots ------------------------------------------------------------------
    R = {}
    for dtype, name in ((0, "q8_0"), (1, "q4_k"), (2, "q6_k")):
        for K in (256, 1024):
            N = 24
            w = synth.make_weight(dtype, K, N, seed=900 + dtype)
            x = synth.make_activation(2, K, seed=910 + dtype)
            R["%s_%d_w" % (name, K)] = w
            R["%s_%d_x" % (name, K)] = x
            R["%s_%d_y" % (name, K)] = gfo.gemv(dtype, w, x, N, which=ref)
            R["%s_%d_dense" % (name, K)] = gfo.dequant(dtype, w, which=ref)
    np.savez_compressed(os.path.join(HERE, "rowdot.npz"), **R)
    for f in ("prepare.npz", "accept.npz", "rowdot.npz"):
        print(f, os.path.getsize(os.path.join(HERE, f)))


if __name__ == "__main__":
    main()
