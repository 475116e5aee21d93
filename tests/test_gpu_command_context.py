"""include/guffin_hip_command_context.hpp at run time: tests/shim/command_context_run (built from the reference's
headers where the reference checkout is present; the executable travels to the GPU box) drives one verify pass's
operators through HipCommandContext on buffers made by allocate_hip_buffer / view_hip_buffer / upload_weight_tiles
-- embedding, norm with a receipt, the projections with the producer's receipt and with the context's own, head
norms, rotation, K/V narrowing, attention over K/V views that start 12 bytes into their allocations
(tests/tensor/gemma3_metal_tests.cpp:765-774), GeGLU, the tied head, request resolution, candidate selection and
the candidate read-back; then, in a second and a third command buffer, the operators around the pass (residual norm,
projections on five rows by the matrix path and by pairs of rows, K/V scatter into those views and copy out of them,
prefill attention over them with and without a window, candidate selection from host-side requests of two rows and of
one) -- and writes every result to a directory.  Here every result is compared, bit for bit,
with the same operator called through the C entry points (ctypes) on the same inputs, and with the oracle where a
tolerance says more than equality.  The program itself checks the exception classes of the error paths."""
import os
import subprocess

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
RUNNER = os.path.join(ROOT, "tests", "shim", "_build", "command_context_run")

H, QW, KW, F, V, CAP, ROWS = 3840, 4096, 2048, 2048, 8192, 64, 2


def raw(path, array):
    np.ascontiguousarray(array).tofile(path)


def bits(t):
    return t.detach().cpu().contiguous().view(-1).numpy().view(np.uint8).tobytes()


@pytest.mark.skipif(not os.path.exists(RUNNER), reason="tests/shim/_build/command_context_run is not built "
                    "(make -C tests/shim, where the reference checkout is present)")
def test_the_command_context_runs_a_verify_pass(tmp_path):
    import torch
    from guffin_amd import hip, synth
    hip.init(0)
    d = str(tmp_path)
    rng = np.random.Generator(np.random.PCG64(11))
    weights = {"embed.q6k": (synth.Q6_K, H, V, 1), "wq.q4k": (synth.Q4_K, H, QW, 2), "wk.q4k": (synth.Q4_K, H, KW, 3),
               "wv.q6k": (synth.Q6_K, H, KW, 4), "wg.q4k": (synth.Q4_K, H, F, 5), "wu.q4k": (synth.Q4_K, H, F, 6)}
    host = {name: synth.make_weight(dt, K, N, seed) for name, (dt, K, N, seed) in weights.items()}
    for name, w in host.items():
        raw(os.path.join(d, name), w)
    tokens = np.array([17, 4099], np.uint32)
    positions = np.array([40, 41], np.uint32)
    schedule = np.array([[0, 40, 0, 1], [0, 40, 1, 2]], np.uint32)     # ring positions 0..39, then the rows' ancestors
    ancestors = np.array([0, 0, 1], np.uint32)
    norms = {n: (1.0 + 0.1 * rng.standard_normal(w)).astype(np.float32) for n, w in (("attn_norm", H), ("q_norm", 256), ("k_norm", 256))}
    ring_k = rng.standard_normal((CAP, KW)).astype(np.float16)
    ring_v = rng.standard_normal((CAP, KW)).astype(np.float16)
    requests = np.zeros(2, hip.selection_row_dtype)
    requests[0]["history_token_ids"][:5] = [3, 9, 9, 4099, 70]
    requests[0]["history_length"], requests[0]["history_window_limit"] = 5, 64
    requests[1]["history_token_ids"][:3] = [8000, 3, 12]
    requests[1]["history_length"], requests[1]["history_window_limit"] = 3, 64
    requests[1]["suffix_token_ids"][0], requests[1]["suffix_count"] = 4099, 1
    raw(os.path.join(d, "tokens.u32"), tokens); raw(os.path.join(d, "positions.u32"), positions)
    raw(os.path.join(d, "schedule.u32"), schedule); raw(os.path.join(d, "ancestors.u32"), ancestors)
    for n, g in norms.items():
        raw(os.path.join(d, n + ".f32"), g)
    raw(os.path.join(d, "ring_k.f16"), ring_k); raw(os.path.join(d, "ring_v.f16"), ring_v)
    raw(os.path.join(d, "requests.raw"), requests)
    # the second command buffer's inputs: five rows for the calls with more than two, a chunk of keys and values
    P = 5
    xp = rng.standard_normal((P, H)).astype(np.float32)
    qp = rng.standard_normal((P, QW)).astype(np.float32)
    chunk_k = rng.standard_normal((P, KW)).astype(np.float16)
    chunk_v = rng.standard_normal((P, KW)).astype(np.float16)
    selected = np.array([1, 0], np.uint32)
    raw(os.path.join(d, "xp.f32"), xp); raw(os.path.join(d, "qp.f32"), qp)
    raw(os.path.join(d, "chunk_k.f16"), chunk_k); raw(os.path.join(d, "chunk_v.f16"), chunk_v)
    raw(os.path.join(d, "selected.u32"), selected)

    print("running the command context", flush=True)
    run = subprocess.run([RUNNER, d], capture_output=True, text=True, timeout=120)
    assert run.returncode == 0, (run.returncode, run.stdout[-2000:], run.stderr[-2000:])
    stats = dict(line.split(" ", 1) for line in open(os.path.join(d, "stats.txt")).read().strip().splitlines())
    assert stats["exceptions"] == "ok"
    assert int(stats["verifier_status"]) == 0 and int(stats["operator_status"]) == 0
    assert int(stats["commit_count"]) == 1 and int(stats["synchronous_wait_count"]) == 1 and int(stats["command_buffer_count"]) == 1
    assert int(stats["memory_barrier_count"]) == 8
    assert int(stats["q4_width_two"]) == 5 and int(stats["q6_width_two"]) == 2      # q (twice), k, gate, up; v and the head
    assert int(stats["attention_dispatches"]) == 1 and int(stats["attention_tokens"]) == 42
    assert 20_000 < int(stats["gpu_duration_ns"]) < 100_000_000

    def out(name, dtype=np.uint8):
        return np.fromfile(os.path.join(d, name), dtype)

    # ---- the same operators through the C entry points ----------------------------------------------------------
    dev = {name: torch.from_numpy(w).cuda() for name, w in host.items()}
    tiles = {name: hip.repack(weights[name][0], dev[name], weights[name][1], weights[name][2]) for name in host}
    gam = {n: torch.from_numpy(g).cuda() for n, g in norms.items()}
    t_tokens = torch.from_numpy(tokens.view(np.int32)).cuda()
    t_pos = torch.from_numpy(positions.view(np.int32)).cuda()
    status = hip.new_status()
    x0 = hip.embed(synth.Q6_K, dev["embed.q6k"], t_tokens, H, float(np.sqrt(np.float32(H))), V, status=status)
    u, receipt_u = hip.rms_norm(x0, gam["attn_norm"], want_sums=True, status=status)
    q = hip.gemv_packed(synth.Q4_K, tiles["wq.q4k"], u, receipt_u, QW)
    q_own = hip.gemv_packed(synth.Q4_K, tiles["wq.q4k"], u, hip.group_sums(u), QW)
    k = hip.gemv_packed(synth.Q4_K, tiles["wk.q4k"], u, receipt_u, KW)
    v = hip.gemv_packed(synth.Q6_K, tiles["wv.q6k"], u, receipt_u, KW)
    qn = hip.head_rms_norm(q, gam["q_norm"], 16, 256)
    kn = hip.head_rms_norm(k, gam["k_norm"], 8, 256)
    qr = hip.rope_neox(qn, t_pos, 16, 256, 256, 1e6, 0.125)
    priv_k, priv_v = hip.kv_store_f16(kn, v, t_pos, 8, 256, 256, 1e6, 0.125, status=status)
    attn, receipt_a = hip.attention_decode(qr, torch.from_numpy(ring_k).cuda(), torch.from_numpy(ring_v).cuda(), priv_k, priv_v,
                                           torch.from_numpy(schedule.view(np.int32)).cuda(), torch.from_numpy(ancestors.view(np.int32)).cuda(),
                                           42, CAP - 1, 16, 8, 256, 0.0625, want_sums=True, status=status)
    gate = hip.gemv_packed(synth.Q4_K, tiles["wg.q4k"], u, receipt_u, F)
    up = hip.gemv_packed(synth.Q4_K, tiles["wu.q4k"], u, receipt_u, F)
    h, receipt_h = hip.geglu(gate, up, want_sums=True)
    logits = hip.gemv_packed(synth.Q6_K, tiles["embed.q6k"], u, hip.group_sums(u), V)
    resolved, _, request_status = hip.selection_requests(requests, V, 40, True)
    result, row_status = hip.select_candidates_resolved(logits, 320, resolved)
    torch.cuda.synchronize()
    assert int(status.item()) == 0 and int(request_status.item()) == 0 and int(row_status.abs().sum()) == 0

    expected = {"x0": x0, "u": u, "receipt_u": receipt_u, "q": q, "q_own": q_own, "k": k, "v": v, "qn": qn, "kn": kn, "qr": qr,
                "priv_k": priv_k, "priv_v": priv_v, "attn": attn, "receipt_a": receipt_a, "h": h, "receipt_h": receipt_h,
                "logits": logits, "resolved": resolved}
    for name, tensor in expected.items():
        got, want = out(name + ".out").tobytes(), bits(tensor)
        assert got[:len(want)] == want, name          # (a receipt buffer is allocated in whole words: compare its bytes)
    # the producer's receipt and the context's own give the same projection (what the reference asks of its
    # prepared and unprepared kernels, tests/tensor/gemma3_metal_tests.cpp:452-453)
    assert out("q.out").tobytes() == out("q_own.out").tobytes()
    cands = hip.candidates_to_numpy(result)
    for r in range(2):
        flat = out("candidates%d.out" % r, np.uint32)
        count = int(flat[0])
        assert count == int(cands[r]["count"]) and count >= 40
        assert np.array_equal(flat[1:1 + 2 * count:2], cands[r]["values"]["token"][:count])
        assert np.array_equal(flat[2:2 + 2 * count:2], cands[r]["values"]["logit"][:count].view(np.uint32))
    # and the numbers mean something: the 12-byte views feed the attention the rows they hold
    from oracle import gfo
    gfo.build()
    want_q = gfo.gemv(synth.Q4_K, host["wq.q4k"], u.cpu().numpy(), QW)
    scale = np.sqrt((want_q.astype(np.float64) ** 2).mean())
    assert np.max(np.abs(out("q.out", np.float32).reshape(2, QW) - want_q)) <= 1e-3 * scale


    # ---- the second and third command buffers ------------------------------------------------------------------------
    assert int(stats["launches_two"]) == 2 and int(stats["launches_one"]) == 2
    assert int(stats["second_command_buffers"]) == 2 and int(stats["second_commits"]) == 2 and int(stats["third_commits"]) == 3
    assert int(stats["q4_generic_tiled"]) == 1 and int(stats["q6_generic_tiled"]) == 1 and int(stats["q4_small_batch"]) == 3
    assert int(stats["third_gpu_duration_ns"]) > 0
    assert int(out("marks.out", np.uint32)[0]) == 0xC0FFEE
    t_xp, t_qp = torch.from_numpy(xp).cuda(), torch.from_numpy(qp).cuda()
    y_add = hip.rms_norm(u, gam["attn_norm"], residual=x0, status=status)
    image = hip.prefill_pack(t_xp)
    yp_matrix = hip.prefill_gemm(synth.Q4_K, tiles["wq.q4k"], image, P, H, QW)
    yv_matrix = hip.prefill_gemm(synth.Q6_K, tiles["wv.q6k"], image, P, H, KW)
    yp_pairs = torch.cat([hip.gemv_packed(synth.Q4_K, tiles["wq.q4k"], t_xp[r:r + 2].contiguous(), hip.group_sums(t_xp[r:r + 2].contiguous()), QW)
                          for r in range(0, P, 2)])
    rk, rv = torch.from_numpy(ring_k).cuda(), torch.from_numpy(ring_v).cuda()
    hip.kv_scatter(priv_k, priv_v, torch.from_numpy(selected.view(np.int32)).cuda(), rk, rv, 40, KW, CAP - 1)
    ck, cv = torch.zeros((16, KW), dtype=torch.float16, device="cuda"), torch.zeros((16, KW), dtype=torch.float16, device="cuda")
    hip.kv_cache_copy(rk, rv, ck, cv, 30, 12, CAP - 1, 15)
    t_ck, t_cv = torch.from_numpy(chunk_k).cuda(), torch.from_numpy(chunk_v).cuda()
    pattn = hip.prefill_attention(t_qp, rk, rv, t_ck, t_cv, 42, 0, CAP - 1, 16, 8, 256, 0.0625, matrix_core=False)
    pattn_window = hip.prefill_attention(t_qp, rk, rv, t_ck, t_cv, 42, 16, CAP - 1, 16, 8, 256, 0.0625, matrix_core=False)
    host_requests = np.zeros(2, hip.resolved_row_dtype)
    host_requests[0]["top_k"], host_requests[0]["base_candidate_count"], host_requests[0]["history_count"] = 40, 43, 3
    host_requests[0]["history_token_ids"][:3] = [3, 9, 70]
    host_requests[1]["top_k"], host_requests[1]["base_candidate_count"] = 1, 1
    d_requests = torch.from_numpy(host_requests.view(np.uint8).copy()).cuda()
    pair, pair_status = hip.select_candidates_resolved(logits, 43, d_requests)
    single, single_status = hip.select_candidates_resolved(logits[:1].contiguous(), 43, d_requests[:hip.resolved_row_dtype.itemsize].contiguous())
    torch.cuda.synchronize()
    assert int(status.item()) == 0 and int(pair_status.abs().sum()) == 0 and int(single_status.abs().sum()) == 0
    assert torch.equal(rk[40], priv_k[1]) and torch.equal(rk[41], priv_k[0]) and torch.equal(ck[(30 + 11) & 15], rk[41])
    second = {"y_add": y_add, "yp_matrix": yp_matrix, "yv_matrix": yv_matrix, "yp_pairs": yp_pairs, "ring_k_after": rk,
              "ring_v_after": rv, "copy_k": ck, "copy_v": cv, "pattn": pattn, "pattn_window": pattn_window}
    for name, tensor in second.items():
        assert out(name + ".out").tobytes() == bits(tensor), name
    # rows of the matrix path agree with the decode path's to the operator bound, and the window changes the answer
    assert float((yp_matrix - yp_pairs).abs().max()) <= 1e-3 * float(yp_pairs.abs().max())
    assert not torch.equal(pattn, pattn_window)
    for name, record in (("pair0", hip.candidates_to_numpy(pair)[0]), ("pair1", hip.candidates_to_numpy(pair)[1]),
                         ("single", hip.candidates_to_numpy(single)[0])):
        flat = out(name + ".out", np.uint32)
        count = int(flat[0])
        assert count == int(record["count"]) and count >= 1
        assert np.array_equal(flat[1:1 + 2 * count:2], record["values"]["token"][:count])
        assert np.array_equal(flat[2:2 + 2 * count:2], record["values"]["logit"][:count].view(np.uint32))
    assert int(out("pair1.out", np.uint32)[0]) == 1 and int(out("pair0.out", np.uint32)[0]) >= 40
    assert out("single.out").tobytes() == out("pair0.out").tobytes()
