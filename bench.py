#!/usr/bin/env python3
"""Benchmark of the H1 speculative decode step on one MI355X.

Workload (configuration 4 of the benchmark): one H1 cycle of the Gemma-3-12B-shaped Q4_K_M target
(48 blocks, 2-row verify at an 8192-token fp16 KV context, tied Q6_K 262144 head, top-64
selection, lossless accept) with the 270M-shaped Q8_0 drafter (1 row, 4096-token context),
seeded random weights drawn on the device.  A step is one whole cycle replayed as a HIP
graph; `value` is the mean step latency in microseconds with every input resident in HBM.

Extra objects on the JSON line:
  roofline      the dominant kernel (2-row Q4_K gate+up GEMV fused with GeGLU, 66.4 MB of weights
                per launch): algorithmic bytes / mean launch duration, measured with HIP events
                around a graph of 48 back-to-back launches over the 48 blocks' own weights
                (3.2 GB, far beyond the caches) on the launch stream.
  configs       configs 0-3 on their own (one Q4_K GEMV at 1 row; one block's seven GEMVs at 2 rows;
                the drafter's decode with head and argmax; the Q6_K head with selection and
                acceptance): microseconds per unit as HIP graphs, algorithmic bytes, GB/s and the
                fraction of the 8 TB/s HBM peak.
  prefill       config 4's second half: a 2048-token prompt through the same stack.
  cpu_baseline  the reference's own CPU row dot (oracle/_ref) or the oracle port timed on the
                host cores on a bounded sample (one block's seven GEMVs at 2 rows, a column
                subset), extrapolated to a whole step by weight count; `all_cores` is the oracle's
                threaded row dot on the same GEMVs over the host's cores.  Reported, not a target.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0


def model_bytes(sh, rows, pos):
    """Algorithmic HBM bytes of one forward pass with its head: weights once per GEMV, activations in/out,
    KV once per KV head."""
    w = sh.body_weight_bytes() + sh.head_bytes()
    kv = 0
    for l in range(sh.layers):
        tokens = min(pos, sh.sliding_window) if sh.is_local(l) else pos
        kv += tokens * sh.kv_width * 2 * 2
    act = sh.layers * rows * 4 * (2 * sh.hidden * 4 + 2 * sh.q_width + 2 * sh.kv_width + 3 * sh.ffn)
    logits = rows * sh.vocab * 4 * 2
    norms = sh.layers * (4 * sh.hidden + 2 * sh.head_dim) * 4
    return w + kv + act + logits + norms


def step_bytes(T, D, t_pos, d_pos):
    """Algorithmic HBM bytes of one cycle."""
    return model_bytes(T, 2, t_pos) + model_bytes(D, 1, d_pos)


def timed_graph(fn, reps=10, warm=3):
    """fn's launches captured as one HIP graph; microseconds per replay, from events on the launch stream."""
    import torch
    fn()
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        fn()
    for _ in range(warm):
        graph.replay()
    stream = torch.cuda.current_stream()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record(stream)
    for _ in range(reps):
        graph.replay()
    e1.record(stream)
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) * 1e3 / reps


def config_figures(target, drafter, T, D, d_pos):
    """Configs 0-3 of the baseline on their own: microseconds, algorithmic bytes, GB/s and fraction of the
    HBM peak.  Every GEMV graph walks the 48 blocks' own weights, so the bytes come from HBM."""
    import ctypes as C
    import torch
    from guffin_amd import hip, synth
    lib = hip.lib()
    H, F, QW, KW = T.hidden, T.ffn, T.q_width, T.kv_width
    dts = [int(d) for d in T.dtypes]

    def figure(us, nbytes, what):
        gbs = nbytes / us / 1e3
        return {"what": what, "us": round(us, 2), "bytes": int(nbytes), "GB/s": round(gbs, 1),
                "hbm_frac": round(gbs / HBM_PEAK_GBS, 4)}

    def gemv(dtype, tiles, x, xs, parts, out, rows, K, N):
        hip.check(lib.guffin_hip_gemv_packed(hip._stream(), dtype, C.c_void_p(tiles), hip._p(x), hip._p(xs), hip._p(parts),
                                             hip._p(out), rows, K, N))

    def buffers(rows, K, N, dtype):
        x = torch.randn(rows, K, device="cuda")
        return (x, hip.group_sums(x), torch.empty((hip.gemv_packed_slices(dtype, K, N), rows, N), device="cuda"),
                torch.empty((rows, N), device="cuda"))

    out = {}
    print("bench: timing config 0", file=sys.stderr, flush=True)
    # config 0: one Q4_K matvec, 1 row, 3840 -> 15360 (the gate matrices of the 48 blocks in turn)
    x1, xs1, parts1, y1 = buffers(1, H, F, dts[4])
    us = timed_graph(lambda: [gemv(dts[4], target.layers[l].tiles[4], x1, xs1, parts1, y1, 1, H, F)
                              for l in range(T.layers)]) / T.layers
    out["0"] = figure(us, synth.weight_bytes(dts[4], H, F) + H * 4 + F * 4,
                      "one Q4_K GEMV, 1 row, 3840 -> 15360 (gemv_packed_kernel<Q4_K, 1>)")

    print("bench: timing config 1", file=sys.stderr, flush=True)
    # config 1: the seven GEMVs of one block at 2 rows, as the step launches them (q/k/v in one launch,
    # o, gate+up fused with GeGLU, down)
    x2, xs2, _, _ = buffers(2, H, F, dts[4])
    qkv_n = (C.c_uint32 * 3)(QW, KW, KW)
    qkv_dt = (C.c_int * 3)(dts[0], dts[1], dts[2])
    lib.guffin_hip_gemv_packed_multi_slices.restype = C.c_uint32
    S = lib.guffin_hip_gemv_packed_multi_slices(3, qkv_dt, qkv_n, H)
    qkv_parts = [torch.empty((S, 2, n), device="cuda") for n in (QW, KW, KW)]
    qkv_pp = (C.c_void_p * 3)(*[t.data_ptr() for t in qkv_parts])
    xa, xas, parts_o, y_o = buffers(2, QW, H, dts[3])
    xh, xhs, parts_d, y_d = buffers(2, F, H, dts[6])
    h_out, h_sums = torch.empty(2, F, device="cuda"), hip._receipt(2, F, "cuda")

    def block_gemvs():
        for l in range(T.layers):
            L = target.layers[l]
            tl = (C.c_void_p * 3)(L.tiles[0], L.tiles[1], L.tiles[2])
            hip.check(lib.guffin_hip_gemv_packed_multi(hip._stream(), 3, qkv_dt, tl, qkv_n, qkv_pp, hip._p(x2), hip._p(xs2), 2, H))
            gemv(dts[3], L.tiles[3], xa, xas, parts_o, None, 2, QW, H)   # partial planes out, as in the step
            hip.check(lib.guffin_hip_gateup_geglu(hip._stream(), dts[4], C.c_void_p(L.tiles[4]), C.c_void_p(L.tiles[5]),
                                                  hip._p(x2), hip._p(xs2), hip._p(h_out), hip._p(h_sums), 2, H, F))
            gemv(dts[6], L.tiles[6], xh, xhs, parts_d, None, 2, F, H)

    us = timed_graph(block_gemvs) / T.layers
    acts = 2 * 4 * (H + QW + 2 * KW + QW + H + H + F + F + H)   # rows x fp32 x (inputs and outputs of the four launches)
    out["1"] = figure(us, T.layer_weight_bytes() + acts,
                      "the 7 GEMVs of one 12B block at 2 rows: q/k/v (one launch), o, gate+up+GeGLU, down")

    print("bench: timing config 2", file=sys.stderr, flush=True)
    # config 2: drafter decode of one token at a 4096-token cache, tied Q8_0 head, greedy argmax
    token = torch.full((1,), 2, dtype=torch.int32, device="cuda")
    head_d = drafter.head_tiles
    assert head_d.numel() == hip.packed_bytes(int(D.embed_dtype), D.hidden, D.vocab)

    def draft_decode():
        hidden, sums, _, _, _ = drafter.forward(token, d_pos)
        hip.argmax(hip.gemv_packed(int(D.embed_dtype), head_d, hidden, sums, D.vocab))

    out["2"] = figure(timed_graph(draft_decode), model_bytes(D, 1, d_pos),
                      "270M Q8_0 drafter: 18 blocks at a %d-token cache, 262144 x 640 head, argmax" % d_pos)

    print("bench: timing config 3", file=sys.stderr, flush=True)
    # config 3: Q6_K head on 2 rows, top-64 selection, draft law of N(0, 4) logits, acceptance
    xo, xos, _, _ = buffers(2, H, 64, dts[4])
    q_logits = 2.0 * torch.randn(T.vocab, device="cuda")
    options = hip.SamplerOptions(1.0, 64, 0.95, 0.0, 1.0)
    head_t = target.head_tiles
    assert head_t.numel() == hip.packed_bytes(int(T.embed_dtype), H, T.vocab)

    def head_accept():
        p = hip.gemv_packed(int(T.embed_dtype), head_t, xo, xos, T.vocab)
        cands, _ = hip.select_candidates(p, 64)
        law, proposal, status = hip.draft_law(q_logits, options, seed=0, step=0)
        hip.spec_accept(cands, law, proposal, options, seed=0, step=0, status=status)

    out["3"] = figure(timed_graph(head_accept), T.head_bytes() + 2 * 2 * T.vocab * 4 + T.vocab * 4,
                      "262144 x 3840 Q6_K head on 2 rows, top-64 selection, draft law, accept / residual")
    return out


def cpu_baseline(T, D, budget_s=20.0):
    """Times the CPU path on a bounded sample and extrapolates to one step by weight count."""
    import numpy as np
    from guffin_amd import synth
    from oracle import gfo
    gfo.build()
    ref = gfo.ref()
    kind = "reference" if ref is not None else "port"
    cores = 1 if ref is not None else (os.cpu_count() or 1)
    shapes = list(zip(T.dtypes, T.proj_shapes()))
    # calibrate on a small slice, then size the sample to the budget
    dt, (K, N) = shapes[0]
    w = synth.make_weight(dt, K, 64, 1)
    x = synth.make_activation(2, K, 2)
    t0 = time.perf_counter()
    gfo.gemv(dt, w, x, 64, threads=cores, which=ref)
    per_weight = (time.perf_counter() - t0) / (K * 64)
    layer_weights = sum(K * N for _, (K, N) in shapes)
    frac = min(1.0, budget_s / (per_weight * layer_weights * 1.3))
    done_weights, elapsed = 0, 0.0
    # whole blocks' worth of GEMVs (fresh weights each time) until about half the budget is spent
    repeats = max(1, int(0.6 * budget_s / max(per_weight * layer_weights * frac, 1e-9)))
    for rep in range(repeats):
        for i, (dt, (K, N)) in enumerate(shapes):
            n = max(64, int(N * frac) // 64 * 64)
            w = synth.make_weight(dt, K, n, 10 + i + 100 * rep)
            x = synth.make_activation(2, K, 20 + i + 100 * rep)
            t0 = time.perf_counter()
            gfo.gemv(dt, w, x, n, threads=cores, which=ref)
            elapsed += time.perf_counter() - t0
            done_weights += K * n
    step_weights = (T.layers * layer_weights + T.hidden * T.vocab
                    + 0.5 * (D.layers * sum(K * N for K, N in D.proj_shapes()) + D.hidden * D.vocab))  # drafter: 1 row
    value_us = elapsed / done_weights * step_weights * 1e6
    # the same rows spread over the host's cores (rows of W are independent; a row's arithmetic is
    # unchanged): the oracle's threaded row dot on one block's GEMVs
    many = min(os.cpu_count() or 1, 16)
    par_weights, par_elapsed = 0, 0.0
    for i, (dt, (K, N)) in enumerate(shapes):
        n = max(64, int(N * min(1.0, 4.0 * frac)) // 64 * 64)
        w = synth.make_weight(dt, K, n, 900 + i)
        x = synth.make_activation(2, K, 920 + i)
        t0 = time.perf_counter()
        gfo.gemv(dt, w, x, n, threads=many)
        par_elapsed += time.perf_counter() - t0
        par_weights += K * n
    return {
        "value": round(value_us, 1), "unit": "us", "cores": cores, "kind": kind,
        "all_cores": {"value": round(par_elapsed / par_weights * step_weights * 1e6, 1), "unit": "us", "cores": many,
                      "kind": "port", "sample": "one 12B block's 7 GEMVs at 2 rows (%.2f s), oracle row dots on %d threads"
                                                % (par_elapsed, many)},
        "sample": "%d x one 12B block's 7 GEMVs at 2 rows, first %.1f%% of each matrix's columns (%.2f s of CPU work), "
                  "scaled to the step's weight count; %s" % (
                      repeats, 100 * frac, elapsed,
                      "reference dot_q4_k_row_f32 / dot_q6_k_row_f32 (src/tensor/quantization.cpp), single thread"
                      if ref is not None else "oracle gfo_gemv_mt on all host threads"),
    }


def prefill_figure(target, T, tokens=2048):
    """Config 4's second half: a 2048-token prompt through the 48 blocks on the matrix core."""
    import torch
    ids = torch.randint(0, T.vocab, (tokens,), dtype=torch.int32, device="cuda")
    target.prefill(ids, 0)                      # warm-up (also sizes the scratch arena)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    _, status = target.prefill(ids, 0)
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) * 1e3
    macs = tokens * T.layers * sum(K * N for K, N in T.proj_shapes())
    # every MAC is issued twice (fp16 hi and lo halves of the activation) on the f16 matrix pipe
    issued_flops = 2 * 2 * macs
    return {"tokens": tokens, "ms": round(ms, 2), "tokens_per_s": round(tokens / ms * 1e3, 1),
            "model_tflops": round(2 * macs / ms / 1e9, 1), "bound": "mfma",
            "mfma_frac": round(issued_flops / (ms * 1e-3) / 2.5e15, 4), "peak": "2.5 PFLOP/s f16 dense",
            "status": int(status.item())}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--layers", type=int, default=0, help="debug: truncate the target to this many blocks")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-prefill", action="store_true", help="skip the 2048-token prefill figure")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs the H1 step on ONE GPU; --gpus %d is not supported "
              "(no collectives or sharding are part of it)" % args.gpus, file=sys.stderr)
        sys.exit(2)

    import torch
    from dataclasses import replace
    from guffin_amd import hip, model
    hip.init(0)

    T, D = model.GEMMA3_12B, model.GEMMA3_270M
    if args.layers:
        T = replace(T, layers=args.layers)
    t_pos, d_pos = 8190, 4096
    target = model.DeviceModel.random(T, seed=0, position=t_pos)
    drafter = model.DeviceModel.random(D, seed=1, position=d_pos)
    plan = model.H1Plan(target, drafter, t_pos, d_pos, temperature=1.0, top_k=64, top_p=0.95, min_p=0.0,
                        seed=0, publish=True)
    plan.root.fill_(2)

    # eager once (validates the path end to end), then capture the whole cycle as a HIP graph
    plan.step(0)
    torch.cuda.synchronize()
    first = plan.read_result()
    if int(plan.status.item()) != 0 or first["status"] != 0:
        raise RuntimeError("H1 step failed: device status %d, law status %d" % (int(plan.status.item()), first["status"]))
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        plan.step(0)
    for _ in range(args.warmup):
        graph.replay()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        graph.replay()
    torch.cuda.synchronize()
    ms_per_step = (time.perf_counter() - t0) * 1e3 / args.steps
    replayed = plan.read_result()
    if (replayed["accepted"], replayed["token"], replayed["next_root"]) != (first["accepted"], first["token"], first["next_root"]):
        raise RuntimeError("graph replay changed the step's decision")

    # ---- roofline of the dominant kernel: fused 2-row Q4_K gate+up GEMV + GeGLU, one launch per block -----
    import ctypes as C
    H, F = T.hidden, T.ffn
    x = torch.randn(2, H, device="cuda")
    xs = hip.group_sums(x)
    h_out = torch.empty(2, F, device="cuda")
    h_sums = hip._receipt(2, F, "cuda")
    lib = hip.lib()

    def launch_all():
        for l in range(T.layers):
            L = target.layers[l]
            # (ctypes passes a bare Python int as a 32-bit C int: pointers must be wrapped)
            hip.check(lib.guffin_hip_gateup_geglu(hip._stream(), int(L.dtype[4]), C.c_void_p(L.tiles[4]), C.c_void_p(L.tiles[5]),
                                                  hip._p(x), hip._p(xs), hip._p(h_out), hip._p(h_sums), 2, H, F))

    launch_all()
    torch.cuda.synchronize()
    kgraph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(kgraph):
        launch_all()
    for _ in range(3):
        kgraph.replay()
    stream = torch.cuda.current_stream()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    reps = 10
    e0.record(stream)
    for _ in range(reps):
        kgraph.replay()
    e1.record(stream)
    torch.cuda.synchronize()
    launch_us = e0.elapsed_time(e1) * 1e3 / (reps * T.layers)
    # the same kernel dispatched alone (one launch, then a wait): the reference's benchmark reports both an
    # isolated and a sustained mode (include/local_gguf_engine/benchmarks/quick_benchmark.hpp:13-17)
    isolated = []
    for rep in range(3 * T.layers):
        L = target.layers[rep % T.layers]
        e0.record(stream)
        hip.check(lib.guffin_hip_gateup_geglu(hip._stream(), int(L.dtype[4]), C.c_void_p(L.tiles[4]), C.c_void_p(L.tiles[5]),
                                              hip._p(x), hip._p(xs), hip._p(h_out), hip._p(h_sums), 2, H, F))
        e1.record(stream)
        torch.cuda.synchronize()
        isolated.append(e0.elapsed_time(e1) * 1e3)
    isolated_us = sorted(isolated)[len(isolated) // 2]
    from guffin_amd import synth
    # weights once, activation rows in (fp32 rows are the operator's input; the kernel reads their receipt), h out
    kernel_bytes = 2 * synth.weight_bytes(T.dtypes[4], H, F) + 2 * H * 4 + 2 * F * 4
    achieved = kernel_bytes / launch_us / 1e3  # GB/s

    # a plain 256 MiB device copy: the reference reading for FETCH_SIZE / WRITE_SIZE counter runs
    cal_src = torch.empty(64 << 20, dtype=torch.float32, device="cuda").fill_(1.0)
    cal_dst = torch.empty_like(cal_src)
    cal_dst.copy_(cal_src)
    torch.cuda.synchronize()
    del cal_src, cal_dst

    total_bytes = step_bytes(T, D, t_pos, d_pos)
    line = {
        "metric": "h1_step_latency_us", "value": round(ms_per_step * 1e3, 1), "unit": "us",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": False, "scaling": "weak", "vs_baseline": None, "dtype": "f32",
        "data": "synthetic",
        "config": {
            "workload": "config 4: full Gemma-3-12B-shaped Q4_K_M H1 step (270M Q8_0 drafter 1 row @4096 ctx, "
                        "48-block 2-row verify @8192-token fp16 KV, Q6_K 262144 head, top-64 select, lossless accept)",
            "target_blocks": T.layers, "rows": 2, "kv_context": t_pos + 2, "vocab": T.vocab,
            "step_algorithmic_bytes": total_bytes,
            "step_hbm_frac": round(total_bytes / (ms_per_step * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
            "accepted": int(first["accepted"]),
        },
        "roofline": {
            "kernel": "gateup_geglu_kernel<Q4_K, 2> (Q4_K gate+up GEMV + GeGLU, 2 rows, K=3840, N=2x15360)",
            "bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
            "frac": round(achieved / HBM_PEAK_GBS, 4),
            # HBM bytes per launch from the FETCH_SIZE / WRITE_SIZE counter runs recorded in
            # profiles/gateup_geglu_q4k_hbm_traffic.txt (copy-calibrated: fetch x 1.9997, write x 1)
            "traffic": 67046400,
            "bytes_per_launch": kernel_bytes, "launch_us": round(launch_us, 3),
            "sustained_dispatches": T.layers, "isolated_launch_us": round(isolated_us, 3),
        },
    }
    line["configs"] = config_figures(target, drafter, T, D, d_pos)
    if not args.no_prefill:
        line["prefill"] = prefill_figure(target, T)
    if not args.no_cpu_baseline:
        line["cpu_baseline"] = cpu_baseline(T, D)
    print(json.dumps(line))


if __name__ == "__main__":
    main()
