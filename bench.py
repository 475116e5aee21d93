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
                around graphs of 48 back-to-back launches over the 48 blocks' own weights
                (3.2 GB, far beyond the caches) on the launch stream; min / max over the replays and
                over single launches; `traffic` is read from the committed counter profile.
  rooflines     the same figures for the step's other streaming kernels worth watching: the local
                layers' attention (the kernel furthest from its bound) and the global layers', the down
                projection, the q/k/v launch, the o projection and the two head GEMVs.
  configs       configs 0-3 on their own (one Q4_K GEMV at 1 row; one block's seven GEMVs at 2 rows;
                the drafter's decode with head and argmax; the Q6_K head with selection and
                acceptance): microseconds per unit as HIP graphs, algorithmic bytes, GB/s and the
                fraction of the 8 TB/s HBM peak.
  chain         the same step recorded once and replayed as dispatch packets on the library's own queue
                (guffin_hip_chain_*): wall microseconds per replay with its wait, and the device's clock
                between the first packet's start and the last packet's end.
  prefill       config 4's second half: a 2048-token prompt through the same stack.
  cpu_baseline  the reference's own CPU row dot (oracle/_ref) or the oracle port timed on the
                host cores: configs 0 and 1 in full, config 3 on a vocabulary slice plus the oracle's
                selection, law and acceptance in full, config 2 by weight count; the step is 48 blocks +
                head + drafter from those.  Each config's figure also sits in configs[i].cpu_baseline.
                `all_cores` is the oracle's threaded row dot over the host's cores.  Reported, not a target.
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


def replay_times(fn, reps=10, warm=3):
    """fn's launches captured as one HIP graph; microseconds of each of `reps` warmed replays, from event
    pairs on the launch stream (recorded back to back, read after one synchronisation)."""
    import torch
    fn()
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        fn()
    for _ in range(warm):
        graph.replay()
    stream = torch.cuda.current_stream()
    marks = [torch.cuda.Event(enable_timing=True) for _ in range(reps + 1)]
    marks[0].record(stream)
    for i in range(reps):
        graph.replay()
        marks[i + 1].record(stream)
    torch.cuda.synchronize()
    return [marks[i].elapsed_time(marks[i + 1]) * 1e3 for i in range(reps)]


def timed_graph(fn, reps=10, warm=3):
    """Mean microseconds per replay."""
    times = replay_times(fn, reps, warm)
    return sum(times) / len(times)


def profile_traffic(kernel_prefix):
    """HBM bytes per launch of a kernel from the committed counter profile (two rocprofv3 --pmc runs,
    copy-calibrated): the line `FETCH_SIZE a KiB x f + WRITE_SIZE b KiB x g` under the kernel's name."""
    import re
    path = os.path.join(ROOT, "profiles", "gateup_geglu_q4k_hbm_traffic.txt")
    if not os.path.exists(path):
        return None, None
    lines = open(path).read().splitlines()
    for i, text in enumerate(lines[:-1]):
        if text.startswith(kernel_prefix):
            m = re.search(r"FETCH_SIZE ([0-9.]+) KiB x ([0-9.]+) \+ WRITE_SIZE ([0-9.]+) KiB x ([0-9.]+)", lines[i + 1])
            if m:
                a, f, b, g = (float(v) for v in m.groups())
                return int(round((a * f + b * g) * 1024)), "profiles/gateup_geglu_q4k_hbm_traffic.txt"
    return None, None


def kernel_roofline(name, launch, layers, bytes_per_launch, traffic_prefix, replays=12):
    """Roofline object of one streaming kernel.  launch(l) enqueues the kernel on block l's own operands, so
    a graph of `layers` launches streams from HBM; sustained figures come from `replays` warmed replays
    (layers * replays >= 100 launches), single-launch figures from event pairs around 3 * layers launches
    enqueued back to back."""
    import torch

    def all_layers():
        for l in layers:
            launch(l)

    per_replay = [t / len(layers) for t in replay_times(all_layers, reps=max(replays, -(-100 // len(layers))))]
    launch_us = sum(per_replay) / len(per_replay)
    stream = torch.cuda.current_stream()
    count = 3 * len(layers)
    marks = [torch.cuda.Event(enable_timing=True) for _ in range(count + 1)]
    all_layers()                      # warm
    torch.cuda.synchronize()
    marks[0].record(stream)
    for i in range(count):
        launch(layers[i % len(layers)])
        marks[i + 1].record(stream)
    torch.cuda.synchronize()
    single = sorted(marks[i].elapsed_time(marks[i + 1]) * 1e3 for i in range(count))
    # the same kernel dispatched alone (one launch, then a wait): the reference's benchmark reports both an
    # isolated and a sustained mode (include/local_gguf_engine/benchmarks/quick_benchmark.hpp:13-17)
    isolated = []
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    for rep in range(len(layers)):
        e0.record(stream)
        launch(layers[rep])
        e1.record(stream)
        torch.cuda.synchronize()
        isolated.append(e0.elapsed_time(e1) * 1e3)
    achieved = bytes_per_launch / launch_us / 1e3  # GB/s
    traffic, source = profile_traffic(traffic_prefix) if traffic_prefix else (None, None)
    return {
        "kernel": name, "bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
        "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": traffic, "traffic_source": source,
        "bytes_per_launch": int(bytes_per_launch), "launch_us": round(launch_us, 3),
        "launch_us_min": round(min(per_replay), 3), "launch_us_max": round(max(per_replay), 3),
        "launches": len(per_replay) * len(layers), "sustained_dispatches": len(layers),
        "single_launch_us": {"min": round(single[0], 3), "median": round(single[len(single) // 2], 3),
                             "max": round(single[-1], 3), "launches": count},
        "isolated_launch_us": round(sorted(isolated)[len(isolated) // 2], 3),
    }


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


def cpu_baseline(T, D):
    """The CPU path on the host's cores, per config and for the step.  Configs 0 and 1 run in full, config 3's
    head on a vocabulary slice (scaled) with the oracle's selection, law and acceptance in full, config 2 by
    weight count from one drafter block and a slice of its head; the step is 48 blocks + head + drafter."""
    import ctypes as C
    import numpy as np
    from guffin_amd import synth
    from oracle import gfo
    gfo.build()
    ref = gfo.ref()
    kind = "reference" if ref is not None else "port"
    cores = 1 if ref is not None else min(os.cpu_count() or 1, 16)
    how = ("reference dot_q4_k_row_f32 / dot_q6_k_row_f32 (src/tensor/quantization.cpp), single thread" if ref is not None
           else "oracle gfo_gemv_mt on %d host threads" % cores)
    seeds = iter(range(10, 10 ** 6))

    def gemv_seconds(dt, K, n, rows, threads=cores, which=ref):
        w = synth.make_weight(dt, K, n, next(seeds))
        x = synth.make_activation(rows, K, next(seeds))
        t0 = time.perf_counter()
        gfo.gemv(dt, w, x, n, threads=threads, which=which)
        return time.perf_counter() - t0

    def figure(seconds, sample):
        return {"us": round(seconds * 1e6, 1), "cores": cores, "kind": kind, "sample": sample}

    print("bench: cpu baseline, config 1 (one block in full, twice)", file=sys.stderr, flush=True)
    shapes = list(zip(T.dtypes, T.proj_shapes()))
    repeats = 2
    block_s = sum(gemv_seconds(dt, K, N, 2) for _ in range(repeats) for dt, (K, N) in shapes) / repeats
    print("bench: cpu baseline, configs 0, 3, 2", file=sys.stderr, flush=True)
    gate_dt, (gK, gN) = shapes[4]
    config0_s = gemv_seconds(gate_dt, gK, gN, 1)
    # config 3: a 1/16 slice of the head's columns at 2 rows, then selection, law and acceptance on whole rows
    slice_n = T.vocab // 16
    head_s = gemv_seconds(T.embed_dtype, T.hidden, slice_n, 2) * (T.vocab / slice_n)
    rng = np.random.default_rng(3)
    p_logits = rng.normal(0, 2, (2, T.vocab)).astype(np.float32)
    q_logits = rng.normal(0, 2, T.vocab).astype(np.float32)
    opt = gfo.SamplerOptions(1.0, 64, 0.95, 0.0, 1.0)
    t0 = time.perf_counter()
    r0, r1 = gfo.select_candidates(p_logits[0], 64), gfo.select_candidates(p_logits[1], 64)
    rc, law = gfo.draft_law_compact(q_logits, opt)
    word, ua, ur, un = gfo.step_draws(0, 0)
    proposal = gfo.lib().gfo_draft_select(C.byref(law), C.c_uint32(word))
    gfo.spec_accept(r0, r1, law, proposal, opt, ua, ur, un)
    sampling_s = time.perf_counter() - t0
    # config 2: one drafter block in full at 1 row, its head on a 1/16 slice, scaled by weight count
    d_shapes = list(zip(D.dtypes, D.proj_shapes()))
    d_block_s = sum(gemv_seconds(dt, K, N, 1) for dt, (K, N) in d_shapes)
    d_head_s = gemv_seconds(D.embed_dtype, D.hidden, D.vocab // 16, 1) * 16
    drafter_s = D.layers * d_block_s + d_head_s
    step_s = T.layers * block_s + head_s + sampling_s + drafter_s
    spent = repeats * block_s + config0_s + head_s / 16 + sampling_s + d_block_s + d_head_s / 16

    # the same rows spread over the host's cores (rows of W are independent; a row's arithmetic is
    # unchanged): the oracle's threaded row dot on one block's GEMVs
    many = min(os.cpu_count() or 1, 16)
    par_s = sum(gemv_seconds(dt, K, N, 2, threads=many, which=None) for dt, (K, N) in shapes)
    layer_weights = sum(K * N for _, (K, N) in shapes)
    step_weights = (T.layers * layer_weights + T.hidden * T.vocab
                    + 0.5 * (D.layers * sum(K * N for K, N in D.proj_shapes()) + D.hidden * D.vocab))  # drafter: 1 row
    return {
        "value": round(step_s * 1e6, 1), "unit": "us", "cores": cores, "kind": kind,
        "sample": "%.1f s of CPU work: one 12B block's 7 GEMVs at 2 rows in full (x%d), the gate GEMV at 1 row, 1/16 of the "
                  "head's columns at 2 rows, selection + law + acceptance on whole rows, one drafter block and 1/16 of its head "
                  "at 1 row; step = 48 blocks + head + sampling + 18 drafter blocks + drafter head; %s" % (spent, repeats, how),
        "all_cores": {"value": round(par_s / layer_weights * step_weights * 1e6, 1), "unit": "us", "cores": many,
                      "kind": "port", "sample": "one 12B block's 7 GEMVs at 2 rows (%.2f s), oracle row dots on %d threads, "
                                                "scaled to the step's weight count" % (par_s, many)},
        "configs": {
            "0": figure(config0_s, "the whole 3840 -> 15360 Q4_K GEMV at 1 row; " + how),
            "1": figure(block_s, "the block's 7 GEMVs at 2 rows in full, mean of %d; %s" % (repeats, how)),
            "2": figure(drafter_s, "one drafter block's 7 Q8_0 GEMVs at 1 row in full x 18, plus 1/16 of the head's columns x 16 "
                                   "(by weight count; no attention or argmax); reference Q8_0 block decode, single thread"
                        if ref is not None else "by weight count; " + how),
            "3": figure(head_s + sampling_s, "1/16 of the Q6_K head's columns at 2 rows x 16 (%.2f s scaled), plus the oracle's "
                                             "top-64 selection of 2 rows, compact law and acceptance on whole rows (%.3f s); %s"
                        % (head_s, sampling_s, how)),
        },
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
    # mfma_frac counts the algorithmic flops (2 per weight and token); every MAC is issued twice on the f16 matrix
    # pipe (fp16 hi and lo halves of the activation), which mfma_frac_issued counts
    return {"tokens": tokens, "ms": round(ms, 2), "tokens_per_s": round(tokens / ms * 1e3, 1),
            "model_tflops": round(2 * macs / ms / 1e9, 1), "bound": "mfma",
            "mfma_frac": round(2 * macs / (ms * 1e-3) / 2.5e15, 4),
            "mfma_frac_issued": round(2 * 2 * macs / (ms * 1e-3) / 2.5e15, 4), "peak": "2.5 PFLOP/s f16 dense",
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

    # the same step once more as a recorded chain (the library's own command buffer: AQL packets on its own queue);
    # wall time per replay and the device's own clock between the first and the last packet
    chain = hip.Chain()
    with chain:
        plan.step(0)
    for _ in range(2):
        chain.launch()
        chain.wait()
    chain_steps = min(args.steps, 20)
    t0 = time.perf_counter()
    device_ns = 0
    for _ in range(chain_steps):
        chain.launch()
        chain.wait()
        device_ns += chain.gpu_ns()
    chain_us = (time.perf_counter() - t0) * 1e6 / chain_steps
    chained = plan.read_result()
    if (chained["accepted"], chained["token"], chained["next_root"]) != (first["accepted"], first["token"], first["next_root"]):
        raise RuntimeError("chain replay changed the step's decision")
    chain_figure = {"launches": chain.launches(), "replays": chain_steps, "us_per_replay_wall": round(chain_us, 1),
                    "us_per_replay_device": round(device_ns / chain_steps / 1e3, 1)}
    chain.close()

    # ---- rooflines: the dominant kernel (fused 2-row Q4_K gate+up GEMV + GeGLU, one launch per block), then the
    # local layers' attention and the down projection -----
    import ctypes as C
    from guffin_amd import synth
    H, F, QW, KW = T.hidden, T.ffn, T.q_width, T.kv_width
    x = torch.randn(2, H, device="cuda")
    xs = hip.group_sums(x)
    h_out = torch.empty(2, F, device="cuda")
    h_sums = hip._receipt(2, F, "cuda")
    lib = hip.lib()
    every = list(range(T.layers))

    def gateup(l):
        L = target.layers[l]
        # (ctypes passes a bare Python int as a 32-bit C int: pointers must be wrapped)
        hip.check(lib.guffin_hip_gateup_geglu(hip._stream(), int(L.dtype[4]), C.c_void_p(L.tiles[4]), C.c_void_p(L.tiles[5]),
                                              hip._p(x), hip._p(xs), hip._p(h_out), hip._p(h_sums), 2, H, F))

    print("bench: timing the gate+up kernel", file=sys.stderr, flush=True)
    # weights once, activation rows in (fp32 rows are the operator's input; the kernel reads their receipt), h out
    gateup_bytes = 2 * synth.weight_bytes(T.dtypes[4], H, F) + 2 * H * 4 + 2 * F * 4
    roofline = kernel_roofline("gateup_geglu_kernel<Q4_K, 2> (Q4_K gate+up GEMV + GeGLU, 2 rows, K=3840, N=2x15360)",
                               gateup, every, gateup_bytes, "gateup_geglu_kernel<Q4_K, 2>")

    print("bench: timing the down kernel", file=sys.stderr, flush=True)
    xh = torch.randn(2, F, device="cuda")
    xhs = hip.group_sums(xh)
    down_dt = int(T.dtypes[6])
    down_slices = hip.gemv_packed_slices(down_dt, F, H)
    down_parts = torch.empty((down_slices, 2, H), device="cuda")

    def down(l):
        hip.check(lib.guffin_hip_gemv_packed(hip._stream(), down_dt, C.c_void_p(target.layers[l].tiles[6]), hip._p(xh), hip._p(xhs),
                                             hip._p(down_parts), None, 2, F, H))

    down_bytes = synth.weight_bytes(down_dt, F, H) + 2 * F * 4 + down_slices * 2 * H * 4
    down_line = kernel_roofline("gemv_q6k_single_kernel<2> (Q6_K down GEMV, 2 rows, K=15360, N=3840, %d partial planes out)"
                                % down_slices, down, [l for l in every if int(target.layers[l].dtype[6]) == down_dt],
                                down_bytes, "gemv_q6k_single_kernel<2>")

    print("bench: timing the q/k/v and o projections", file=sys.stderr, flush=True)
    qkv_dt = [int(d) for d in T.dtypes[:3]]
    qkv_n = [QW, KW, KW]
    c_dt, c_n = (C.c_int * 3)(*qkv_dt), (C.c_uint32 * 3)(*qkv_n)
    lib.guffin_hip_gemv_packed_multi_slices.restype = C.c_uint32
    qkv_slices = int(lib.guffin_hip_gemv_packed_multi_slices(3, c_dt, c_n, H))
    if qkv_slices == 0:
        raise RuntimeError("q/k/v split: " + lib.guffin_hip_last_error().decode())
    qkv_parts = [torch.empty((qkv_slices, 2, n), device="cuda") for n in qkv_n]
    c_parts = (C.c_void_p * 3)(*[p.data_ptr() for p in qkv_parts])

    def qkv(l):
        L = target.layers[l]
        hip.check(lib.guffin_hip_gemv_packed_multi(hip._stream(), 3, c_dt, (C.c_void_p * 3)(*[L.tiles[i] for i in range(3)]), c_n,
                                                   c_parts, hip._p(x), hip._p(xs), 2, H))

    same_qkv = [l for l in every if [int(d) for d in target.layers[l].dtype[:3]] == qkv_dt]
    qkv_bytes = (sum(synth.weight_bytes(dt, H, n) for dt, n in zip(qkv_dt, qkv_n)) + 2 * H * 4
                 + qkv_slices * 2 * sum(qkv_n) * 4)
    qkv_line = kernel_roofline("gemv_packed_multi_kernel<2, 3, mixed> (q/k/v GEMVs of one block in one launch, 2 rows, K=3840, "
                               "N=4096+2048+2048, %d partial planes out)" % qkv_slices, qkv, same_qkv, qkv_bytes,
                               "gemv_packed_multi_kernel<2, 3, mixed>")
    xo = torch.randn(2, QW, device="cuda")
    xos = hip.group_sums(xo)
    o_dt = int(T.dtypes[3])
    o_slices = hip.gemv_packed_slices(o_dt, QW, H)
    o_parts = torch.empty((o_slices, 2, H), device="cuda")

    def o_proj(l):
        hip.check(lib.guffin_hip_gemv_packed(hip._stream(), o_dt, C.c_void_p(target.layers[l].tiles[3]), hip._p(xo), hip._p(xos),
                                             hip._p(o_parts), None, 2, QW, H))

    o_bytes = synth.weight_bytes(o_dt, QW, H) + 2 * QW * 4 + o_slices * 2 * H * 4
    o_line = kernel_roofline("gemv_packed_kernel<Q4_K, 2> (o projection, 2 rows, K=4096, N=3840, %d partial planes out)" % o_slices,
                             o_proj, [l for l in every if int(target.layers[l].dtype[3]) == o_dt], o_bytes,
                             "gemv_packed_kernel<Q4_K, 2> (o")

    print("bench: timing the local layers' attention", file=sys.stderr, flush=True)
    # as the step runs it on a local layer: head norms, rotation, fp16 narrowing and attention of 2 rows over the
    # 1024-token window in one launch, then the partition merge (its time is part of the figure, its bytes are not)
    locals_ = [l for l in every if T.is_local(l)]
    planes = 2
    q_raw, k_raw, v_raw = (0.1 * torch.randn(planes, 2, w, device="cuda") for w in (QW, KW, KW))
    q_norm, k_norm = torch.ones(T.head_dim, device="cuda"), torch.ones(T.head_dim, device="cuda")
    positions = torch.tensor([t_pos, t_pos + 1], dtype=torch.int32, device="cuda")
    table = hip.rope_table(positions, T.head_dim, T.local_base, 1.0)
    sched_rows = []
    for row in range(2):   # row r sees the last `window` positions up to its own: ring slots, then private rows
        pos = t_pos + row
        start = max(pos + 1 - T.sliding_window, 0)
        base_start = min(t_pos, start)
        first_private = max(start - t_pos, 0)
        sched_rows.append([base_start, t_pos - base_start, first_private, row + 1 - first_private])
    schedule = torch.tensor(sched_rows, dtype=torch.int32, device="cuda")
    ancestors = torch.arange(2, dtype=torch.int32, device="cuda")
    ring_tokens = max(r[0] + r[1] for r in sched_rows) - min(r[0] for r in sched_rows)

    def local_attention(l):
        hip.qkv_attention(q_raw, k_raw, v_raw, q_norm, k_norm, table, target.ring_k[l], target.ring_v[l], schedule, ancestors,
                          ring_tokens + 2, T.ring_local - 1, T.q_heads, T.kv_heads, T.head_dim, T.head_dim ** -0.5)

    # K and V rows of the window once per KV head, the projections' planes in, the attention rows out
    attention_bytes = ring_tokens * KW * 2 * 2 + planes * 2 * (QW + 2 * KW) * 4 + 2 * QW * 4
    attention_line = kernel_roofline("qkv attention of a local layer (2 rows, 16 query / 8 KV heads, %d-token window, fp16 K/V) "
                                     "with its partition merge" % ring_tokens, local_attention, locals_, attention_bytes,
                                     "attn_partial_kernel<2, 2, 256> (local layer")

    print("bench: timing the global layers' attention and the two heads", file=sys.stderr, flush=True)
    globals_ = [l for l in every if not T.is_local(l)]
    g_table = hip.rope_table(positions, T.head_dim, T.global_base, T.global_scale)
    g_schedule = torch.tensor([[0, t_pos, 0, row + 1] for row in range(2)], dtype=torch.int32, device="cuda")

    def global_attention(l):
        hip.qkv_attention(q_raw, k_raw, v_raw, q_norm, k_norm, g_table, target.ring_k[l], target.ring_v[l], g_schedule, ancestors,
                          t_pos + 2, T.ring_global - 1, T.q_heads, T.kv_heads, T.head_dim, T.head_dim ** -0.5)

    g_attention_bytes = t_pos * KW * 2 * 2 + planes * 2 * (QW + 2 * KW) * 4 + 2 * QW * 4
    g_attention_line = kernel_roofline("qkv attention of a global layer (2 rows, 16 query / 8 KV heads, %d tokens, fp16 K/V) with its "
                                       "partition merge" % t_pos, global_attention, globals_, g_attention_bytes,
                                       "attn_partial_kernel<2, 2, 256> (global layer")
    # the two heads: one matrix each (far larger than the caches), so the graph launches it eight times over
    xt = torch.randn(2, H, device="cuda")
    xts = hip.group_sums(xt)
    t_logits = torch.empty(2, T.vocab, device="cuda")
    head_dt = int(T.embed_dtype)
    t_parts = torch.empty((hip.gemv_packed_slices(head_dt, H, T.vocab), 2, T.vocab), device="cuda")
    t_head_line = kernel_roofline("gemv_packed_kernel<Q6_K, 2> (target head, 262144 x 3840, 2 rows)",
                                  lambda l: hip.check(lib.guffin_hip_gemv_packed(hip._stream(), head_dt, hip._p(target.head_tiles), hip._p(xt),
                                                                                 hip._p(xts), hip._p(t_parts), hip._p(t_logits), 2, H, T.vocab)),
                                  [0] * 8, T.head_bytes() + 2 * H * 4 + 2 * T.vocab * 4, "gemv_packed_kernel<Q6_K, 2> (target head")
    xd = torch.randn(1, D.hidden, device="cuda")
    xds = hip.group_sums(xd)
    d_logits = torch.empty(1, D.vocab, device="cuda")
    d_head_dt = int(D.embed_dtype)
    d_parts = torch.empty((hip.gemv_packed_slices(d_head_dt, D.hidden, D.vocab), 1, D.vocab), device="cuda")
    d_head_line = kernel_roofline("gemv_packed_kernel<Q8_0, 1> (drafter head, 262144 x 640, 1 row)",
                                  lambda l: hip.check(lib.guffin_hip_gemv_packed(hip._stream(), d_head_dt, hip._p(drafter.head_tiles), hip._p(xd),
                                                                                 hip._p(xds), hip._p(d_parts), hip._p(d_logits), 1, D.hidden, D.vocab)),
                                  [0] * 8, D.head_bytes() + D.hidden * 4 + D.vocab * 4, "gemv_packed_kernel<Q8_0, 1> (drafter head")

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
        "roofline": roofline,
        "rooflines": [attention_line, g_attention_line, down_line, qkv_line, o_line, t_head_line, d_head_line],
        "chain": chain_figure,
    }
    line["configs"] = config_figures(target, drafter, T, D, d_pos)
    if not args.no_prefill:
        line["prefill"] = prefill_figure(target, T)
    if not args.no_cpu_baseline:
        line["cpu_baseline"] = cpu_baseline(T, D)
        for key, figure in line["cpu_baseline"].pop("configs").items():
            line["configs"][key]["cpu_baseline"] = figure
    print(json.dumps(line))


if __name__ == "__main__":
    main()
