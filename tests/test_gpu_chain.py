"""Recorded launch chains (guffin_hip_chain_*): a cycle recorded once and replayed as AQL packets on the library's
own queue gives the results of the same calls made directly, bit for bit, on every replay; the replay's device time
is reported; calls out of order are refused."""
import ctypes as C
from dataclasses import replace

import pytest

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def hip():
    from guffin_amd import hip as module
    module.init(0)
    return module


def snapshot(plan):
    import torch
    bufs = {k: v.clone() for k, v in plan.buffers().items() if v is not None}
    return bufs, plan.result.clone(), plan.t_pk.clone(), plan.t_pv.clone(), plan.d_pk.clone(), plan.d_pv.clone(), int(plan.status.item())


def equal(a, b):
    import torch
    if a[6] != b[6]:
        return False
    for x, y in zip(a[1:6], b[1:6]):
        if not torch.equal(x, y):
            return False
    return all(torch.equal(a[0][k].view(torch.uint8), b[0][k].view(torch.uint8)) for k in a[0])


@pytest.mark.parametrize("step", [0, 3])
def test_a_replayed_cycle_equals_the_direct_cycle(hip, step):
    import torch
    from guffin_amd import model
    T = replace(model.GEMMA3_12B, layers=7, vocab=16384, ring_global=2048)
    D = replace(model.GEMMA3_270M, layers=7, vocab=16384, ring_global=2048)
    pos = 1300
    target = model.DeviceModel.random(T, seed=3, position=pos)
    drafter = model.DeviceModel.random(D, seed=4, position=pos)
    plan = model.H1Plan(target, drafter, pos, pos, seed=5, publish=False)
    plan.root.fill_(123)
    plan.step(step)
    torch.cuda.synchronize()
    want = snapshot(plan)
    assert want[6] == 0
    chain = hip.Chain()
    with chain:
        plan.step(step)          # recorded, not run
    assert chain.launches() > 60
    for replay in range(3):
        plan.scratch.zero_(); plan.result.zero_(); plan.t_pk.zero_(); plan.t_pv.zero_()
        torch.cuda.synchronize()
        print("chain replay", step, replay, flush=True)
        chain.launch()
        chain.wait()
        assert equal(snapshot(plan), want)
        ns = chain.gpu_ns()
        assert 50_000 < ns < 50_000_000     # a seven-block cycle: tenths of a millisecond on the device
    chain.close()


def test_calls_out_of_order_are_refused(hip):
    import torch
    lib = hip.lib()
    handle, other = C.c_void_p(), C.c_void_p()
    stream = hip._stream()
    assert lib.guffin_hip_chain_begin(stream, C.byref(handle)) == 0
    assert lib.guffin_hip_chain_begin(stream, C.byref(other)) == -6          # one chain records at a time
    assert lib.guffin_hip_chain_launch(handle) == -6                         # not ended yet
    assert lib.guffin_hip_chain_end(handle) == -6                            # nothing was recorded
    assert lib.guffin_hip_chain_destroy(handle) == 0
    # launches on another stream are not recorded: they run
    x = torch.randn(2, 256, device="cuda")
    chain = hip.Chain()
    side = torch.cuda.Stream()
    with chain:
        with torch.cuda.stream(side):
            sums = hip.group_sums(x)      # runs on `side`
        hip.group_sums(x)                 # recorded
    side.synchronize()
    assert chain.launches() == 1
    assert float(sums.abs().sum()) > 0
    ns = C.c_uint64()
    assert lib.guffin_hip_chain_gpu_ns(chain.handle, C.byref(ns)) == -6      # no replay has run
    chain.close()


def test_a_kernel_that_spills_runs_in_a_chain(hip):
    """The canonical two-row Q4_K GEMV at four columns per wave keeps part of its state in scratch memory (a private
    segment of 96 bytes per lane); the library's queue gets that memory from the runtime on demand, as a stream's
    queue does."""
    import torch
    from guffin_amd import synth
    K, N = 4096, 8192
    w = torch.from_numpy(synth.make_weight(hip.Q4_K, K, N, seed=9)).cuda()
    x = torch.from_numpy(synth.make_activation(2, K, seed=10)).cuda()
    want = hip.gemv(hip.Q4_K, w, x, N)
    torch.cuda.synchronize()
    out = torch.zeros_like(want)
    chain = hip.Chain()
    with chain:
        hip.gemv(hip.Q4_K, w, x, N, out=out)
    assert chain.launches() == 1
    for replay in range(2):
        out.zero_()
        torch.cuda.synchronize()
        print("chain with a private segment, replay", replay, flush=True)
        chain.launch()
        chain.wait()
        assert torch.equal(out, want)
    chain.close()
