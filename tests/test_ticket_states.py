"""Order and argument rules of the verify-pass ticket (guffin_hip_ticket_*), on the host alone.

The rules are the reference's (src/engine/target_verifier_runtime.cpp:447-688 and the destructor
:315-335): a call out of order is refused and changes nothing, a selected path must be one causal
path from the pass's root, a retained count cannot exceed what was provisionally committed, a
poisoned ticket accepts nothing.  None of these paths reaches the GPU.
"""
import ctypes as C
from dataclasses import replace

import pytest

from guffin_amd import hip, model

E_ARG, E_SHAPE, E_ALIGN, E_CAPACITY, E_STATE = -1, -2, -3, -4, -6


def make_ticket(retain=64, scratch_bytes=1 << 34):
    sh = replace(model.GEMMA3_12B, layers=6, vocab=2048, ring_global=2048)
    desc = model.ModelDesc()
    for name in ("hidden", "ffn", "q_heads", "kv_heads", "head_dim", "vocab", "sliding_window", "global_period",
                 "local_base", "global_base", "global_scale", "eps", "ring_local", "ring_global"):
        setattr(desc, name, getattr(sh, name))
    desc.layer_count = sh.layers
    desc.embed_dtype = desc.head_dtype = sh.embed_dtype
    layers = (model.LayerDesc * sh.layers)()
    for l in range(sh.layers):
        for i, dt in enumerate(sh.dtypes):
            layers[l].dtype[i] = dt
    desc.layers = C.cast(layers, C.POINTER(model.LayerDesc))
    fake = 0x7F0000000000   # never dereferenced on the paths below; 256-byte aligned
    desc.embed_rows = desc.head_tiles = desc.out_norm = fake
    t = model.VerifyTicketDesc()
    t.target = C.pointer(desc)
    for name in ("scratch", "priv_k", "priv_v", "backup_k", "backup_v", "tokens", "selected", "candidates", "status"):
        setattr(t, name, fake)
    t.scratch_bytes = scratch_bytes
    t.retain = retain
    t.state = model.TXN_IDLE
    return t, (desc, layers)


def tokens(*values):
    return (C.c_uint32 * len(values))(*values)


def test_calls_out_of_order_are_refused_and_change_nothing():
    lib = hip.lib()
    t, keep = make_ticket()
    assert lib.guffin_hip_ticket_submit(None, C.byref(t)) == E_STATE
    assert lib.guffin_hip_ticket_complete(None, C.byref(t), None) == E_STATE
    assert lib.guffin_hip_ticket_provisional_commit(None, C.byref(t), tokens(0), 1) == E_STATE
    assert lib.guffin_hip_ticket_finalize(None, C.byref(t), 0) == E_STATE
    assert t.state == model.TXN_IDLE
    assert lib.guffin_hip_ticket_discard(None, C.byref(t)) == 0      # an idle ticket has nothing to discard
    assert lib.guffin_hip_ticket_release(None, C.byref(t)) == 0
    assert lib.guffin_hip_ticket_encode(C.byref(t), tokens(5, 6), 2, 100) == 0
    assert (t.state, t.rows, t.position, list(t.row_tokens)) == (model.TXN_ENCODED, 2, 100, [5, 6])
    assert lib.guffin_hip_ticket_encode(C.byref(t), tokens(5, 6), 2, 100) == E_STATE   # one pass at a time
    assert lib.guffin_hip_ticket_complete(None, C.byref(t), None) == E_STATE
    assert lib.guffin_hip_ticket_provisional_commit(None, C.byref(t), tokens(0), 1) == E_STATE
    assert lib.guffin_hip_ticket_finalize(None, C.byref(t), 0) == E_STATE
    assert t.state == model.TXN_ENCODED
    assert lib.guffin_hip_ticket_discard(None, C.byref(t)) == 0 and t.state == model.TXN_IDLE
    assert lib.guffin_hip_ticket_encode(C.byref(t), tokens(9), 1, 0) == 0 and t.rows == 1
    assert lib.guffin_hip_ticket_release(None, C.byref(t)) == 0 and t.state == model.TXN_IDLE


def test_encode_checks_its_arguments():
    lib = hip.lib()
    lib.guffin_hip_ticket_scratch_bytes.restype = C.c_uint64
    t, keep = make_ticket()
    need = lib.guffin_hip_ticket_scratch_bytes(C.byref(t), 2046)
    assert need > 0 and need >= lib.guffin_hip_ticket_scratch_bytes(C.byref(t), 0)
    assert lib.guffin_hip_ticket_encode(C.byref(t), None, 2, 0) == E_ARG
    assert lib.guffin_hip_ticket_encode(C.byref(t), tokens(1, 2, 3), 0, 0) == E_SHAPE
    assert lib.guffin_hip_ticket_encode(C.byref(t), tokens(1, 2, 3), 3, 0) == E_SHAPE
    assert lib.guffin_hip_ticket_encode(C.byref(t), tokens(1, 2), 2, 2047) == E_CAPACITY   # row 1 would leave the ring
    assert lib.guffin_hip_ticket_encode(C.byref(t), tokens(1, 2), 2, 2046) == 0
    assert lib.guffin_hip_ticket_discard(None, C.byref(t)) == 0
    small, keep2 = make_ticket(scratch_bytes=need - 1)
    assert lib.guffin_hip_ticket_encode(C.byref(small), tokens(1, 2), 2, 2046) == E_CAPACITY
    wide, keep3 = make_ticket(retain=385)
    assert lib.guffin_hip_ticket_encode(C.byref(wide), tokens(1), 1, 0) == E_CAPACITY
    odd, keep4 = make_ticket()
    odd.scratch += 64
    assert lib.guffin_hip_ticket_encode(C.byref(odd), tokens(1), 1, 0) == E_ALIGN
    null, keep5 = make_ticket()
    null.backup_k = None
    assert lib.guffin_hip_ticket_encode(C.byref(null), tokens(1), 1, 0) == E_ARG
    assert all(x.state == model.TXN_IDLE for x in (t, small, wide, odd, null))
    assert b"ticket_encode" in lib.guffin_hip_last_error()


@pytest.mark.parametrize("path", [(1,), (0, 0), (1, 0), (0, 2), (0, 1, 1), ()])
def test_selected_path_must_be_one_causal_path(path):
    lib = hip.lib()
    t, keep = make_ticket()
    t.state, t.rows, t.position = model.TXN_COMPLETED, 2, 40   # as guffin_hip_ticket_complete leaves it
    arr = tokens(*path) if path else tokens(0)
    assert lib.guffin_hip_ticket_provisional_commit(None, C.byref(t), arr, len(path)) == E_ARG
    assert t.state == model.TXN_COMPLETED and t.provisional_count == 0
    one, keep1 = make_ticket()
    one.state, one.rows = model.TXN_COMPLETED, 1
    assert lib.guffin_hip_ticket_provisional_commit(None, C.byref(one), tokens(0, 1), 2) == E_ARG   # row 1 was not in the pass


def test_finalize_cannot_retain_an_uncommitted_row():
    lib = hip.lib()
    t, keep = make_ticket()
    t.state, t.rows, t.provisional_count = model.TXN_PROVISIONAL, 2, 1
    assert lib.guffin_hip_ticket_finalize(None, C.byref(t), 2) == E_ARG
    assert t.state == model.TXN_PROVISIONAL
    assert lib.guffin_hip_ticket_finalize(None, C.byref(t), 1) == 0 and t.state == model.TXN_IDLE   # nothing to restore


def test_a_poisoned_or_submitted_ticket_cannot_be_reused_or_discarded():
    lib = hip.lib()
    t, keep = make_ticket()
    t.state = model.TXN_POISONED
    assert lib.guffin_hip_ticket_encode(C.byref(t), tokens(1), 1, 0) == E_STATE
    assert lib.guffin_hip_ticket_discard(None, C.byref(t)) == E_STATE
    assert lib.guffin_hip_ticket_release(None, C.byref(t)) == 0 and t.state == model.TXN_POISONED
    s, keep2 = make_ticket()
    s.state, s.rows = model.TXN_SUBMITTED, 2
    assert lib.guffin_hip_ticket_discard(None, C.byref(s)) == E_STATE and s.state == model.TXN_SUBMITTED
    assert lib.guffin_hip_ticket_release(None, C.byref(s)) == 0 and s.state == model.TXN_POISONED   # work still in flight
    c, keep3 = make_ticket()
    c.state, c.rows = model.TXN_COMPLETED, 2
    assert lib.guffin_hip_ticket_release(None, C.byref(c)) == 0 and c.state == model.TXN_IDLE
