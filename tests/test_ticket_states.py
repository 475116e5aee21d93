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


def make_ticket(retain=64, scratch_bytes=1 << 34, **shape_changes):
    sh = replace(model.GEMMA3_12B, layers=6, vocab=2048, ring_global=2048, **shape_changes)
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


ROOT = 0xFFFFFFFF


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
    assert (t.state, t.rows, t.position, list(t.row_tokens)[:2]) == (model.TXN_ENCODED, 2, 100, [5, 6])
    assert list(t.parents)[:2] == [ROOT, 0] and list(t.depths)[:2] == [0, 1]
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
    wide, keep3 = make_ticket(retain=321)   # the selection keeps at most 320 candidates per row
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
    t.parents[0], t.parents[1] = ROOT, 0
    arr = tokens(*path) if path else tokens(0)
    assert lib.guffin_hip_ticket_provisional_commit(None, C.byref(t), arr, len(path)) == E_ARG
    assert t.state == model.TXN_COMPLETED and t.provisional_count == 0
    one, keep1 = make_ticket()
    one.state, one.rows = model.TXN_COMPLETED, 1
    assert lib.guffin_hip_ticket_provisional_commit(None, C.byref(one), tokens(0, 1), 2) == E_ARG   # row 1 was not in the pass


def test_trees_are_encoded_in_topological_order_and_paths_follow_parents():
    """A verify tree (VerifierTopologyDescriptor): one root, parents before children, at most 4 rows; a
    provisional commit takes a root-to-node path and nothing else."""
    lib = hip.lib()
    t, keep = make_ticket()
    enc = lambda toks, parents, position=100: lib.guffin_hip_ticket_encode_tree(C.byref(t), tokens(*toks), tokens(*parents), len(toks), position)
    assert enc((5, 6, 7), (ROOT, 0, 0)) == 0
    assert (t.state, t.rows, list(t.parents)[:3], list(t.depths)[:3]) == (model.TXN_ENCODED, 3, [ROOT, 0, 0], [0, 1, 1])
    assert lib.guffin_hip_ticket_discard(None, C.byref(t)) == 0
    assert enc((5, 6, 7, 8), (ROOT, 0, 1, 0)) == 0 and list(t.depths) == [0, 1, 2, 1]
    assert lib.guffin_hip_ticket_discard(None, C.byref(t)) == 0
    for parents in ((0, 0, 0), (ROOT, ROOT, 0), (ROOT, 1, 0), (ROOT, 0, 2), (ROOT, 0, 5)):
        assert enc((5, 6, 7), parents) == E_ARG and t.state == model.TXN_IDLE, parents
    assert enc((1, 2, 3, 4, 5), (ROOT, 0, 1, 2, 3)) == E_SHAPE                  # more rows than a ticket holds
    assert lib.guffin_hip_ticket_encode(C.byref(t), tokens(1, 2, 3), 3, 100) == E_SHAPE   # a chain pass has 1 or 2 rows
    assert enc((5, 6, 7), (ROOT, 0, 1), 2046) == E_CAPACITY                  # depth 2 at position 2046 of 2048
    assert enc((5, 6, 7), (ROOT, 0, 0), 2046) == 0                           # depth 1 fits
    t.state = model.TXN_COMPLETED
    for path in ((0, 1, 2), (2,), (0, 2, 1), (1, 2), (0, 3)):
        arr = tokens(*path)
        assert lib.guffin_hip_ticket_provisional_commit(None, C.byref(t), arr, len(path)) == E_ARG, path
    assert t.state == model.TXN_COMPLETED


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


def test_forward_entry_points_refuse_rows_beyond_the_ring_capacity():
    """forward_rows, prefill_rows and h1_step check what ticket_encode checks: the rows must fit the
    global rings, and a local ring must hold the window before a row (no GPU is reached)."""
    lib = hip.lib()
    t, (desc, layers) = make_ticket()
    fake = C.c_void_p(0x7F0000000000)
    big = C.c_uint64(1 << 40)
    args = lambda rows, position: (None, C.byref(desc), fake, rows, position, fake, big, fake, fake, fake, fake, fake)
    assert lib.guffin_hip_forward_rows(*args(2, 2047)) == E_CAPACITY
    assert lib.guffin_hip_forward_rows(*args(1, 2048)) == E_CAPACITY
    assert b"forward_rows" in lib.guffin_hip_last_error()
    assert lib.guffin_hip_prefill_rows(None, C.byref(desc), fake, 100, 1949, fake, big, fake, fake) == E_CAPACITY
    assert b"prefill_rows" in lib.guffin_hip_last_error()
    narrow, (ndesc, nlayers) = make_ticket(ring_local=512)   # window 1024 needs 1023 ring rows
    assert lib.guffin_hip_forward_rows(None, C.byref(ndesc), fake, 1, 0, fake, big, fake, fake, fake, fake, fake) == E_CAPACITY
    h1 = model.H1Desc()
    h1.target, h1.drafter = C.pointer(desc), C.pointer(desc)
    h1.target_position, h1.drafter_position, h1.top_k = 2047, 0, 64
    step = lambda: lib.guffin_hip_h1_step(None, C.byref(h1), fake, fake, big, fake, fake, fake, fake, fake, fake)
    assert step() == E_CAPACITY and b"verify rows" in lib.guffin_hip_last_error()
    h1.target_position, h1.drafter_position = 0, 2048
    assert step() == E_CAPACITY and b"drafter" in lib.guffin_hip_last_error()


@pytest.mark.parametrize("period", [0, 1])
def test_a_model_without_local_layers_is_global_in_the_ticket_as_in_the_forward_pass(period):
    """With a global period of 0 or 1 every layer is global (src/engine/model.cpp:607-610): the pass must
    fit the global rings whatever the local capacity says, and the arena is the forward pass's."""
    lib = hip.lib()
    lib.guffin_hip_ticket_scratch_bytes.restype = C.c_uint64
    lib.guffin_hip_forward_scratch_bytes.restype = C.c_uint64
    t, (desc, layers) = make_ticket(global_period=period, ring_local=16)
    assert lib.guffin_hip_ticket_encode(C.byref(t), tokens(1, 2), 2, 2046) == 0     # ring_local 16 is never used
    assert lib.guffin_hip_ticket_discard(None, C.byref(t)) == 0
    assert lib.guffin_hip_ticket_encode(C.byref(t), tokens(1, 2), 2, 2047) == E_CAPACITY
    # every layer attends the whole context: the forward arena grows with the position on all six layers
    assert lib.guffin_hip_forward_scratch_bytes(C.byref(desc), 2, 2000) > lib.guffin_hip_forward_scratch_bytes(C.byref(desc), 2, 10)
