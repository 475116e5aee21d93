"""The resident pass hands its intermediate rows from CU to CU through memory that no cache invalidation covers:
what keeps a reader from seeing a stale line is that regions written in different phases never share a cache line
and that every block of a launch has a set of its own.  The layout the launch uses (guffin_hip_resident_layout is
the function resident_launch itself takes its addresses from) is held to that here, on the CPU, for every shape
the pass covers."""
import ctypes as C
from dataclasses import replace

import pytest

LINE = 128


def layout(lib, model, shape, rows, block_dtype):
    layers = (model.LayerDesc * shape.layers)()
    for l in range(shape.layers):
        for i in range(7):
            layers[l].dtype[i] = block_dtype
    desc = model.ModelDesc()
    desc.hidden, desc.ffn, desc.q_heads, desc.kv_heads, desc.head_dim = shape.hidden, shape.ffn, shape.q_heads, shape.kv_heads, shape.head_dim
    desc.layer_count, desc.vocab, desc.sliding_window, desc.global_period = shape.layers, shape.vocab, shape.sliding_window, shape.global_period
    desc.ring_local, desc.ring_global = shape.ring_local, shape.ring_global
    desc.layers = layers
    offsets, sizes = (C.c_uint64 * 8)(), (C.c_uint64 * 8)()
    set_bytes, sets, total = C.c_uint64(), C.c_uint32(), C.c_uint64()
    rc = lib.guffin_hip_resident_layout(C.byref(desc), rows, offsets, sizes, C.byref(set_bytes), C.byref(sets), C.byref(total))
    assert rc == 0, lib.guffin_hip_last_error()
    return list(offsets), list(sizes), set_bytes.value, sets.value, total.value


@pytest.mark.parametrize("which,rows", [("drafter", 1), ("drafter", 2), ("target", 1), ("target", 2)])
def test_exchange_regions_never_share_a_cache_line(which, rows):
    from guffin_amd import hip, model
    lib = hip.lib()
    lib.guffin_hip_last_error.restype = C.c_char_p
    base = model.GEMMA3_270M if which == "drafter" else model.GEMMA3_12B
    shapes = [base, replace(base, layers=7)]
    if which == "drafter":
        shapes.append(replace(base, hidden=512, ffn=1024))
    for shape in shapes:
        offsets, sizes, set_bytes, sets, total = layout(lib, model, shape, rows, model.Q8_0 if which == "drafter" else model.Q4_K)
        assert sets == 6 and all(size > 0 for size in sizes)
        assert offsets[0] == 0 and set_bytes % (2 * LINE) == 0
        for i in range(8):
            assert offsets[i] % (2 * LINE) == 0, "region %d starts inside a line pair" % i
            end = offsets[i] + sizes[i]
            assert end <= (offsets[i + 1] if i < 7 else set_bytes), "region %d runs into the next one" % i
        assert offsets[7] + sizes[7] == set_bytes, "the set is longer than its regions"
        # a set per block of a launch, then the barrier words; sets do not share a line either
        assert total >= sets * set_bytes and (total - sets * set_bytes) % (2 * LINE) == 0
        lines = set()
        for block in range(sets):
            for i in range(8):
                first = (block * set_bytes + offsets[i]) // LINE
                last = (block * set_bytes + offsets[i] + sizes[i] - 1) // LINE
                assert first not in lines and last not in lines
                lines.update((first, last))


def test_layout_refuses_what_it_is_not_made_for():
    from guffin_amd import hip, model
    lib = hip.lib()
    offsets, sizes = (C.c_uint64 * 8)(), (C.c_uint64 * 8)()
    a, b, c = C.c_uint64(), C.c_uint32(), C.c_uint64()
    assert lib.guffin_hip_resident_layout(None, 1, offsets, sizes, C.byref(a), C.byref(b), C.byref(c)) == -1
    desc = model.ModelDesc()
    layers = (model.LayerDesc * 1)()
    desc.layers = layers
    desc.hidden, desc.ffn, desc.q_heads, desc.kv_heads, desc.head_dim, desc.layer_count = 640, 2048, 4, 1, 256, 1
    assert lib.guffin_hip_resident_layout(C.byref(desc), 3, offsets, sizes, C.byref(a), C.byref(b), C.byref(c)) == -1
    desc.q_heads = 3
    desc.kv_heads = 2
    assert lib.guffin_hip_resident_layout(C.byref(desc), 1, offsets, sizes, C.byref(a), C.byref(b), C.byref(c)) != 0
