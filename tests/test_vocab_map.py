"""The host check of a vocabulary map (guffin_vocab_map_invert) on the reference's refusals
(tests/engine/gemma3_draft_tests.cpp:498-508, src/engine/gemma3_draft.mm:655-675): no GPU call is made."""
import numpy as np
import pytest

from guffin_amd import hip


def test_identity_and_partial_maps_invert():
    t2d, mapped = hip.vocab_map_invert(np.arange(1000), 1000)
    assert mapped == 1000 and np.array_equal(t2d, np.arange(1000))
    d2t = np.full(1000, -1, np.int32)
    d2t[[3, 7, 999]] = [70000, 0, 5]
    t2d, mapped = hip.vocab_map_invert(d2t, 262144)
    assert mapped == 3 and t2d[70000] == 3 and t2d[0] == 7 and t2d[5] == 999 and int((t2d >= 0).sum()) == 3


@pytest.mark.parametrize("edit,reason", [
    (lambda m: m.__setitem__(1, m[0]), "not injective"),
    (lambda m: m.fill(-1), "intersection is empty"),
    (lambda m: m.__setitem__(5, 1000), "out of bounds"),
    (lambda m: m.__setitem__(5, -2), "out of bounds"),
])
def test_malformed_maps_are_refused(edit, reason):
    d2t = np.arange(1000, dtype=np.int32)
    edit(d2t)
    with pytest.raises(hip.GuffinError) as err:
        hip.vocab_map_invert(d2t, 1000)
    assert err.value.code == -1 and reason in str(err.value)
