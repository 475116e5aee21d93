"""Raw sampler-history rows for the selection-request tests: the cases of the reference's
test_raw_history_suffixes_append_truncate_then_deduplicate (tests/engine/sampling_tests.cpp:232-291)
and the malformed rows its device resolver flags (src/tensor/backends/metal/metal_kernels.mm:2351-2358)."""
import numpy as np


def observe(tokens, limit):
    """The ring a sampler holds after observing `tokens` (TokenSampler::observe_tokens): a full window
    overwrites its oldest slot and moves the head.  Returns (slots[64], head, length)."""
    slots = np.zeros(64, np.uint32)
    head = length = 0
    if limit == 0:
        return slots, 0, 0
    for t in tokens:
        if length < limit:
            slots[(head + length) % limit] = t
            length += 1
        else:
            slots[head] = t
            head = (head + 1) % limit
    return slots, head, length


def raw_row(gfo, base, suffix, limit=64):
    row = np.zeros((), gfo.selection_row)
    slots, head, length = observe(base, limit)
    row["history_token_ids"] = slots
    row["history_head"], row["history_length"], row["history_window_limit"] = head, length, limit
    row["suffix_token_ids"][:len(suffix)] = suffix
    row["suffix_count"] = len(suffix)
    return row


def expected_unique(base, suffix, limit):
    """Append, keep the last `limit`, then drop later duplicates: what the reference's test states."""
    chronological = (list(base) + list(suffix))[-limit:] if limit else []
    unique = []
    for t in chronological:
        if t not in unique:
            unique.append(t)
    return unique


def reference_cases():
    """(base, suffix) of the reference's sweep: base lengths 0, 1, 63, 64, 65, every suffix length 0..23."""
    for base_length in (0, 1, 63, 64, 65):
        base = [(i * 7) % 19 for i in range(base_length)]
        for suffix_length in range(24):
            yield base, [(i * 5 + base_length) % 23 for i in range(suffix_length)]


def random_cases(seed, count, vocab):
    """Rows with wrapped heads, short windows and tokens that repeat."""
    rng = np.random.default_rng(seed)
    for _ in range(count):
        limit = int(rng.choice([0, 1, 2, 3, 7, 16, 33, 63, 64]))
        base = rng.integers(0, min(vocab, 40), int(rng.integers(0, 150))).tolist()
        suffix = rng.integers(0, min(vocab, 40), int(rng.integers(0, 24))).tolist()
        yield base, suffix, limit


def malformed_rows(gfo):
    rows = []
    r = raw_row(gfo, [1, 2, 3], []); r["history_window_limit"] = 65; rows.append(("window over 64", r))
    r = raw_row(gfo, [1, 2, 3], [], limit=2); r["history_length"] = 3; rows.append(("length over the window", r))
    r = raw_row(gfo, [1, 2, 3], [4]); r["suffix_count"] = 24; rows.append(("suffix over 23", r))
    r = raw_row(gfo, [], [4]); r["history_head"] = 1; rows.append(("head without history", r))
    r = raw_row(gfo, [1], [], limit=64); r["history_head"] = 64; rows.append(("head outside the window", r))
    return rows
