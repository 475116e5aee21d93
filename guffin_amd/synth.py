"""Seeded synthetic GGUF-block weights and activations of the benchmark shapes.

Weight matrices are [K inputs, N output columns] stored per output column: column n owns
the K/block contiguous blocks (reference: src/tensor/backends/cpu_backend.cpp:43-53).
Random bytes are a uniform law over every bit field of a block (6-bit scales/mins,
4/6-bit quants, int8 scales); only the fp16 super-scales are drawn as |N(0, 0.02)|.
"""
import numpy as np

Q8_0, Q4_K, Q6_K = 0, 1, 2
BLOCK_BYTES = {Q8_0: 34, Q4_K: 144, Q6_K: 210}
BLOCK_ELEMS = {Q8_0: 32, Q4_K: 256, Q6_K: 256}
DTYPE_NAME = {Q8_0: "q8_0", Q4_K: "q4_k", Q6_K: "q6_k"}


def weight_bytes(dtype, K, N):
    return N * (K // BLOCK_ELEMS[dtype]) * BLOCK_BYTES[dtype]


def _f16_abs_normal(rng, n, sigma):
    return np.abs(rng.normal(0.0, sigma, n)).astype(np.float16).view(np.uint16)


def make_blocks(dtype, n_blocks, seed, sigma=0.02):
    """n_blocks random blocks as a uint8 array [n_blocks, block_bytes]."""
    rng = np.random.Generator(np.random.PCG64(seed))
    bb = BLOCK_BYTES[dtype]
    raw = rng.integers(0, 256, size=(n_blocks, bb), dtype=np.uint8)
    if dtype == Q8_0:
        q = raw[:, 2:]
        q[q == 0x80] = 0x81  # int8 uniform on -127..127
        raw[:, 0:2] = _f16_abs_normal(rng, n_blocks, sigma).reshape(-1, 1).view(np.uint8)
    elif dtype == Q4_K:
        raw[:, 0:2] = _f16_abs_normal(rng, n_blocks, sigma).reshape(-1, 1).view(np.uint8)
        raw[:, 2:4] = _f16_abs_normal(rng, n_blocks, sigma).reshape(-1, 1).view(np.uint8)
    else:
        raw[:, 208:210] = _f16_abs_normal(rng, n_blocks, sigma).reshape(-1, 1).view(np.uint8)
    return raw


def make_weight(dtype, K, N, seed, sigma=0.02):
    """Quantised [K, N] weight as a flat uint8 array (column-major blocks)."""
    return make_blocks(dtype, N * (K // BLOCK_ELEMS[dtype]), seed, sigma).reshape(-1)


def make_activation(rows, K, seed, sigma=1.0):
    rng = np.random.Generator(np.random.PCG64(seed))
    return rng.normal(0.0, sigma, (rows, K)).astype(np.float32)


# ---- block field setters used to build closed-form blocks in tests -----------
def q4k_set_scale_min(block, group, scale, minimum):
    s = block[4:16]
    if group < 4:
        s[group] = (int(s[group]) & 0xC0) | (scale & 63)
        s[group + 4] = (int(s[group + 4]) & 0xC0) | (minimum & 63)
    else:
        s[group + 4] = (scale & 15) | ((minimum & 15) << 4)
        s[group - 4] = (int(s[group - 4]) & 0x3F) | ((scale >> 4) << 6)
        s[group] = (int(s[group]) & 0x3F) | ((minimum >> 4) << 6)


def q4k_set_nibble(block, element, value):
    i = 16 + (element // 64) * 32 + element % 32
    if element % 64 < 32:
        block[i] = (int(block[i]) & 0xF0) | (value & 15)
    else:
        block[i] = (int(block[i]) & 0x0F) | ((value & 15) << 4)


def q6k_set_value(block, element, value):
    q = (value + 32) & 63
    half, r = divmod(element, 128)
    lane = r % 32
    lo = half * 64 + ((r // 32) % 2) * 32 + lane
    if r < 64:
        block[lo] = (int(block[lo]) & 0xF0) | (q & 15)
    else:
        block[lo] = (int(block[lo]) & 0x0F) | ((q & 15) << 4)
    hi = 128 + half * 32 + lane
    shift = (r // 32) * 2
    block[hi] = (int(block[hi]) & (0xFF ^ (3 << shift))) | ((q >> 4) << shift)


def q6k_set_scale(block, group, value):
    block[192 + group] = value & 0xFF
