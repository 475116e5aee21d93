"""The reference's deterministic test operands restated as formulas (tests/support/tensor_test_support.cpp:264-427,
tests/tensor/gemma3_metal_tests.cpp:67-74): block streams in GGUF order (per output column, K / 256 blocks) and
activation patterns.  Packing follows the formats themselves (Q4_K: 6-bit scale / offset pairs in 12 bytes, 64
elements per 32 bytes with the first 32 in the low nibbles; Q6_K: low nibbles, then 2-bit highs, then 16 signed
scales, then d)."""
import numpy as np


def _q4k_blocks(d_bits, dmin_bits, scale, minimum, nibble):
    """scale, minimum: [blocks][8] in 0..63; nibble: [blocks][256] in 0..15 -> [blocks][144] bytes."""
    n = scale.shape[0]
    out = np.zeros((n, 144), np.uint8)
    out[:, 0:2] = np.array([d_bits], np.uint16).view(np.uint8)
    out[:, 2:4] = np.array([dmin_bits], np.uint16).view(np.uint8)
    sc, mn = scale.astype(np.uint8) & 63, minimum.astype(np.uint8) & 63
    out[:, 4:8] = sc[:, :4] | ((sc[:, 4:] & 0x30) << 2)
    out[:, 8:12] = mn[:, :4] | ((mn[:, 4:] & 0x30) << 2)
    out[:, 12:16] = (sc[:, 4:] & 15) | ((mn[:, 4:] & 15) << 4)
    q = nibble.astype(np.uint8).reshape(n, 4, 2, 32)
    out[:, 16:] = (q[:, :, 0, :] | (q[:, :, 1, :] << 4)).reshape(n, 128)
    return out


def _q6k_blocks(d_bits, scale, value):
    """scale: [blocks][16] int8; value: [blocks][256] in -32..31 -> [blocks][210] bytes."""
    n = scale.shape[0]
    out = np.zeros((n, 210), np.uint8)
    enc = (value.astype(np.int16) + 32).astype(np.uint8).reshape(n, 2, 4, 32)     # half block, run of 32, lane
    low, high = enc & 15, enc >> 4
    ql = np.zeros((n, 2, 2, 32), np.uint8)
    ql[:, :, 0, :] = low[:, :, 0, :] | (low[:, :, 2, :] << 4)
    ql[:, :, 1, :] = low[:, :, 1, :] | (low[:, :, 3, :] << 4)
    out[:, :128] = ql.reshape(n, 128)
    qh = high[:, :, 0, :] | (high[:, :, 1, :] << 2) | (high[:, :, 2, :] << 4) | (high[:, :, 3, :] << 6)
    out[:, 128:192] = qh.reshape(n, 64)
    out[:, 192:208] = scale.astype(np.int8).view(np.uint8)
    out[:, 208:210] = np.array([d_bits], np.uint16).view(np.uint8)
    return out


def _grid(shared, columns):
    nblk = shared // 256
    column = np.repeat(np.arange(columns, dtype=np.int64), nblk)[:, None]
    block = np.tile(np.arange(nblk, dtype=np.int64), columns)[:, None]
    return column, block


def q4k_stress(shared, columns, seed):
    """tensor_q4_k_stress_gguf_weight_matrix: d = 0.125, dmin = 0.03125, scales and offsets over all of 1..63."""
    column, block = _grid(shared, columns)
    group, element = np.arange(8)[None, :], np.arange(256)[None, :]
    scale = 1 + (seed + 17 * column + 11 * block + 9 * group) % 63
    minimum = 1 + (seed + 13 * column + 7 * block + 15 * group) % 63
    nibble = (seed + 3 * column + 5 * block + 7 * element) % 16
    return _q4k_blocks(0x3000, 0x2800, scale, minimum, nibble).reshape(-1)


def q6k_stress(shared, columns, seed):
    """tensor_q6_k_stress_gguf_weight_matrix: d = 0.03125, signed scales over -31..31 (0 -> -17), all 64 quants."""
    column, block = _grid(shared, columns)
    group, element = np.arange(16)[None, :], np.arange(256)[None, :]
    raw = (seed + 11 * column + 7 * block + 13 * group) % 63 - 31
    scale = np.where(raw == 0, -17, raw)
    value = (seed + 5 * column + 3 * block + 17 * element) % 64 - 32
    return _q6k_blocks(0x2800, scale, value).reshape(-1)


def q4k_plain(shared, columns, seed):
    """tensor_q4_k_gguf_weight_matrix: d = 1, no offsets, scales 1..5."""
    column, block = _grid(shared, columns)
    group, element = np.arange(8)[None, :], np.arange(256)[None, :]
    scale = 1 + (seed + column + block + group) % 5
    nibble = (seed + column + 3 * block + 5 * element) % 16
    return _q4k_blocks(0x3C00, 0x0000, scale, np.zeros_like(scale), nibble).reshape(-1)


def q6k_plain(shared, columns, seed):
    """tensor_q6_k_gguf_weight_matrix: d = 0.5, scales in {-3..3} with 0 -> 2, quants -15..15."""
    column, block = _grid(shared, columns)
    group, element = np.arange(16)[None, :], np.arange(256)[None, :]
    raw = (seed + column + block + group) % 7 - 3
    scale = np.where(raw == 0, 2, raw)
    value = (seed + column + 5 * block + 7 * element) % 31 - 15
    return _q6k_blocks(0x3800, scale, value).reshape(-1)


def projection_values(rows, columns):
    """tensor_f32_projection_values: ((7 i + 3) % 11 - 5) / 8."""
    i = np.arange(rows * columns, dtype=np.int64)
    return (((i * 7 + 3) % 11 - 5).astype(np.float32) * np.float32(0.125)).reshape(rows, columns)


def pattern(count, scale=0.15):
    """sin(0.071 (i % 8191)) scale + cos(0.027 (i % 997)) 0.37 scale, in float as the reference forms it."""
    i = np.arange(count, dtype=np.int64)
    scale = np.float32(scale)
    a = np.sin((i % 8191).astype(np.float32) * np.float32(0.071)).astype(np.float32) * scale
    b = np.cos((i % 997).astype(np.float32) * np.float32(0.027)).astype(np.float32) * scale * np.float32(0.37)
    return (a + b).astype(np.float32)


def q8_0_from_values(values):
    """quantize_f16_gguf_weight_q8_0 (src/tensor/quantization.cpp:634-676) of a [shared][columns] value table
    stored the way tensor_f16_gguf_matrix stores it (a column's `shared` halves contiguous): per 32 elements the
    scale is max|v| / 127 in float, kept as a half, and the quants are round-half-away(v / scale)."""
    shared, columns = values.shape
    v = values.astype(np.float16).astype(np.float32).T.reshape(columns, shared // 32, 32)
    scale = (np.abs(v).max(2) / np.float32(127.0)).astype(np.float32)
    inverse = np.where(scale == 0, np.float32(0), np.float32(1.0) / np.where(scale == 0, np.float32(1), scale)).astype(np.float32)
    scaled = (v * inverse[:, :, None]).astype(np.float32)
    quants = (np.sign(scaled) * np.floor(np.abs(scaled) + np.float32(0.5))).astype(np.int8)
    blocks = np.zeros((columns, shared // 32, 34), np.uint8)
    blocks[:, :, 0:2] = np.ascontiguousarray(scale.astype(np.float16)).view(np.uint8).reshape(columns, shared // 32, 2)
    blocks[:, :, 2:] = np.ascontiguousarray(quants).view(np.uint8)
    return blocks.reshape(-1)
