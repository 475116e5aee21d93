"""The reference's whole-target fixture restated (tests/engine/gemma3_target_runtime_tests.cpp:37-241 with the
geometry of tests/support/gemma3_target_test_support.hpp:22-56): a six-block Gemma 3 target, 256 wide, FFN 256,
2 query heads on 1 KV head of 256, window 8, block 5 global (base 1e6, scale 1/8), 32 tokens, Q4_K q/k/o/gate/up
and Q6_K v/down/embedding, every weight a dyadic number so that the packed blocks and an independently kept
dense copy agree exactly:

  f32 (norm) tensors    0.75 + (mix(seed + i) % 65) / 128
  Q4_K blocks           d = dmin = 2^-9, every group scale 1 and offset 8, quant = mix(seed + i) & 15 -> (q - 8) / 512
  Q6_K blocks           d = 2^-11, group scale (g % 3 + 1) (-1)^g, quant = mix(seed + i) & 63 -> (q - 32) scale / 2048

with seed the 32-bit FNV-1a hash of the tensor's GGUF name.  `Reference` evaluates the block graph from the dense
values (double sums, float between operators, K/V rounded to binary16 before a token's own attention, as the
fp16 cache does).  Tolerances of the reference's tests: logits 3e-4 + 3e-4 |e|; fp16 cache rows by the budget of
its close_f16_checkpoint_cache (see assert_cache_row).  The vocabulary is padded from 32 to 64 rows of zero blocks here (the
head works on tiles of 64 columns); tokens 32..63 are never used and their logits are ignored."""
import math
from dataclasses import replace

import numpy as np

WIDTH, LAYERS, VOCAB, PADDED_VOCAB, WINDOW = 256, 6, 32, 64, 8
TOKENS = (2, 7, 1, 19, 3, 11, 5, 13, 17, 29, 23, 0, 31)
MATRICES = ("attn_q", "attn_k", "attn_v", "attn_output", "ffn_gate", "ffn_up", "ffn_down")
OUTPUTS = (512, 256, 256, 256, 256, 256, 256)
INPUTS = (256, 256, 256, 512, 256, 256, 256)
Q6 = (False, False, True, False, False, False, True)
NORMS = ("attn_norm", "attn_q_norm", "attn_k_norm", "post_attention_norm", "ffn_norm", "post_ffw_norm")


def mix(value):
    value = np.asarray(value, np.uint64) & 0xFFFFFFFF
    value ^= value >> 16
    value = (value * 0x7feb352d) & 0xFFFFFFFF
    value ^= value >> 15
    value = (value * 0x846ca68b) & 0xFFFFFFFF
    return (value ^ (value >> 16)).astype(np.uint32)


def seed_of(name):
    seed = 2166136261
    for c in name.encode():
        seed = ((seed ^ c) * 16777619) & 0xFFFFFFFF
    return seed


def f32_tensor(name, count):
    return (0.75 + (mix(seed_of(name) + np.arange(count, dtype=np.uint64)) % 65).astype(np.float32) / 128.0).astype(np.float32)


def q4k_tensor(name, outputs, inputs):
    """(canonical bytes, dense [outputs][inputs])."""
    count = outputs * inputs
    quant = (mix(seed_of(name) + np.arange(count, dtype=np.uint64)) & 15).astype(np.uint8).reshape(-1, 256)
    blocks = np.zeros((count // 256, 144), np.uint8)
    blocks[:, 1] = 0x18
    blocks[:, 3] = 0x18
    blocks[:, 4:8] = 1
    blocks[:, 8:12] = 8
    blocks[:, 12:16] = 0x81
    for run in range(4):            # 64 elements per 32 bytes: the first 32 in the low nibbles, the next 32 in the high
        low, high = quant[:, 64 * run:64 * run + 32], quant[:, 64 * run + 32:64 * run + 64]
        blocks[:, 16 + 32 * run:16 + 32 * run + 32] = low | (high << 4)
    dense = ((quant.astype(np.int32) - 8) / 512.0).astype(np.float32).reshape(outputs, inputs)
    return blocks.reshape(-1), dense


def q6k_tensor(name, outputs, inputs):
    count = outputs * inputs
    quant = (mix(seed_of(name) + np.arange(count, dtype=np.uint64)) & 63).astype(np.uint8).reshape(-1, 256)
    blocks = np.zeros((count // 256, 210), np.uint8)
    blocks[:, 209] = 0x10
    group = np.arange(16)
    scale = ((group % 3) + 1) * np.where(group % 2 == 0, 1, -1)
    blocks[:, 192:208] = scale.astype(np.int8).view(np.uint8)
    i = np.arange(256)
    within = i % 128
    low_index = (i // 128) * 64 + ((within // 32) % 2) * 32 + within % 32
    low_shift = np.where(within < 64, 0, 4)
    high_index = 128 + (i // 128) * 32 + within % 32
    high_shift = 2 * (within // 32)
    for e in range(256):
        blocks[:, low_index[e]] |= ((quant[:, e] & 15) << np.uint8(low_shift[e])).astype(np.uint8)
        blocks[:, high_index[e]] |= ((quant[:, e] >> 4) << np.uint8(high_shift[e])).astype(np.uint8)
    dense = ((quant.astype(np.int32) - 32) * scale[i // 16] / 2048.0).astype(np.float32).reshape(outputs, inputs)
    return blocks.reshape(-1), dense


class Fixture:
    def __init__(self):
        self.dense, self.packed = {}, {}
        self.packed["token_embd.weight"], self.dense["token_embd.weight"] = q6k_tensor("token_embd.weight", VOCAB, WIDTH)
        self.dense["output_norm.weight"] = f32_tensor("output_norm.weight", WIDTH)
        for layer in range(LAYERS):
            prefix = "blk.%d." % layer
            for suffix in NORMS:
                self.dense[prefix + suffix + ".weight"] = f32_tensor(prefix + suffix + ".weight", WIDTH)
            for name, o, i, six in zip(MATRICES, OUTPUTS, INPUTS, Q6):
                full = prefix + name + ".weight"
                self.packed[full], self.dense[full] = (q6k_tensor if six else q4k_tensor)(full, o, i)

    def host_model(self, model, ring_global=32):
        """A guffin_amd.model.HostModel with these weights, empty caches, rings of 8 (local) and 32 (global) rows."""
        shape = model.Shape(WIDTH, 256, 2, 1, 256, LAYERS, PADDED_VOCAB, WINDOW, 6, 1e4, 1e6, 0.125, 8, ring_global)
        host = object.__new__(model.HostModel)
        host.shape = shape
        host.w, host.norm, host.ring_k, host.ring_v = [], [], [], []
        for layer in range(LAYERS):
            prefix = "blk.%d." % layer
            host.w.append([self.packed[prefix + name + ".weight"] for name in MATRICES])
            host.norm.append([self.dense[prefix + suffix + ".weight"] for suffix in NORMS])
            cap = shape.ring_local if shape.is_local(layer) else shape.ring_global
            host.ring_k.append(np.zeros((cap, 256), np.float16))
            host.ring_v.append(np.zeros((cap, 256), np.float16))
        pad = np.zeros((PADDED_VOCAB - VOCAB) * 210, np.uint8)
        host.embed = np.concatenate([self.packed["token_embd.weight"], pad])
        host.head = host.embed
        host.out_norm = self.dense["output_norm.weight"]
        return host


class Reference:
    """Token-by-token evaluation from the dense values; K/V rows are rounded to binary16 when they are made."""

    def __init__(self, fixture):
        self.f = fixture
        self.key = [[] for _ in range(LAYERS)]
        self.value = [[] for _ in range(LAYERS)]
        self.logits = []

    def matrix(self, name, x):
        return (self.f.dense[name].astype(np.float64) @ np.asarray(x, np.float32).astype(np.float64)).astype(np.float32)

    def norm(self, name, x):
        x = np.asarray(x, np.float32)
        scale = np.float32(1.0 / math.sqrt(float((x.astype(np.float64) ** 2).sum()) / x.size + 1e-6))
        return (x * scale * self.f.dense[name]).astype(np.float32)

    def append(self, token):
        position = len(self.logits)
        hidden = (np.float32(16.0) * self.f.dense["token_embd.weight"][token]).astype(np.float32)
        for layer in range(LAYERS):
            p = "blk.%d." % layer
            n = self.norm(p + "attn_norm.weight", hidden)
            q, k, v = (self.matrix(p + m + ".weight", n) for m in ("attn_q", "attn_k", "attn_v"))
            q = np.concatenate([self.norm(p + "attn_q_norm.weight", q[h * 256:(h + 1) * 256]) for h in range(2)])
            k = self.norm(p + "attn_k_norm.weight", k)
            local = layer != 5
            i = np.arange(128)
            angle = position * (1.0 if local else 0.125) * np.power(10000.0 if local else 1000000.0, -2.0 * i / 256.0)
            c, s = np.cos(angle), np.sin(angle)

            def rotate(vec):
                heads = vec.reshape(-1, 256)
                a, b = heads[:, :128].astype(np.float64), heads[:, 128:].astype(np.float64)
                return np.concatenate([(a * c - b * s).astype(np.float32), (a * s + b * c).astype(np.float32)], axis=1).reshape(-1)

            q, k = rotate(q), rotate(k)
            k, v = k.astype(np.float16).astype(np.float32), v.astype(np.float16).astype(np.float32)
            self.key[layer].append(k)
            self.value[layer].append(v)
            first = position - 7 if local and position >= 8 else 0
            K = np.stack(self.key[layer][first:position + 1]).astype(np.float64)
            V = np.stack(self.value[layer][first:position + 1]).astype(np.float64)
            attended = np.zeros(512, np.float32)
            for head in range(2):
                scores = K @ q[head * 256:(head + 1) * 256].astype(np.float64) / 16.0
                w = np.exp(scores - scores.max())
                attended[head * 256:(head + 1) * 256] = ((w @ V) / w.sum()).astype(np.float32)
            projected = self.norm(p + "post_attention_norm.weight", self.matrix(p + "attn_output.weight", attended))
            hidden = (hidden + projected).astype(np.float32)
            f_in = self.norm(p + "ffn_norm.weight", hidden)
            gate, up = self.matrix(p + "ffn_gate.weight", f_in), self.matrix(p + "ffn_up.weight", f_in)
            x = gate
            act = (np.float32(0.5) * x * (np.float32(1.0) + np.tanh(np.float32(0.7978845608028654)
                   * (x + np.float32(0.044715) * x * x * x))) * up).astype(np.float32)
            projected = self.norm(p + "post_ffw_norm.weight", self.matrix(p + "ffn_down.weight", act))
            hidden = (hidden + projected).astype(np.float32)
        self.logits.append(self.matrix("token_embd.weight", self.norm("output_norm.weight", hidden)))
        return self.logits[-1]


def assert_close(actual, expected, label, absolute=3e-4, relative=3e-4):
    actual, expected = np.asarray(actual, np.float32).reshape(-1), np.asarray(expected, np.float32).reshape(-1)
    error = np.abs(actual.astype(np.float64) - expected)
    assert np.all(np.isfinite(actual)) and np.all(error <= absolute + relative * np.abs(expected)), \
        (label, float((error / (absolute + relative * np.abs(expected))).max()))
    return float((error / (absolute + relative * np.abs(expected))).max())


def assert_cache_row(actual, expected, label):
    """The reference's budget for fp16 cache rows (close_f16_checkpoint_cache,
    tests/engine/gemma3_target_runtime_tests.cpp:258-307): two correct fp32 evaluations can round a component to
    different neighbours in binary16, and that one-ulp difference travels through the later blocks, so a row of 256
    is held to 5e-4 + (3e-4 + 2^-10) s with s its RMS for the row's RMS error, and s = max(|e|, RMS) per component."""
    actual, expected = np.asarray(actual, np.float64).reshape(-1), np.asarray(expected, np.float64).reshape(-1)
    assert actual.size == 256 and np.all(np.isfinite(actual))
    absolute, relative = 5e-4, 3e-4 + 2.0 ** -10
    rms = math.sqrt(float((expected ** 2).mean()))
    error = np.abs(actual - expected)
    assert math.sqrt(float((error ** 2).mean())) <= absolute + relative * rms, label
    assert np.all(error <= absolute + relative * np.maximum(np.abs(expected), rms)), \
        (label, float((error / (absolute + relative * np.maximum(np.abs(expected), rms))).max()))


def assert_cache(host_or_rows, reference, count, read):
    """Rows of the positions a layer still holds (the last 8 of a local layer) against the reference's;
    read(layer, position) -> (k row, v row) as float32."""
    for layer in range(LAYERS):
        first = count - 8 if layer != 5 and count > 8 else 0
        for position in range(first, count):
            k, v = read(layer, position)
            assert_cache_row(k, reference.key[layer][position], "block %d key %d" % (layer, position))
            assert_cache_row(v, reference.value[layer][position], "block %d value %d" % (layer, position))
