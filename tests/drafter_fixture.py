"""The reference's whole-drafter fixture restated (tests/engine/gemma3_draft_tests.cpp:31-162): the complete
270M geometry (640 wide, FFN 2048, 4 query heads on 1 KV head of 256, 18 blocks, 262144 tokens, Q8_0 throughout)
with weights simple enough for an independent scalar evaluation in double precision:

  norm weight of column j         1 + ((j % 7) - 3) / 64                    (every norm of every block, and the output norm)
  embedding / tied head (r, j)    (((17 r + 13 j) % 53) - 26) / 64          (int8 quants, block scale 1/64)
  projection m of any block       row r has one non-zero, 8 / 64 = 0.125, at column (7 r + 11 + 3 m) % inputs

so a projection is a gather scaled by 1/8 and the logits take 53 distinct values.  `host_model()` builds the
weights in the layout the oracle and the device binding consume; `Reference` is the closed form, evaluated in
double with the reference's rounding points (float between operators).  Tolerances of the reference's own test:
logits 0.03 + 0.001 |e|, cache rows 0.004 + 0.002 |e|."""
import math
from dataclasses import replace

import numpy as np

WIDTH, FF, VOCAB, LAYERS, HEAD = 640, 2048, 262144, 18, 256
TOKENS = (2, 9259, 12074, 108)
INPUTS = (WIDTH, WIDTH, WIDTH, 1024, WIDTH, WIDTH, FF)
OUTPUTS = (1024, 256, 256, WIDTH, FF, FF, WIDTH)


def norm_weight(width):
    j = np.arange(width)
    return (1.0 + ((j % 7) - 3) / 64.0).astype(np.float32)


def embedding_quants(rows, width):
    r = np.arange(rows, dtype=np.int64)[:, None]
    j = np.arange(width, dtype=np.int64)[None, :]
    return (((r * 17 + j * 13) % 53) - 26).astype(np.int8)


def q8_matrix(quants):
    """[outputs][inputs] int8 -> canonical Q8_0 bytes (per output: inputs / 32 blocks of {fp16 1/64, 32 int8})."""
    outputs, inputs = quants.shape
    blocks = np.zeros((outputs, inputs // 32, 34), np.uint8)
    blocks[:, :, 0:2] = np.array([1.0 / 64], np.float16).view(np.uint8)
    blocks[:, :, 2:] = quants.reshape(outputs, inputs // 32, 32).view(np.uint8)
    return blocks.reshape(-1)


def projection_quants(inputs, outputs, matrix):
    q = np.zeros((outputs, inputs), np.int8)
    r = np.arange(outputs)
    q[r, (r * 7 + 11 + matrix * 3) % inputs] = 8
    return q


def host_model(model, ring_global=1024):
    """A guffin_amd.model.HostModel with the fixture's weights and empty caches."""
    shape = replace(model.GEMMA3_270M, ring_global=ring_global)
    assert (shape.hidden, shape.ffn, shape.layers, shape.vocab, shape.sliding_window, shape.global_period) == \
        (WIDTH, FF, LAYERS, VOCAB, 512, 6)
    host = object.__new__(model.HostModel)
    host.shape = shape
    host.w, host.norm, host.ring_k, host.ring_v = [], [], [], []
    projections = [q8_matrix(projection_quants(i, o, m)) for m, (i, o) in enumerate(zip(INPUTS, OUTPUTS))]
    for l in range(LAYERS):
        host.w.append(list(projections))
        host.norm.append([norm_weight(w) for w in (WIDTH, HEAD, HEAD, WIDTH, WIDTH, WIDTH)])
        cap = shape.ring_local if shape.is_local(l) else shape.ring_global
        host.ring_k.append(np.zeros((cap, HEAD), np.float16))
        host.ring_v.append(np.zeros((cap, HEAD), np.float16))
    host.embed = q8_matrix(embedding_quants(VOCAB, WIDTH))
    host.head = host.embed
    host.out_norm = norm_weight(WIDTH)
    return host


class Reference:
    """The scalar evaluation: double inside an operator, float between operators."""

    def __init__(self):
        self.keys = [[] for _ in range(LAYERS)]
        self.values = [[] for _ in range(LAYERS)]
        self.hidden = None
        self.position = 0

    @staticmethod
    def norm(x, length):
        x = np.asarray(x, np.float32).reshape(-1, length).astype(np.float64)
        inv = 1.0 / np.sqrt((x * x).sum(-1, keepdims=True) / length + 1e-6)
        return (x * inv * norm_weight(length).astype(np.float64)).astype(np.float32).reshape(-1)

    @staticmethod
    def linear(x, outputs, matrix):
        r = np.arange(outputs)
        return (np.float32(0.125) * np.asarray(x, np.float32)[(r * 7 + 11 + matrix * 3) % len(x)]).astype(np.float32)

    def step(self, token, zero_prefix=False):
        """zero_prefix: every earlier position of the caches holds zero keys and values (the reference's
        seed_zero_cache_prefix_for_testing): their scores are 0, so the current token's weight is
        1 / (1 + n exp(-s)) over the n earlier positions in reach and the output that weight times its value."""
        j = np.arange(WIDTH, dtype=np.int64)
        emb = ((((token * 17 + j * 13) % 53) - 26) / 64.0).astype(np.float32)
        x = (emb * np.float32(math.sqrt(np.float32(WIDTH)))).astype(np.float32)
        pos = self.position
        for layer in range(LAYERS):
            n = self.norm(x, WIDTH)
            q = self.norm(self.linear(n, 1024, 0), HEAD)
            k = self.norm(self.linear(n, 256, 1), HEAD)
            v = self.linear(n, 256, 2)
            local = layer % 6 != 5
            jj = np.arange(128)
            angle = pos * np.power(10000.0 if local else 1000000.0, -jj / 128.0)
            c, s = np.cos(angle), np.sin(angle)

            def rotate(vec):
                heads = vec.reshape(-1, HEAD).astype(np.float64)
                one, two = heads[:, :128].copy(), heads[:, 128:].copy()
                heads[:, :128] = one * c - two * s
                heads[:, 128:] = one * s + two * c
                return heads.astype(np.float32).reshape(-1)

            q, k = rotate(q), rotate(k)
            self.keys[layer].append(k)
            self.values[layer].append(v)
            first = pos - 511 if local and pos >= 511 else 0
            attended = np.zeros(1024, np.float32)
            if zero_prefix:
                for head in range(4):
                    score = float(q[head * HEAD:(head + 1) * HEAD].astype(np.float64) @ k.astype(np.float64))
                    current = 1.0 / (1.0 + (pos - first) * math.exp(-score / 16.0))
                    attended[head * HEAD:(head + 1) * HEAD] = (current * v.astype(np.float64)).astype(np.float32)
            else:
                K = np.stack(self.keys[layer][first:pos + 1]).astype(np.float64)
                V = np.stack(self.values[layer][first:pos + 1]).astype(np.float64)
                for head in range(4):
                    scores = K @ q[head * HEAD:(head + 1) * HEAD].astype(np.float64) / 16.0
                    w = np.exp(scores - scores.max())
                    attended[head * HEAD:(head + 1) * HEAD] = ((w / w.sum()) @ V).astype(np.float32)
            x = x + self.norm(self.linear(attended, WIDTH, 3), WIDTH)
            nf = self.norm(x, WIDTH)
            gate = self.linear(nf, FF, 4).astype(np.float64)
            up = self.linear(nf, FF, 5)
            act = (0.5 * gate * (1.0 + np.tanh(math.sqrt(2.0 / math.pi) * (gate + 0.044715 * gate ** 3)))
                   * up.astype(np.float64)).astype(np.float32)
            x = x + self.norm(self.linear(act, WIDTH, 6), WIDTH)
        self.hidden = self.norm(x, WIDTH)
        self.position += 1

    def logits(self):
        distinct = embedding_quants(53, WIDTH).astype(np.float64) / 64.0 @ self.hidden.astype(np.float64)
        return distinct.astype(np.float32)[np.arange(VOCAB) % 53]


def assert_logits_close(actual, expected, label):
    error = np.abs(actual.astype(np.float64) - expected)
    assert np.all(np.isfinite(actual)) and np.all(error <= 0.03 + 0.001 * np.abs(expected)), (label, float(error.max()))
    return float(error.max())


def assert_cache_close(actual, expected, label):
    actual, expected = np.asarray(actual, np.float32).reshape(-1), np.asarray(expected, np.float32).reshape(-1)
    error = np.abs(actual - expected)
    assert np.all(np.isfinite(actual)) and np.all(error <= 0.004 + 0.002 * np.abs(expected)), (label, float(error.max()))
