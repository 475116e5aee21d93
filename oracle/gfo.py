"""ctypes binding of the CPU oracle (libgfo.so) and of the compiled reference
(_ref/libguffin_ref.so).  TEST INFRASTRUCTURE ONLY: imported by tests/,
__graft_entry__.smoke() and the cpu_baseline leg of bench.py, never by guffin_amd.
"""
import ctypes as C
import os
import subprocess

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
Q8_0, Q4_K, Q6_K = 0, 1, 2
BLOCK_BYTES = {Q8_0: 34, Q4_K: 144, Q6_K: 210}
BLOCK_ELEMS = {Q8_0: 32, Q4_K: 256, Q6_K: 256}

token_logit = np.dtype([("token", np.uint32), ("logit", np.float32)])
# one verify row's raw sampler history and its resolved form (364 and 272 bytes, the reference's layouts)
selection_row = np.dtype([("history_token_ids", np.uint32, 64), ("suffix_token_ids", np.uint32, 23),
                          ("history_head", np.uint32), ("history_length", np.uint32),
                          ("history_window_limit", np.uint32), ("suffix_count", np.uint32)])
resolved_row = np.dtype([("top_k", np.uint32), ("base_candidate_count", np.uint32), ("history_count", np.uint32),
                         ("reserved", np.uint32), ("history_token_ids", np.uint32, 64)])


class SamplerOptions(C.Structure):
    _fields_ = [("temperature", C.c_float), ("top_k", C.c_uint32), ("top_p", C.c_float),
                ("min_p", C.c_float), ("repetition_penalty", C.c_float)]


class Prepared(C.Structure):
    _fields_ = [("count", C.c_uint32), ("pad", C.c_uint32), ("total_sampling_weight", C.c_double),
                ("token", C.c_uint32 * 256), ("probability", C.c_double * 256),
                ("sampling_weight", C.c_double * 256)]


class DraftLaw(C.Structure):
    _fields_ = [("count", C.c_uint32), ("pad", C.c_uint32), ("ids", C.c_uint32 * 256),
                ("cdf", C.c_uint64 * 257)]


class SpecResult(C.Structure):
    _fields_ = [("accepted", C.c_uint32), ("token", C.c_uint32), ("next_root", C.c_uint32),
                ("status", C.c_uint32), ("acceptance_probability", C.c_double),
                ("residual_total", C.c_double), ("residual_count", C.c_uint32), ("pad", C.c_uint32)]


class ModelConfig(C.Structure):
    _fields_ = [(n, C.c_uint32) for n in
                ("hidden", "ffn", "q_heads", "kv_heads", "head_dim", "layers", "vocab",
                 "sliding_window", "global_period")] + \
               [(n, C.c_float) for n in ("local_base", "global_base", "global_scale", "eps")] + \
               [("ring_local", C.c_uint32), ("ring_global", C.c_uint32)]


class Layer(C.Structure):
    _fields_ = [("dtype", C.c_int * 7), ("w", C.c_void_p * 7), ("norm", C.c_void_p * 6),
                ("ring_k", C.c_void_p), ("ring_v", C.c_void_p)]


def build(force=False):
    """Compile libgfo.so (and the reference library when the checkout is present)."""
    if force or not os.path.exists(os.path.join(HERE, "libgfo.so")):
        subprocess.check_call(["make", "-C", HERE, "-j8"], stdout=subprocess.DEVNULL)


_lib = None
_ref = None


def _ptr(a):
    return a.ctypes.data_as(C.c_void_p) if a is not None else None


def lib():
    global _lib
    if _lib is None:
        build()
        _lib = C.CDLL(os.path.join(HERE, "libgfo.so"))
        _lib.gfo_f16_to_f32.restype = C.c_float
        _lib.gfo_f16_to_f32.argtypes = [C.c_uint16]
        _lib.gfo_f32_to_f16_rne.restype = C.c_uint16
        _lib.gfo_f32_to_f16_rne.argtypes = [C.c_float]
        _lib.gfo_exp_f32.restype = C.c_float
        _lib.gfo_exp_f32.argtypes = [C.c_float]
        _lib.gfo_argmax.restype = C.c_uint32
        _lib.gfo_draft_select.restype = C.c_uint32
        _lib.gfo_draft_select_full.restype = C.c_uint32
    return _lib


def ref():
    """The compiled reference, or None when oracle/_ref was not built."""
    global _ref
    if _ref is None:
        path = os.path.join(HERE, "_ref", "libguffin_ref.so")
        if not os.path.exists(path):
            return None
        _ref = C.CDLL(path)
        _ref.gfr_f16_to_f32.restype = C.c_float
        _ref.gfr_f16_to_f32.argtypes = [C.c_uint16]
        _ref.gfr_argmax.restype = C.c_uint32
        _ref.gfr_select_draft_token.restype = C.c_uint32
    return _ref


# ---- thin numpy wrappers -------------------------------------------------
def _u8(a):
    a = np.ascontiguousarray(a, dtype=np.uint8)
    return a


def dequant(dtype, blocks, which=None):
    blocks = _u8(blocks)
    n = blocks.size // BLOCK_BYTES[dtype]
    out = np.empty(n * BLOCK_ELEMS[dtype], np.float32)
    if which is None:
        lib().gfo_dequant(dtype, _ptr(blocks), C.c_uint64(n), _ptr(out))
    else:
        assert which.gfr_dequant(dtype, _ptr(blocks), C.c_uint64(n), _ptr(out)) == 0
    return out


def gemv(dtype, w, x, N, threads=1, as_written=False, which=None):
    w = _u8(w)
    x = np.ascontiguousarray(x, np.float32).reshape(-1, x.shape[-1])
    rows, K = x.shape
    assert w.size == N * (K // BLOCK_ELEMS[dtype]) * BLOCK_BYTES[dtype]
    y = np.empty((rows, N), np.float32)
    if which is not None:
        assert which.gfr_gemv(dtype, _ptr(w), _ptr(x), _ptr(y), rows, K, N) == 0
    elif as_written:
        lib().gfo_gemv_as_written(dtype, _ptr(w), _ptr(x), _ptr(y), rows, K, N)
    else:
        lib().gfo_gemv_mt(dtype, _ptr(w), _ptr(x), _ptr(y), rows, K, N, threads)
    return y


def rms_norm(x, gamma, eps=1e-6, residual=None):
    x = np.ascontiguousarray(x, np.float32)
    rows, width = x.reshape(-1, x.shape[-1]).shape
    y = np.empty_like(x)
    g = np.ascontiguousarray(gamma, np.float32)
    if residual is None:
        lib().gfo_rms_norm(_ptr(x), _ptr(g), _ptr(y), rows, width, C.c_float(eps))
    else:
        r = np.ascontiguousarray(residual, np.float32)
        lib().gfo_rms_norm_add(_ptr(x), _ptr(g), _ptr(r), _ptr(y), rows, width, C.c_float(eps))
    return y


def rope_neox(x, positions, heads, head_dim, rope_dim, base, scale=1.0):
    x = np.ascontiguousarray(x, np.float32)
    rows = x.shape[0]
    pos = np.ascontiguousarray(positions, np.uint32)
    y = np.empty_like(x)
    lib().gfo_rope_neox(_ptr(x), _ptr(y), _ptr(pos), rows, heads, head_dim, rope_dim,
                        C.c_float(base), C.c_float(scale))
    return y


def kv_store_f16(raw_k, raw_v, positions, heads, head_dim, rope_dim, base, scale=1.0):
    raw_k = np.ascontiguousarray(raw_k, np.float32)
    raw_v = np.ascontiguousarray(raw_v, np.float32)
    rows = raw_k.shape[0]
    pos = np.ascontiguousarray(positions, np.uint32)
    k = np.empty(raw_k.shape, np.uint16)
    v = np.empty(raw_v.shape, np.uint16)
    lib().gfo_kv_store_f16(_ptr(raw_k), _ptr(raw_v), _ptr(pos), _ptr(k), _ptr(v), rows, heads,
                           head_dim, rope_dim, C.c_float(base), C.c_float(scale))
    return k, v


def geglu(gate, up):
    gate = np.ascontiguousarray(gate, np.float32)
    up = np.ascontiguousarray(up, np.float32)
    out = np.empty_like(gate)
    lib().gfo_geglu(_ptr(gate), _ptr(up), _ptr(out), C.c_uint64(gate.size))
    return out


def embed(dtype, w, tokens, width, scale):
    w = _u8(w)
    tokens = np.ascontiguousarray(tokens, np.uint32)
    out = np.empty((tokens.size, width), np.float32)
    lib().gfo_embed(dtype, _ptr(w), _ptr(tokens), _ptr(out), tokens.size, width, C.c_float(scale))
    return out


def attention(q, ring_k, ring_v, priv_k, priv_v, schedule, ancestors, row_mask, q_heads, kv_heads,
              head_dim, scale):
    q = np.ascontiguousarray(q, np.float32)
    rows = q.shape[0]
    out = np.empty_like(q)
    sched = np.ascontiguousarray(schedule, np.uint32)
    anc = np.ascontiguousarray(ancestors, np.uint32)
    lib().gfo_attention(_ptr(q), _ptr(ring_k), _ptr(ring_v), _ptr(priv_k), _ptr(priv_v),
                        _ptr(sched), _ptr(anc), _ptr(out), rows, row_mask, q_heads, kv_heads,
                        head_dim, C.c_float(scale))
    return out


def select_candidates(logits, k, history=()):
    logits = np.ascontiguousarray(logits, np.float32)
    hist = np.ascontiguousarray(history, np.uint32)
    out = np.zeros(k + hist.size, token_logit)
    n = lib().gfo_select_candidates(_ptr(logits), logits.size, k, _ptr(hist), hist.size, _ptr(out))
    if n < 0:
        raise ValueError("non-finite selected logit")
    return out[:n]


def selection_request(raw, vocab, top_k, repetition_enabled=True):
    """raw: one selection_row record -> (resolved_row record, status bits)."""
    raw = np.ascontiguousarray(raw, selection_row).reshape(1)
    out = np.zeros(1, resolved_row)
    fn = lib().gfo_selection_request
    fn.restype = C.c_uint32
    status = fn(_ptr(raw), C.c_uint32(vocab), C.c_uint32(top_k), C.c_int(1 if repetition_enabled else 0), _ptr(out))
    return out[0], int(status)


def ref_selection_request(raw, top_k, repetition_enabled=True):
    """The compiled reference's make_token_selection_request; None where it throws."""
    raw = np.ascontiguousarray(raw, selection_row).reshape(1)
    out = np.zeros(1, resolved_row)
    rc = ref().gfr_selection_request(_ptr(raw), C.c_uint32(top_k), C.c_int(1 if repetition_enabled else 0), _ptr(out))
    return out[0] if rc == 0 else None


def prepare(cands, opt, history=(), which=None):
    cands = np.ascontiguousarray(cands, token_logit)
    hist = np.ascontiguousarray(history, np.uint32)
    out = Prepared()
    fn = lib().gfo_prepare_token_distribution if which is None else which.gfr_prepare_token_distribution
    rc = fn(_ptr(cands), cands.size, C.byref(opt), _ptr(hist), hist.size, C.byref(out))
    return rc, out


def draft_law_compact(logits, opt):
    logits = np.ascontiguousarray(logits, np.float32)
    law = DraftLaw()
    rc = lib().gfo_draft_law_compact(_ptr(logits), logits.size, C.byref(opt), C.byref(law))
    return rc, law


def draft_law_compact_mapped(logits, opt, draft_to_target):
    logits = np.ascontiguousarray(logits, np.float32)
    d2t = np.ascontiguousarray(draft_to_target, np.int32)
    law = DraftLaw()
    rc = lib().gfo_draft_law_compact_mapped(_ptr(logits), logits.size, C.byref(opt), _ptr(d2t), C.byref(law))
    return rc, law


def draft_law_full(logits, opt):
    logits = np.ascontiguousarray(logits, np.float32)
    cdf = np.zeros(logits.size + 1, np.uint64)
    rc = lib().gfo_draft_law_full(_ptr(logits), logits.size, C.byref(opt), _ptr(cdf))
    return rc, cdf


def spec_accept(row0, row1, law, proposal, opt, u_accept, u_residual, u_next, which=None):
    row0 = np.ascontiguousarray(row0, token_logit)
    row1 = np.ascontiguousarray(row1, token_logit)
    out = SpecResult()
    fn = lib().gfo_spec_accept if which is None else which.gfr_spec_accept
    rc = fn(_ptr(row0), row0.size, _ptr(row1), row1.size, C.byref(law), C.c_uint32(proposal),
            C.byref(opt), C.c_double(u_accept), C.c_double(u_residual), C.c_double(u_next),
            C.byref(out))
    return rc, out


def spec_accept_history(row0, hist0, row1, hist1, law, proposal, opt, u_accept, u_residual, u_next):
    row0 = np.ascontiguousarray(row0, token_logit)
    row1 = np.ascontiguousarray(row1, token_logit)
    hist0 = np.ascontiguousarray(hist0, np.uint32)
    hist1 = np.ascontiguousarray(hist1, np.uint32)
    out = SpecResult()
    rc = lib().gfo_spec_accept_history(_ptr(row0), row0.size, _ptr(hist0), hist0.size, _ptr(row1), row1.size,
                                       _ptr(hist1), hist1.size, C.byref(law), C.c_uint32(proposal), C.byref(opt),
                                       C.c_double(u_accept), C.c_double(u_residual), C.c_double(u_next),
                                       C.byref(out))
    return rc, out


def spec_accept_mapped(row0, hist0, row1, hist1, law, target_to_draft, proposal, opt, u_accept, u_residual, u_next):
    row0 = np.ascontiguousarray(row0, token_logit)
    row1 = np.ascontiguousarray(row1, token_logit)
    hist0 = np.ascontiguousarray(hist0, np.uint32)
    hist1 = np.ascontiguousarray(hist1, np.uint32)
    t2d = np.ascontiguousarray(target_to_draft, np.int32)
    out = SpecResult()
    rc = lib().gfo_spec_accept_mapped(_ptr(row0), row0.size, _ptr(hist0), hist0.size, _ptr(row1), row1.size,
                                      _ptr(hist1), hist1.size, C.byref(law), _ptr(t2d), C.c_uint32(proposal),
                                      C.byref(opt), C.c_double(u_accept), C.c_double(u_residual), C.c_double(u_next),
                                      C.byref(out))
    return rc, out


def draft_law_full_mapped(logits, opt, draft_to_target):
    logits = np.ascontiguousarray(logits, np.float32)
    d2t = np.ascontiguousarray(draft_to_target, np.int32)
    cdf = np.zeros(logits.size + 1, np.uint64)
    rc = lib().gfo_draft_law_full_mapped(_ptr(logits), logits.size, C.byref(opt), _ptr(d2t), _ptr(cdf))
    return rc, cdf


def spec_accept_full_mapped(row0, row1, cdf, target_to_draft, proposal, opt, u_accept, u_residual, u_next):
    row0 = np.ascontiguousarray(row0, token_logit)
    row1 = np.ascontiguousarray(row1, token_logit)
    cdf = np.ascontiguousarray(cdf, np.uint64)
    t2d = np.ascontiguousarray(target_to_draft, np.int32)
    out = SpecResult()
    rc = lib().gfo_spec_accept_full_mapped(_ptr(row0), row0.size, _ptr(row1), row1.size, _ptr(cdf),
                                           C.c_uint32(cdf.size - 1), _ptr(t2d), C.c_uint32(proposal), C.byref(opt),
                                           C.c_double(u_accept), C.c_double(u_residual), C.c_double(u_next), C.byref(out))
    return rc, out


def spec_accept_full(row0, row1, cdf, proposal, opt, u_accept, u_residual, u_next):
    row0 = np.ascontiguousarray(row0, token_logit)
    row1 = np.ascontiguousarray(row1, token_logit)
    cdf = np.ascontiguousarray(cdf, np.uint64)
    out = SpecResult()
    rc = lib().gfo_spec_accept_full(_ptr(row0), row0.size, _ptr(row1), row1.size, _ptr(cdf),
                                    C.c_uint32(cdf.size - 1), C.c_uint32(proposal), C.byref(opt),
                                    C.c_double(u_accept), C.c_double(u_residual), C.c_double(u_next),
                                    C.byref(out))
    return rc, out


def draft_select_full(cdf, word):
    cdf = np.ascontiguousarray(cdf, np.uint64)
    lib().gfo_draft_select_full.restype = C.c_uint32
    return lib().gfo_draft_select_full(_ptr(cdf), C.c_uint32(cdf.size - 1), C.c_uint32(word))


def philox(counter, key):
    c = (C.c_uint32 * 4)(*counter)
    k = (C.c_uint32 * 2)(*key)
    o = (C.c_uint32 * 4)()
    lib().gfo_philox4x32_10(c, k, o)
    return list(o)


def step_draws(seed, step):
    w = C.c_uint32()
    a, r, n = C.c_double(), C.c_double(), C.c_double()
    lib().gfo_step_draws(C.c_uint64(seed), C.c_uint64(step), C.byref(w), C.byref(a), C.byref(r),
                         C.byref(n))
    return w.value, a.value, r.value, n.value


def model_config(host):
    """ModelConfig of a synthetic host model (any object with a `.shape` of the benchmark's Shape fields)."""
    sh = host.shape
    return ModelConfig(sh.hidden, sh.ffn, sh.q_heads, sh.kv_heads, sh.head_dim, sh.layers, sh.vocab,
                       sh.sliding_window, sh.global_period, sh.local_base, sh.global_base,
                       sh.global_scale, sh.eps, sh.ring_local, sh.ring_global)


def model_layers(host):
    """The host model's canonical weights, norms and rings as the oracle's Layer array (views, not copies)."""
    sh = host.shape
    arr = (Layer * sh.layers)()
    for l in range(sh.layers):
        for i in range(7):
            arr[l].dtype[i] = sh.dtypes_of(l)[i]
            arr[l].w[i] = host.w[l][i].ctypes.data
        for i in range(6):
            arr[l].norm[i] = host.norm[l][i].ctypes.data
        arr[l].ring_k = host.ring_k[l].ctypes.data
        arr[l].ring_v = host.ring_v[l].ctypes.data
    return arr


def forward(host, tokens, position, threads=8):
    """gfo_forward_rows on a host model: (output-normed rows, private K rows, private V rows)."""
    sh = host.shape
    rows = len(tokens)
    tok = np.asarray(tokens, np.uint32)
    pk = np.zeros((sh.layers, rows, sh.kv_width), np.uint16)
    pv = np.zeros_like(pk)
    out = np.zeros((rows, sh.hidden), np.float32)
    cfg = model_config(host)
    layers = model_layers(host)
    lib().gfo_forward_rows(C.byref(cfg), layers, sh.embed_dtype, host.embed.ctypes.data_as(C.c_void_p),
                           host.out_norm.ctypes.data_as(C.c_void_p), tok.ctypes.data_as(C.c_void_p),
                           rows, position, pk.ctypes.data_as(C.c_void_p), pv.ctypes.data_as(C.c_void_p),
                           out.ctypes.data_as(C.c_void_p), threads)
    return out, pk, pv


def correlating_map(q_logits, p_logits, protect, count=64):
    """A draft -> target vocabulary permutation (and its inverse) under which the drafter's `count` best
    tokens are the target's `count` best, rank by rank: two unrelated random models then propose tokens
    the target gives mass to, so a test sees accepted and rejected proposals.  `protect` (the root) keeps
    its id on both sides, so the drafter's input is what it was when q_logits were taken."""
    q_logits, p_logits = np.asarray(q_logits), np.asarray(p_logits)
    vocab = q_logits.size
    assert p_logits.size == vocab
    d2t = np.arange(vocab, dtype=np.int32)
    t2d = np.arange(vocab, dtype=np.int32)
    q_top = [int(t) for t in np.argsort(-q_logits, kind="stable") if t != protect][:count]
    p_top = [int(t) for t in np.argsort(-p_logits, kind="stable") if t != protect][:count]
    for a, b in zip(q_top, p_top):
        c, other = int(d2t[a]), int(t2d[b])   # a -> c and other -> b become a -> b and other -> c
        if other == protect or c == protect:
            continue
        d2t[a], d2t[other] = b, c
        t2d[b], t2d[c] = a, other
    assert d2t[protect] == protect and np.array_equal(d2t[t2d], np.arange(vocab))
    return d2t, t2d
