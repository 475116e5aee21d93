"""ctypes binding of libguffin_hip.so over torch device tensors."""
import ctypes as C
import os

import torch

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libguffin_hip.so")

Q8_0, Q4_K, Q6_K = 0, 1, 2


class GuffinError(RuntimeError):
    def __init__(self, code, message):
        super().__init__("guffin_hip error %d: %s" % (code, message))
        self.code = code


_lib = None
_inited = set()


def lib():
    """Loads the built library; raises if it is missing (no fallback path exists)."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError(
                "%s is missing: build it with `python -m guffin_amd.build` "
                "(hipcc --offload-arch=gfx950); guffin_amd has no CPU fallback" % LIB_PATH)
        _lib = C.CDLL(LIB_PATH)
        _lib.guffin_hip_last_error.restype = C.c_char_p
        _lib.guffin_hip_arch.restype = C.c_char_p
    return _lib


def check(rc):
    if rc != 0:
        raise GuffinError(rc, lib().guffin_hip_last_error().decode())


def init(device=0):
    if device not in _inited:
        if not torch.cuda.is_available():
            raise RuntimeError("guffin_amd needs a gfx950 GPU; none is visible")
        check(lib().guffin_hip_init(device))
        _inited.add(device)


def set_forward_mode(mode):
    """0: resident pass where the model fits (default), 1: one launch per operator, 2: resident or an error."""
    check(lib().guffin_hip_set_forward_mode(mode))


def set_spin_limit(polls):
    """Bound of every wait inside the resident pass, in polls of a counter (default 2**20)."""
    check(lib().guffin_hip_set_spin_limit(C.c_uint32(polls)))



class Chain:
    """Recorded launches replayed as AQL packets (guffin_hip_chain_*).  Usage:
        chain = Chain()
        with chain:                 # every library call on the current stream is recorded, not run
            plan.step(0)
        chain.launch(); chain.wait()
    """

    def __init__(self):
        self.handle = C.c_void_p()
        self.stream = _stream()

    def __enter__(self):
        check(lib().guffin_hip_chain_begin(self.stream, C.byref(self.handle)))
        return self

    def __exit__(self, exc_type, exc, tb):
        if exc_type is not None:
            lib().guffin_hip_chain_destroy(self.handle)
            self.handle = C.c_void_p()
            return False
        check(lib().guffin_hip_chain_end(self.handle))
        return False

    def launch(self):
        check(lib().guffin_hip_chain_launch(self.handle))

    def wait(self):
        check(lib().guffin_hip_chain_wait(self.handle))

    def gpu_ns(self):
        ns = C.c_uint64()
        check(lib().guffin_hip_chain_gpu_ns(self.handle, C.byref(ns)))
        return ns.value

    def launches(self):
        n = C.c_uint32()
        check(lib().guffin_hip_chain_info(self.handle, C.byref(n)))
        return n.value

    def close(self):
        if self.handle:
            lib().guffin_hip_chain_destroy(self.handle)
            self.handle = C.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


def _stream():
    return C.c_void_p(torch.cuda.current_stream().cuda_stream)


def _p(t):
    return C.c_void_p(t.data_ptr()) if t is not None else C.c_void_p(0)


def dequant(dtype, blocks, n_blocks):
    elems = 32 if dtype == Q8_0 else 256
    out = torch.empty(n_blocks * elems, dtype=torch.float32, device=blocks.device)
    check(lib().guffin_hip_dequant(_stream(), dtype, _p(blocks), C.c_uint64(n_blocks), _p(out)))
    return out


def gemv(dtype, w, x, N, out=None):
    rows, K = x.shape
    if out is None:
        out = torch.empty((rows, N), dtype=torch.float32, device=x.device)
    check(lib().guffin_hip_gemv(_stream(), dtype, _p(w), _p(x), _p(out), rows, K, N))
    return out


def packed_bytes(dtype, K, N):
    lib().guffin_hip_packed_bytes.restype = C.c_uint64
    return lib().guffin_hip_packed_bytes(dtype, K, N)


def repack(dtype, canonical, K, N):
    tiles = torch.empty_like(canonical)
    check(lib().guffin_hip_repack(_stream(), dtype, _p(canonical), _p(tiles), K, N))
    return tiles


def unpack(dtype, tiles, K, N):
    canonical = torch.empty_like(tiles)
    check(lib().guffin_hip_unpack(_stream(), dtype, _p(tiles), _p(canonical), K, N))
    return canonical


def receipt_bytes(rows, K):
    lib().guffin_hip_receipt_bytes.restype = C.c_uint64
    n = lib().guffin_hip_receipt_bytes(rows, K)
    if n == 0:
        raise GuffinError(-2, "receipt: K must be a positive multiple of 32 and rows 1 or 2")
    return n


def _receipt(rows, K, device):
    """New receipt blob; the returned [rows, K/16 + K/32] view of its sums starts at the blob's first byte."""
    blob = torch.zeros(receipt_bytes(rows, K) // 4, dtype=torch.float32, device=device)
    n = K // 16 + K // 32
    return blob[:rows * n].view(rows, n)


def receipt_parts(sums, rows, K):
    """(mult [rows, K/32] float32, image [K/32, 4, 32] float16) of the receipt whose sums view is given."""
    n = K // 16 + K // 32
    nbytes = receipt_bytes(rows, K)
    blob = torch.empty(0, dtype=torch.uint8, device=sums.device).set_(sums.untyped_storage(), sums.storage_offset() * 4,
                                                                      (nbytes,), (1,))
    mult_off = (rows * n * 4 + 255) // 256 * 256
    img_off = (mult_off + rows * (K // 32) * 4 + 255) // 256 * 256
    mult = blob[mult_off:mult_off + rows * (K // 32) * 4].view(torch.float32).view(rows, K // 32)
    image = blob[img_off:img_off + (K // 32) * 256].view(torch.float16).view(K // 32, 4, 32)
    return mult, image


def group_sums(x, out=None):
    """Activation receipt of x (sums, multipliers, matrix-core image); returns its sums view."""
    rows, K = x.shape
    if out is None:
        out = _receipt(rows, K, x.device)
    check(lib().guffin_hip_group_sums(_stream(), _p(x), _p(out), rows, K))
    return out


def gemv_packed_slices(dtype, K, N):
    lib().guffin_hip_gemv_packed_slices.restype = C.c_uint32
    return lib().guffin_hip_gemv_packed_slices(dtype, K, N)


def gemv_packed(dtype, tiles, x, xsums, N, partials=None, out=None, reduce=True):
    rows, K = x.shape
    S = gemv_packed_slices(dtype, K, N)
    if partials is None:
        partials = torch.empty((S, rows, N), dtype=torch.float32, device=x.device)
    if reduce and out is None:
        out = torch.empty((rows, N), dtype=torch.float32, device=x.device)
    check(lib().guffin_hip_gemv_packed(_stream(), dtype, _p(tiles), _p(x), _p(xsums), _p(partials),
                                       _p(out) if reduce else C.c_void_p(0), rows, K, N))
    return out if reduce else partials


def gemv_packed_static(dtype, tiles, x, xsums, N, out):
    """guffin_hip_gemv_packed_static: the packed GEMV with its partial planes in the library's static
    device array; `out` is the caller's [rows, N] result."""
    rows, K = x.shape
    check(lib().guffin_hip_gemv_packed_static(_stream(), dtype, _p(tiles), _p(x), _p(xsums), _p(out), rows, K, N))
    return out


def _f32(shape, like):
    return torch.empty(shape, dtype=torch.float32, device=like.device)


def _planes(x, planes):
    """(planes, plane_stride) of a [planes, ...] tensor or a plain one."""
    if planes is None:
        return 1, 0
    return planes, x[0].numel()


def new_status(device="cuda"):
    return torch.zeros(1, dtype=torch.int32, device=device)


def rms_norm(x, gamma, eps=1e-6, residual=None, planes=None, want_sums=False, status=None):
    pl, stride = _planes(x, planes)
    shape = x.shape[1:] if planes else x.shape
    rows, width = shape
    y = _f32((rows, width), x)
    sums = _receipt(rows, width, x.device) if want_sums else None
    check(lib().guffin_hip_rms_norm(_stream(), _p(x), pl, C.c_uint64(stride), _p(gamma), _p(residual),
                                    _p(y), _p(sums), rows, width, C.c_float(eps), _p(status)))
    return (y, sums) if want_sums else y


def rms_norm_add_norm(x, gamma_post, residual, gamma_next, eps=1e-6, planes=None, want_sums=False, status=None):
    pl, stride = _planes(x, planes)
    shape = x.shape[1:] if planes else x.shape
    rows, width = shape
    out_res, out_norm = _f32((rows, width), x), _f32((rows, width), x)
    sums = _receipt(rows, width, x.device) if want_sums else None
    check(lib().guffin_hip_rms_norm_add_norm(_stream(), _p(x), pl, C.c_uint64(stride), _p(gamma_post),
                                             _p(residual), _p(out_res), _p(gamma_next), _p(out_norm), _p(sums),
                                             rows, width, C.c_float(eps), _p(status)))
    return out_res, out_norm, sums


def head_rms_norm(x, gamma, heads, head_dim, eps=1e-6):
    y = torch.empty_like(x)
    check(lib().guffin_hip_head_rms_norm(_stream(), _p(x), _p(gamma), _p(y), x.shape[0], heads, head_dim,
                                         C.c_float(eps)))
    return y


def rope_neox(x, positions, heads, head_dim, rope_dim, base, scale=1.0):
    y = torch.empty_like(x)
    check(lib().guffin_hip_rope_neox(_stream(), _p(x), _p(positions), _p(y), x.shape[0], heads, head_dim,
                                     rope_dim, C.c_float(base), C.c_float(scale)))
    return y


def kv_store_f16(raw_k, raw_v, positions, heads, head_dim, rope_dim, base, scale=1.0, status=None):
    k = torch.empty(raw_k.shape, dtype=torch.float16, device=raw_k.device)
    v = torch.empty(raw_v.shape, dtype=torch.float16, device=raw_v.device)
    check(lib().guffin_hip_kv_store_f16(_stream(), _p(raw_k), _p(raw_v), _p(positions), _p(k), _p(v),
                                        raw_k.shape[0], heads, head_dim, rope_dim, C.c_float(base),
                                        C.c_float(scale), _p(status)))
    return k, v


def qkv_post(q_raw, k_raw, v_raw, q_norm, k_norm, positions, rows, q_heads, kv_heads, head_dim, rope_dim, base,
             scale=1.0, eps=1e-6, planes=None, status=None, table=None):
    pl = planes or 1
    strides = [t[0].numel() if planes else 0 for t in (q_raw, k_raw, v_raw)]
    q = _f32((rows, q_heads * head_dim), q_raw)
    k = torch.empty((rows, kv_heads * head_dim), dtype=torch.float16, device=q_raw.device)
    v = torch.empty_like(k)
    check(lib().guffin_hip_qkv_post(_stream(), _p(q_raw), _p(k_raw), _p(v_raw), pl, pl, pl, C.c_uint64(strides[0]),
                                    C.c_uint64(strides[1]), C.c_uint64(strides[2]), _p(q_norm), _p(k_norm),
                                    _p(positions), _p(q), _p(k), _p(v), rows, q_heads, kv_heads, head_dim,
                                    rope_dim, C.c_float(base), C.c_float(scale), C.c_float(eps), _p(table),
                                    _p(status)))
    return q, k, v


def rope_table(positions, rope_dim, base, scale=1.0):
    rows = positions.numel()
    table = torch.empty((rows, rope_dim // 2, 2), dtype=torch.float32, device=positions.device)
    check(lib().guffin_hip_rope_table(_stream(), _p(positions), _p(table), rows, rope_dim, C.c_float(base),
                                      C.c_float(scale)))
    return table


def gemv_packed_multi(dtypes, tiles, x, xsums, Ns):
    """Several matrices over the same activation rows in one launch; returns one [S, rows, N_i] tensor each."""
    rows, K = x.shape
    count = len(dtypes)
    dt = (C.c_int * count)(*dtypes)
    n = (C.c_uint32 * count)(*Ns)
    lib().guffin_hip_gemv_packed_multi_slices.restype = C.c_uint32
    S = lib().guffin_hip_gemv_packed_multi_slices(count, dt, n, K)
    if S == 0:
        raise GuffinError(-2, lib().guffin_hip_last_error().decode())
    parts = [torch.empty((S, rows, N), dtype=torch.float32, device=x.device) for N in Ns]
    tl = (C.c_void_p * count)(*[t.data_ptr() for t in tiles])
    pp = (C.c_void_p * count)(*[p.data_ptr() for p in parts])
    check(lib().guffin_hip_gemv_packed_multi(_stream(), count, dt, tl, n, pp, _p(x), _p(xsums), rows, K))
    return parts


def geglu(gate, up, planes=None, want_sums=False):
    pl, stride = _planes(gate, planes)
    rows, width = gate.shape[1:] if planes else gate.shape
    out = _f32((rows, width), gate)
    sums = _receipt(rows, width, gate.device) if want_sums else None
    check(lib().guffin_hip_geglu(_stream(), _p(gate), _p(up), pl, C.c_uint64(stride), _p(out), _p(sums), rows, width))
    return (out, sums) if want_sums else out


def embed(dtype, w, tokens, width, scale, vocab, status=None):
    out = _f32((tokens.numel(), width), w)
    check(lib().guffin_hip_embed(_stream(), dtype, _p(w), _p(tokens), _p(out), tokens.numel(), width,
                                 C.c_float(scale), vocab, _p(status)))
    return out


def kv_scatter(priv_k, priv_v, selected, ring_k, ring_v, position, row_width, ring_mask):
    check(lib().guffin_hip_kv_scatter(_stream(), _p(priv_k), _p(priv_v), _p(selected), _p(ring_k), _p(ring_v),
                                      position, selected.numel(), row_width, ring_mask))


def attention_partitions(max_tokens, kv_heads):
    lib().guffin_hip_attention_partitions.restype = C.c_uint32
    return lib().guffin_hip_attention_partitions(max_tokens, kv_heads)


def attention_decode(q, ring_k, ring_v, priv_k, priv_v, schedule, ancestors, max_tokens, ring_mask, q_heads,
                     kv_heads, head_dim, scale, want_sums=False, status=None):
    rows = q.shape[0]
    P = attention_partitions(max_tokens, kv_heads)
    out = torch.empty_like(q)
    width = q_heads * head_dim
    sums = _receipt(rows, width, q.device) if want_sums else None
    part_out = _f32((rows * q_heads * P * head_dim,), q)
    part_ml = _f32((rows * q_heads * P * 2,), q)
    check(lib().guffin_hip_attention_decode(_stream(), _p(q), _p(ring_k), _p(ring_v), _p(priv_k), _p(priv_v),
                                            _p(schedule), _p(ancestors), _p(out), _p(sums), _p(part_out),
                                            _p(part_ml), rows, priv_k.shape[0], max_tokens, ring_mask, q_heads,
                                            kv_heads, head_dim, C.c_float(scale), _p(status)))
    return (out, sums) if want_sums else out


def qkv_attention(q_raw, k_raw, v_raw, q_norm, k_norm, table, ring_k, ring_v, schedule, ancestors, max_tokens,
                  ring_mask, q_heads, kv_heads, head_dim, scale, eps=1e-6, status=None):
    """Head norms, rotation, fp16 K/V rows and attention from the projections' planes [planes, rows, width].
    Returns (out, receipt, priv_k, priv_v)."""
    planes, rows = q_raw.shape[0], q_raw.shape[1]
    P = attention_partitions(max_tokens, kv_heads)
    out = torch.empty((rows, q_heads * head_dim), dtype=torch.float32, device=q_raw.device)
    sums = _receipt(rows, q_heads * head_dim, q_raw.device)
    pk = torch.empty((rows, kv_heads * head_dim), dtype=torch.float16, device=q_raw.device)
    pv = torch.empty_like(pk)
    part_out = _f32((rows * q_heads * P * head_dim,), q_raw)
    part_ml = _f32((rows * q_heads * P * 2,), q_raw)
    check(lib().guffin_hip_qkv_attention(_stream(), _p(q_raw), _p(k_raw), _p(v_raw), planes,
                                         C.c_uint64(q_raw[0].numel()), C.c_uint64(k_raw[0].numel()),
                                         C.c_uint64(v_raw[0].numel()), _p(q_norm), _p(k_norm), _p(table),
                                         C.c_float(eps), _p(ring_k), _p(ring_v), _p(pk), _p(pv), _p(schedule),
                                         _p(ancestors), _p(out), _p(sums), _p(part_out), _p(part_ml), rows,
                                         max_tokens, ring_mask, q_heads, kv_heads, head_dim, C.c_float(scale),
                                         _p(status)))
    return out, sums, pk, pv


# ---- head selection, proposal law, acceptance ------------------------------------------
import numpy as _np

token_logit = _np.dtype([("token", _np.uint32), ("logit", _np.float32)])
candidates_dtype = _np.dtype([("count", _np.uint32), ("status", _np.uint32), ("values", token_logit, (384,))])
law_dtype = _np.dtype([("count", _np.uint32), ("pad", _np.uint32), ("ids", _np.uint32, (256,)),
                       ("cdf", _np.uint64, (257,))])
result_dtype = _np.dtype([("accepted", _np.uint32), ("token", _np.uint32), ("next_root", _np.uint32),
                          ("status", _np.uint32), ("acceptance_probability", _np.float64),
                          ("residual_total", _np.float64), ("residual_count", _np.uint32),
                          ("proposal", _np.uint32)])
draws_dtype = _np.dtype([("word", _np.uint32), ("pad", _np.uint32), ("u_accept", _np.float64),
                         ("u_residual", _np.float64), ("u_next", _np.float64)])


class SamplerOptions(C.Structure):
    _fields_ = [("temperature", C.c_float), ("top_k", C.c_uint32), ("top_p", C.c_float),
                ("min_p", C.c_float), ("repetition_penalty", C.c_float)]


def _bytes(n, device="cuda"):
    return torch.zeros(int(n), dtype=torch.uint8, device=device)


def select_candidates(logits, retain, history=None, history_count=None, status=None, result=None):
    rows, vocab = logits.shape
    lib().guffin_hip_select_workspace_bytes.restype = C.c_uint64
    ws = _bytes(lib().guffin_hip_select_workspace_bytes(rows, vocab, retain))
    if result is None:
        result = _bytes(rows * candidates_dtype.itemsize)
    if status is None:
        status = torch.zeros(rows, dtype=torch.int32, device=logits.device)
    check(lib().guffin_hip_select_candidates(_stream(), _p(logits), rows, vocab, retain, _p(history),
                                             _p(history_count), _p(ws), _p(result), _p(status)))
    return result, status


selection_row_dtype = _np.dtype([("history_token_ids", _np.uint32, 64), ("suffix_token_ids", _np.uint32, 23),
                                ("history_head", _np.uint32), ("history_length", _np.uint32),
                                ("history_window_limit", _np.uint32), ("suffix_count", _np.uint32)])
resolved_row_dtype = _np.dtype([("top_k", _np.uint32), ("base_candidate_count", _np.uint32),
                               ("history_count", _np.uint32), ("reserved", _np.uint32),
                               ("history_token_ids", _np.uint32, 64)])


def input_validation(actual, expected, vocab, status):
    check(lib().guffin_hip_input_validation(_stream(), _p(actual), _p(expected), actual.numel(), vocab, _p(status)))


def selection_requests(raw, vocab, top_k, repetition_enabled=True):
    """raw: numpy array of selection_row_dtype records.  Returns (resolved rows on the device as bytes,
    histories [rows][64] on the device, the status word on the device)."""
    raw = _np.ascontiguousarray(raw, selection_row_dtype).reshape(-1)
    rows = raw.size
    d_raw = torch.from_numpy(raw.view(_np.uint8).copy()).cuda()
    resolved = _bytes(rows * resolved_row_dtype.itemsize)
    histories = torch.zeros(rows, 64, dtype=torch.int32, device="cuda")
    status = torch.zeros(1, dtype=torch.int32, device="cuda")
    check(lib().guffin_hip_selection_requests(_stream(), _p(d_raw), rows, vocab, top_k, 1 if repetition_enabled else 0,
                                              _p(resolved), _p(histories), _p(status)))
    return resolved, histories, status


def select_candidates_resolved(logits, retain_capacity, resolved, status=None, result=None):
    rows, vocab = logits.shape
    lib().guffin_hip_select_workspace_bytes.restype = C.c_uint64
    ws = _bytes(lib().guffin_hip_select_workspace_bytes(rows, vocab, retain_capacity))
    if result is None:
        result = _bytes(rows * candidates_dtype.itemsize)
    if status is None:
        status = torch.zeros(rows, dtype=torch.int32, device=logits.device)
    check(lib().guffin_hip_select_candidates_resolved(_stream(), _p(logits), rows, vocab, retain_capacity, _p(resolved),
                                                      _p(ws), _p(result), _p(status)))
    return result, status


def candidates_to_numpy(result):
    return result.cpu().numpy().view(candidates_dtype)


def argmax(logits, status=None):
    rows, vocab = logits.shape
    ws = _bytes(rows * 256 * 8)
    token = torch.zeros(rows, dtype=torch.int32, device=logits.device)
    logit = torch.zeros(rows, dtype=torch.float32, device=logits.device)
    check(lib().guffin_hip_argmax(_stream(), _p(logits), rows, vocab, _p(ws), _p(token), _p(logit), _p(status)))
    return token, logit


def draft_law(logits, options, seed=0, step=0, draws=None, law=None, proposal=None, status=None, workspace=None):
    vocab = logits.numel()
    lib().guffin_hip_draft_law_workspace_bytes.restype = C.c_uint64
    if workspace is None:
        workspace = _bytes(lib().guffin_hip_draft_law_workspace_bytes(vocab))
    if law is None:
        law = _bytes(law_dtype.itemsize)
    if proposal is None:
        proposal = torch.zeros(1, dtype=torch.int32, device=logits.device)
    if status is None:
        status = torch.zeros(1, dtype=torch.int32, device=logits.device)
    check(lib().guffin_hip_draft_law(_stream(), _p(logits), vocab, C.byref(options), C.c_uint64(seed),
                                     C.c_uint64(step), _p(draws), _p(workspace), _p(law), _p(proposal), _p(status)))
    return law, proposal, status


def draft_process(logits, history, repetition_penalty):
    """Drafter scores: the logits with the repetition penalty on the history's tokens."""
    scores = torch.empty_like(logits)
    check(lib().guffin_hip_draft_process(_stream(), _p(logits), logits.numel(), _p(history), history.numel(),
                                         C.c_float(repetition_penalty), _p(scores)))
    return scores


def vocab_map_invert(draft_to_target, target_vocab):
    """Host check of a draft -> target vocabulary map; returns (target_to_draft, number of mapped tokens)."""
    d2t = _np.ascontiguousarray(draft_to_target, _np.int32)
    t2d = _np.empty(target_vocab, _np.int32)
    mapped = C.c_uint32(0)
    check(lib().guffin_vocab_map_invert(d2t.ctypes.data_as(C.c_void_p), d2t.size, target_vocab,
                                        t2d.ctypes.data_as(C.c_void_p), C.byref(mapped)))
    return t2d, mapped.value


def draft_law_mapped(logits, draft_to_target, options, history=None, seed=0, step=0, draws=None, status=None):
    """(law in draft ids, draft proposal, target proposal, status) with the drafter's vocabulary map."""
    vocab = logits.numel()
    lib().guffin_hip_draft_law_workspace_bytes.restype = C.c_uint64
    workspace = _bytes(lib().guffin_hip_draft_law_workspace_bytes(vocab))
    scores = torch.empty_like(logits)
    law = _bytes(law_dtype.itemsize)
    draft = torch.zeros(1, dtype=torch.int32, device=logits.device)
    target = torch.zeros(1, dtype=torch.int32, device=logits.device)
    if status is None:
        status = torch.zeros(1, dtype=torch.int32, device=logits.device)
    check(lib().guffin_hip_draft_law_mapped(_stream(), _p(logits), vocab, _p(draft_to_target), _p(history),
                                            0 if history is None else history.numel(), C.byref(options),
                                            C.c_uint64(seed), C.c_uint64(step), _p(draws), _p(workspace), _p(scores),
                                            _p(law), _p(draft), _p(target), _p(status)))
    return law, draft, target, status


def draft_law_any_mapped(logits, draft_to_target, options, history=None, seed=0, step=0, draws=None, status=None):
    """draft_law_mapped by whichever path the options need: (law, full table, draft proposal, target proposal, status)."""
    vocab = logits.numel()
    lib().guffin_hip_draft_law_any_workspace_bytes.restype = C.c_uint64
    workspace = _bytes(lib().guffin_hip_draft_law_any_workspace_bytes(vocab))
    scores = torch.empty_like(logits)
    law = _bytes(law_dtype.itemsize)
    cdf = torch.zeros(vocab + 1, dtype=torch.int64, device=logits.device)
    draft = torch.zeros(1, dtype=torch.int32, device=logits.device)
    target = torch.zeros(1, dtype=torch.int32, device=logits.device)
    if status is None:
        status = torch.zeros(1, dtype=torch.int32, device=logits.device)
    check(lib().guffin_hip_draft_law_any_mapped(_stream(), _p(logits), vocab, _p(draft_to_target), _p(history),
                                                0 if history is None else history.numel(), C.byref(options),
                                                C.c_uint64(seed), C.c_uint64(step), _p(draws), _p(workspace), _p(scores),
                                                _p(law), _p(cdf), _p(draft), _p(target), _p(status)))
    return law, cdf, draft, target, status


def spec_accept_mapped(cands, law, target_to_draft, proposal, options, history=None, history_count=None, seed=0,
                       step=0, draws=None, status=None, full_cdf=None, vocab=0):
    """full_cdf / vocab: the drafter's full table and its vocabulary when the law is held as one."""
    result = _bytes(result_dtype.itemsize)
    check(lib().guffin_hip_spec_accept_mapped(_stream(), _p(cands), _p(law), _p(full_cdf), vocab, _p(target_to_draft), _p(history),
                                              _p(history_count), _p(proposal), C.byref(options), C.c_uint64(seed),
                                              C.c_uint64(step), _p(draws), _p(result), _p(status)))
    return result


def draft_law_any(logits, options, seed=0, step=0, draws=None, status=None):
    """The drafter's law by whichever path it needs: (law, full table, proposal, status)."""
    vocab = logits.numel()
    lib().guffin_hip_draft_law_any_workspace_bytes.restype = C.c_uint64
    workspace = _bytes(lib().guffin_hip_draft_law_any_workspace_bytes(vocab))
    law = _bytes(law_dtype.itemsize)
    cdf = torch.zeros(vocab + 1, dtype=torch.int64, device=logits.device)
    proposal = torch.zeros(1, dtype=torch.int32, device=logits.device)
    if status is None:
        status = torch.zeros(1, dtype=torch.int32, device=logits.device)
    check(lib().guffin_hip_draft_law_any(_stream(), _p(logits), vocab, C.byref(options), C.c_uint64(seed),
                                         C.c_uint64(step), _p(draws), _p(workspace), _p(law), _p(cdf),
                                         _p(proposal), _p(status)))
    return law, cdf, proposal, status


def spec_accept_law(cands, law, cdf, proposal, options, seed=0, step=0, draws=None, result=None, status=None):
    if result is None:
        result = _bytes(result_dtype.itemsize)
    vocab = 0 if cdf is None else cdf.numel() - 1
    check(lib().guffin_hip_spec_accept_law(_stream(), _p(cands), _p(law), _p(cdf), vocab, _p(proposal),
                                           C.byref(options), C.c_uint64(seed), C.c_uint64(step), _p(draws),
                                           _p(result), _p(status)))
    return result


def spec_accept_history(cands, law, history, history_count, proposal, options, seed=0, step=0, draws=None, status=None):
    """history: int32 [2, 64] token ids, history_count: int32 [2] (device tensors)."""
    result = _bytes(result_dtype.itemsize)
    check(lib().guffin_hip_spec_accept_history(_stream(), _p(cands), _p(law), None, 0, _p(history), _p(history_count),
                                               _p(proposal), C.byref(options), C.c_uint64(seed), C.c_uint64(step),
                                               _p(draws), _p(result), _p(status)))
    return result


def spec_accept(cands, law, proposal, options, seed=0, step=0, draws=None, result=None, status=None):
    if result is None:
        result = _bytes(result_dtype.itemsize)
    check(lib().guffin_hip_spec_accept(_stream(), _p(cands), _p(law), _p(proposal), C.byref(options),
                                       C.c_uint64(seed), C.c_uint64(step), _p(draws), _p(result), _p(status)))
    return result


def step_draws(seed, step):
    out = _np.zeros(1, draws_dtype)
    check(lib().guffin_hip_step_draws(C.c_uint64(seed), C.c_uint64(step), out.ctypes.data_as(C.c_void_p)))
    return out[0]


def gateup_geglu(dtype, gate_tiles, up_tiles, x, xsums, F, want_sums=True):
    rows, K = x.shape
    h = torch.empty((rows, F), dtype=torch.float32, device=x.device)
    sums = _receipt(rows, F, x.device) if want_sums else None
    check(lib().guffin_hip_gateup_geglu(_stream(), dtype, _p(gate_tiles), _p(up_tiles), _p(x), _p(xsums), _p(h),
                                        _p(sums), rows, K, F))
    return (h, sums) if want_sums else h


def prefill_pack(x):
    """Matrix-core operand (image, multipliers, sums) of the M rows of x."""
    M, K = x.shape
    lib().guffin_hip_prefill_image_bytes.restype = C.c_uint64
    n = lib().guffin_hip_prefill_image_bytes(M, K)
    if n == 0:
        raise GuffinError(-2, "prefill_pack: K must be a positive multiple of 32")
    image = torch.empty(n, dtype=torch.uint8, device=x.device)
    check(lib().guffin_hip_prefill_pack(_stream(), _p(x), _p(image), M, K))
    return image


def prefill_gemm(dtype, tiles, image, M, K, N):
    y = torch.empty((M, N), dtype=torch.float32, device=tiles.device)
    check(lib().guffin_hip_prefill_gemm(_stream(), dtype, _p(tiles), _p(image), _p(y), M, K, N))
    return y


def prefill_attention(q, ring_k, ring_v, run_k, run_v, position, window, ring_mask, q_heads, kv_heads, head_dim, scale,
                      matrix_core=True):
    rows = q.shape[0]
    out = torch.empty_like(q)
    ws = None
    if matrix_core:
        lib().guffin_hip_prefill_attention_workspace_bytes.restype = C.c_uint64
        ws = _bytes(max(16, lib().guffin_hip_prefill_attention_workspace_bytes(rows, position, window, kv_heads, head_dim)))
    check(lib().guffin_hip_prefill_attention(_stream(), _p(q), _p(ring_k), _p(ring_v), _p(run_k), _p(run_v), _p(out),
                                             rows, position, window, ring_mask, q_heads, kv_heads, head_dim,
                                             C.c_float(scale), _p(ws)))
    return out


def kv_cache_copy(src_k, src_v, dst_k, dst_v, position, tokens, src_mask, dst_mask):
    check(lib().guffin_hip_kv_cache_copy(_stream(), _p(src_k), _p(src_v), _p(dst_k), _p(dst_v), position, tokens,
                                         src_mask, dst_mask, src_k.shape[-1]))


def publish_run(run_k, run_v, ring_k, ring_v, position, ring_mask):
    rows, width = run_k.shape
    check(lib().guffin_hip_publish_run(_stream(), _p(run_k), _p(run_v), _p(ring_k), _p(ring_v), rows, position,
                                       ring_mask, width))
