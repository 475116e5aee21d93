"""Synthetic Gemma-3 shaped models for the H1 step: descriptors, seeded weights, KV rings.

Shapes of the benchmark configurations: the 12B target (48 blocks, hidden 3840, FFN 15360,
16 query / 8 KV heads of 256, sliding window 1024 on 5 of every 6 blocks, Q4_K projections
with Q6_K v_proj / down_proj and a tied Q6_K head) and the 270M drafter (18 blocks, hidden 640,
FFN 2048, 4 query / 1 KV head, window 512, Q8_0 everywhere).  Layer policy and RoPE bases:
reference src/engine/model.cpp:607-619, tests/support/gemma3_target_test_support.hpp:37-38.
"""
import ctypes as C
from dataclasses import dataclass, field, replace

import numpy as np
import torch

from . import hip, synth

Q8_0, Q4_K, Q6_K = 0, 1, 2


class LayerDesc(C.Structure):
    _fields_ = [("dtype", C.c_int32 * 7), ("tiles", C.c_void_p * 7), ("norm", C.c_void_p * 6),
                ("ring_k", C.c_void_p), ("ring_v", C.c_void_p)]


class ModelDesc(C.Structure):
    _fields_ = [(n, C.c_uint32) for n in ("hidden", "ffn", "q_heads", "kv_heads", "head_dim", "layer_count",
                                           "vocab", "sliding_window", "global_period")] + \
               [(n, C.c_float) for n in ("local_base", "global_base", "global_scale", "eps")] + \
               [("ring_local", C.c_uint32), ("ring_global", C.c_uint32),
                ("embed_dtype", C.c_int32), ("embed_rows", C.c_void_p),
                ("head_dtype", C.c_int32), ("head_tiles", C.c_void_p),
                ("out_norm", C.c_void_p), ("layers", C.POINTER(LayerDesc))]


class H1Desc(C.Structure):
    _fields_ = [("target", C.POINTER(ModelDesc)), ("drafter", C.POINTER(ModelDesc)),
                ("target_position", C.c_uint32), ("drafter_position", C.c_uint32),
                ("temperature", C.c_float), ("top_k", C.c_uint32), ("top_p", C.c_float), ("min_p", C.c_float),
                ("seed", C.c_uint64), ("step", C.c_uint64),
                ("target_ring_k", C.c_void_p), ("target_ring_v", C.c_void_p),
                ("drafter_ring_k", C.c_void_p), ("drafter_ring_v", C.c_void_p), ("full_law", C.c_uint32),
                ("drafter_rows", C.c_uint32), ("pending_token", C.c_void_p),
                ("history", C.c_void_p), ("history_count", C.c_uint32), ("repetition_penalty", C.c_float),
                ("draft_to_target", C.c_void_p), ("target_to_draft", C.c_void_p)]


class H1Session(C.Structure):
    _fields_ = [("desc", H1Desc), ("scratch", C.c_void_p), ("scratch_bytes", C.c_uint64),
                ("drafter_priv_k", C.c_void_p), ("drafter_priv_v", C.c_void_p),
                ("target_priv_k", C.c_void_p), ("target_priv_v", C.c_void_p),
                ("tokens", C.c_void_p), ("result", C.c_void_p), ("status", C.c_void_p),
                ("state", C.c_uint32), ("root", C.c_uint32), ("pending", C.c_uint32), ("has_pending", C.c_uint32),
                ("cycles", C.c_uint64), ("accepted", C.c_uint64)]


@dataclass(frozen=True)
class Shape:
    hidden: int
    ffn: int
    q_heads: int
    kv_heads: int
    head_dim: int
    layers: int
    vocab: int
    sliding_window: int
    global_period: int
    local_base: float
    global_base: float
    global_scale: float
    ring_local: int
    ring_global: int
    dtypes: tuple = (Q4_K, Q4_K, Q6_K, Q4_K, Q4_K, Q4_K, Q6_K)   # q k v o gate up down
    embed_dtype: int = Q6_K
    eps: float = 1e-6
    # per-block formats where they differ from `dtypes` (a Q4_K_M file keeps some blocks' attn_v and
    # ffn_down in Q6_K and others in Q4_K): one 7-tuple per block, or None
    layer_dtypes: tuple = None

    @property
    def q_width(self):
        return self.q_heads * self.head_dim

    @property
    def kv_width(self):
        return self.kv_heads * self.head_dim

    def is_local(self, layer):
        return self.global_period > 1 and layer % self.global_period != self.global_period - 1

    def dtypes_of(self, layer):
        return self.layer_dtypes[layer] if self.layer_dtypes else self.dtypes

    def proj_shapes(self):
        """(K, N) of q, k, v, o, gate, up, down."""
        H, F, QW, KW = self.hidden, self.ffn, self.q_width, self.kv_width
        return [(H, QW), (H, KW), (H, KW), (QW, H), (H, F), (H, F), (F, H)]

    def layer_weight_bytes(self, layer=0):
        return sum(synth.weight_bytes(d, K, N) for d, (K, N) in zip(self.dtypes_of(layer), self.proj_shapes()))

    def body_weight_bytes(self):
        return sum(self.layer_weight_bytes(l) for l in range(self.layers))

    def head_bytes(self):
        return synth.weight_bytes(self.embed_dtype, self.hidden, self.vocab)


GEMMA3_12B = Shape(3840, 15360, 16, 8, 256, 48, 262144, 1024, 6, 1e4, 1e6, 0.125, 1024, 8192)
GEMMA3_270M = Shape(640, 2048, 4, 1, 256, 18, 262144, 512, 6, 1e4, 1e6, 1.0, 512, 8192,
                    dtypes=(Q8_0,) * 7, embed_dtype=Q8_0)


def tiny(shape, layers, vocab):
    return replace(shape, layers=layers, vocab=vocab)


class HostModel:
    """Canonical-layout numpy weights (what the CPU oracle consumes)."""

    def __init__(self, shape, seed, position, gamma_sigma=0.1, untied_head=False):
        """untied_head: the output head is a matrix of its own (a GGUF file's output.weight) instead of the
        embedding matrix; with random weights a tied head puts nearly all mass on the input token."""
        self.shape = shape
        rng = np.random.Generator(np.random.PCG64(seed))
        self.w = []      # [layer][7] canonical uint8
        self.norm = []   # [layer][6] float32
        self.ring_k, self.ring_v = [], []
        s = 1000 * seed
        for l in range(shape.layers):
            self.w.append([synth.make_weight(d, K, N, s + 16 * l + i)
                           for i, (d, (K, N)) in enumerate(zip(shape.dtypes_of(l), shape.proj_shapes()))])
            widths = [shape.hidden, shape.head_dim, shape.head_dim, shape.hidden, shape.hidden, shape.hidden]
            self.norm.append([(1.0 + rng.normal(0, gamma_sigma, w)).astype(np.float32) for w in widths])
            cap = shape.ring_local if shape.is_local(l) else shape.ring_global
            k = np.zeros((cap, shape.kv_width), np.float16)
            v = np.zeros((cap, shape.kv_width), np.float16)
            filled = min(position, cap)
            # positions position-filled .. position-1 live at slot p & (cap-1)
            slots = (np.arange(position - filled, position) & (cap - 1))
            k[slots] = rng.normal(0, 1, (filled, shape.kv_width)).astype(np.float16)
            v[slots] = rng.normal(0, 1, (filled, shape.kv_width)).astype(np.float16)
            self.ring_k.append(k)
            self.ring_v.append(v)
        self.embed = synth.make_weight(shape.embed_dtype, shape.hidden, shape.vocab, s + 999)
        self.head = synth.make_weight(shape.embed_dtype, shape.hidden, shape.vocab, s + 998) if untied_head else self.embed
        self.out_norm = (1.0 + rng.normal(0, gamma_sigma, shape.hidden)).astype(np.float32)

    def commit(self, pk, pv, position, rows):
        """Publishes the first `rows` private rows of a pass at `position` into the rings, like the device."""
        for l in range(self.shape.layers):
            cap = self.shape.ring_local if self.shape.is_local(l) else self.shape.ring_global
            for r in range(rows):
                self.ring_k[l][(position + r) & (cap - 1)] = pk[l, r].view(np.float16)
                self.ring_v[l][(position + r) & (cap - 1)] = pv[l, r].view(np.float16)


class DeviceModel:
    """Device weights as wave tiles plus the descriptor the C ABI takes."""

    def __init__(self, shape):
        self.shape = shape
        self.keep = []            # tensors kept alive
        self.layers = (LayerDesc * shape.layers)()
        self.desc = ModelDesc()
        self.ring_k, self.ring_v = [], []

    def _finish(self, embed_rows, head_tiles, out_norm):
        sh, d = self.shape, self.desc
        for name in ("hidden", "ffn", "q_heads", "kv_heads", "head_dim", "vocab", "sliding_window",
                     "global_period", "local_base", "global_base", "global_scale", "eps", "ring_local", "ring_global"):
            setattr(d, name, getattr(sh, name))
        d.layer_count = sh.layers
        d.embed_dtype = d.head_dtype = sh.embed_dtype
        d.embed_rows = embed_rows.data_ptr()
        d.head_tiles = head_tiles.data_ptr()
        d.out_norm = out_norm.data_ptr()
        d.layers = C.cast(self.layers, C.POINTER(LayerDesc))
        self.keep += [embed_rows, head_tiles, out_norm]
        self.head_tiles = head_tiles   # the packed head matrix (tied embedding)
        self.out_norm = out_norm       # device gamma of the output norm (a test may rescale it in place)
        self.ring_k_table = torch.tensor([t.data_ptr() for t in self.ring_k], dtype=torch.int64, device="cuda")
        self.ring_v_table = torch.tensor([t.data_ptr() for t in self.ring_v], dtype=torch.int64, device="cuda")
        return self

    @classmethod
    def from_host(cls, host):
        self = cls(host.shape)
        sh = host.shape
        for l in range(sh.layers):
            for i, (dt, (K, N)) in enumerate(zip(sh.dtypes_of(l), sh.proj_shapes())):
                canonical = torch.from_numpy(host.w[l][i]).cuda()
                tiles = hip.repack(dt, canonical, K, N)
                self.keep.append(tiles)
                self.layers[l].dtype[i] = dt
                self.layers[l].tiles[i] = tiles.data_ptr()
            for i in range(6):
                g = torch.from_numpy(host.norm[l][i]).cuda()
                self.keep.append(g)
                self.layers[l].norm[i] = g.data_ptr()
            rk, rv = torch.from_numpy(host.ring_k[l]).cuda(), torch.from_numpy(host.ring_v[l]).cuda()
            self.ring_k.append(rk)
            self.ring_v.append(rv)
            self.layers[l].ring_k, self.layers[l].ring_v = rk.data_ptr(), rv.data_ptr()
        embed = torch.from_numpy(host.embed).cuda()
        head = hip.repack(sh.embed_dtype, embed if host.head is host.embed else torch.from_numpy(host.head).cuda(),
                          sh.hidden, sh.vocab)
        torch.cuda.synchronize()
        return self._finish(embed, head, torch.from_numpy(host.out_norm).cuda())

    # GGUF tensor names of a Gemma block in the order of LayerDesc.tiles / LayerDesc.norm
    # (src/engine/gemma_model.cpp:36-72 of the reference)
    GGUF_MATRICES = ("attn_q", "attn_k", "attn_v", "attn_output", "ffn_gate", "ffn_up", "ffn_down")
    GGUF_NORMS = ("attn_norm", "attn_q_norm", "attn_k_norm", "post_attention_norm", "ffn_norm", "post_ffw_norm")
    GGUF_TYPES = {8: Q8_0, 12: Q4_K, 14: Q6_K}

    @classmethod
    def from_gguf(cls, reader, ring_local=None, ring_global=8192, arch="gemma3", role="target"):
        """Binds a parsed GGUF file (guffin_amd.gguf.Reader): shape from the `<arch>.*` metadata keys
        (src/engine/model.cpp:330-390), matrices uploaded as they lie in the file ([input, output] with
        the input dimension contiguous, i.e. blocks per output column) and repacked on the device, tied
        head when there is no output.weight (model.cpp:328).  Rings start empty.

        `role` is the caller's statement of what the file is: "target" binds under the reference's target rules
        (256-wide paired GQA heads, K-quant matrices, Q6_K head: gemma_model.cpp:120-124, 137-147), "drafter"
        without the geometry rule and with Q8_0 matrices allowed.  A file that does not fit its role is refused."""
        if role not in ("target", "drafter"):
            raise ValueError("from_gguf: role is 'target' or 'drafter'")
        from . import gguf as gguf_module
        md = reader.metadata()
        key = lambda k: md[arch + "." + k]
        scale = 1.0
        if md.get(arch + ".rope.scaling.type", "none") == "linear":
            scale = 1.0 / float(key("rope.scaling.factor"))
        embed_info = reader.tensor("token_embd.weight")
        hidden, vocab = embed_info["dims"]
        layers = int(key("block_count"))
        window = int(key("attention.sliding_window"))
        # names, shapes and formats are checked by the library before anything is uploaded
        # (guffin_gguf_bind_gemma3: bind_gemma_model_weights + validate_gemma3_model_weights of the reference)
        cfg = gguf_module.Gemma3Config()
        cfg.block_count, cfg.embedding_length, cfg.vocab_size = layers, int(key("embedding_length")), vocab
        cfg.feed_forward_length = int(key("feed_forward_length"))
        cfg.attention_head_count, cfg.attention_head_count_kv = int(key("attention.head_count")), int(key("attention.head_count_kv"))
        cfg.attention_key_length, cfg.attention_value_length = int(key("attention.key_length")), int(key("attention.value_length"))
        cfg.sliding_window, cfg.context_length = window, int(md.get(arch + ".context_length", ring_global))
        cfg.attention_global_layer_period = int(md.get(arch + ".attention.sliding_window_pattern", 6))
        cfg.uses_qk_norm = 1
        cfg.uses_tied_output_weight = 0 if reader.has_tensor("output.weight") else 1
        cfg.target_geometry = 1 if role == "target" else 0
        cfg.rms_norm_epsilon = float(key("attention.layer_norm_rms_epsilon"))
        cfg.attention_logit_softcap = float(md.get(arch + ".attn_logit_softcapping", 0.0))
        cfg.final_logit_softcap = float(md.get(arch + ".final_logit_softcapping", 0.0))
        cfg.rope_freq_base = float(key("rope.freq_base"))
        cfg.local_rope_freq_base = float(md.get(arch + ".rope.freq_base_swa", 10000.0))
        cfg.rope_freq_scale = scale
        binding, blocks = reader.bind_gemma3(cfg)

        def matrix_type(name):
            return cls.GGUF_TYPES[reader.tensor(name)["type_id"]]

        names = [["blk.%d.%s.weight" % (l, m) for m in cls.GGUF_MATRICES] for l in range(layers)]
        per_layer = tuple(tuple(cls.GGUF_TYPES[blocks[l].type_id[i]] for i in range(7)) for l in range(layers))
        uniform = all(row == per_layer[0] for row in per_layer)
        shape = Shape(hidden=hidden, ffn=int(key("feed_forward_length")), q_heads=int(key("attention.head_count")),
                      kv_heads=int(key("attention.head_count_kv")), head_dim=int(key("attention.key_length")),
                      layers=layers, vocab=vocab, sliding_window=window,
                      global_period=int(md.get(arch + ".attention.sliding_window_pattern", 6)),
                      local_base=float(md.get(arch + ".rope.freq_base_swa", 10000.0)),
                      global_base=float(key("rope.freq_base")), global_scale=scale,
                      ring_local=ring_local or 1 << (window - 1).bit_length(), ring_global=ring_global,
                      dtypes=per_layer[0], embed_dtype=matrix_type("token_embd.weight"),
                      eps=float(key("attention.layer_norm_rms_epsilon")),
                      layer_dtypes=None if uniform else per_layer)
        self = cls(shape)

        def upload(name):
            return torch.from_numpy(np.array(reader.payload(name))).cuda()   # staged through a writable copy

        def norm(name, width):
            return upload(name).view(torch.float32)

        widths = [hidden, shape.head_dim, shape.head_dim, hidden, hidden, hidden]
        for l in range(layers):
            for i, (m, (K, N)) in enumerate(zip(cls.GGUF_MATRICES, shape.proj_shapes())):
                name = names[l][i]
                dt = per_layer[l][i]
                tiles = hip.repack(dt, upload(name), K, N)
                self.keep.append(tiles)
                self.layers[l].dtype[i] = dt
                self.layers[l].tiles[i] = tiles.data_ptr()
            for i, (n, w) in enumerate(zip(cls.GGUF_NORMS, widths)):
                g = norm("blk.%d.%s.weight" % (l, n), w)
                self.keep.append(g)
                self.layers[l].norm[i] = g.data_ptr()
            cap = shape.ring_local if shape.is_local(l) else shape.ring_global
            rk = torch.zeros((cap, shape.kv_width), dtype=torch.float16, device="cuda")
            rv = torch.zeros_like(rk)
            self.ring_k.append(rk)
            self.ring_v.append(rv)
            self.layers[l].ring_k, self.layers[l].ring_v = rk.data_ptr(), rv.data_ptr()
        embed = upload("token_embd.weight")
        head_name = "token_embd.weight" if binding.tied_output else "output.weight"
        head = hip.repack(matrix_type(head_name), embed if head_name == "token_embd.weight" else upload(head_name),
                          hidden, vocab)
        torch.cuda.synchronize()
        return self._finish(embed, head, norm("output_norm.weight", hidden))

    @classmethod
    def random(cls, shape, seed, position):
        """Weights drawn on the device (full-size benchmark: no host copy of the 7 GB)."""
        self = cls(shape)
        gen = torch.Generator(device="cuda")
        gen.manual_seed(seed)

        def blocks(dt, K, N):
            nb = N * (K // synth.BLOCK_ELEMS[dt])
            raw = torch.randint(0, 256, (nb, synth.BLOCK_BYTES[dt]), dtype=torch.uint8, device="cuda", generator=gen)
            d = torch.randn(nb, device="cuda", generator=gen).mul_(0.02).abs_().to(torch.float16).view(torch.uint8).view(nb, 2)
            if dt == Q4_K:
                raw[:, 0:2] = d
                raw[:, 2:4] = torch.randn(nb, device="cuda", generator=gen).mul_(0.02).abs_().to(torch.float16).view(torch.uint8).view(nb, 2)
            elif dt == Q6_K:
                raw[:, 208:210] = d
            else:
                raw[:, 0:2] = d
                q = raw[:, 2:]
                q[q == 0x80] = 0x81
            return raw.view(-1)

        for l in range(shape.layers):
            for i, (dt, (K, N)) in enumerate(zip(shape.dtypes_of(l), shape.proj_shapes())):
                tiles = hip.repack(dt, blocks(dt, K, N), K, N)
                self.keep.append(tiles)
                self.layers[l].dtype[i] = dt
                self.layers[l].tiles[i] = tiles.data_ptr()
            widths = [shape.hidden, shape.head_dim, shape.head_dim, shape.hidden, shape.hidden, shape.hidden]
            for i, w in enumerate(widths):
                g = torch.ones(w, dtype=torch.float32, device="cuda")
                self.keep.append(g)
                self.layers[l].norm[i] = g.data_ptr()
            cap = shape.ring_local if shape.is_local(l) else shape.ring_global
            rk = torch.randn((cap, shape.kv_width), device="cuda", generator=gen).to(torch.float16)
            rv = torch.randn((cap, shape.kv_width), device="cuda", generator=gen).to(torch.float16)
            self.ring_k.append(rk)
            self.ring_v.append(rv)
            self.layers[l].ring_k, self.layers[l].ring_v = rk.data_ptr(), rv.data_ptr()
        embed = blocks(shape.embed_dtype, shape.hidden, shape.vocab)
        head = hip.repack(shape.embed_dtype, embed, shape.hidden, shape.vocab)
        torch.cuda.synchronize()
        return self._finish(embed, head, torch.ones(shape.hidden, dtype=torch.float32, device="cuda"))

    def private_rows(self, rows):
        sh = self.shape
        return (torch.zeros((sh.layers, rows, sh.kv_width), dtype=torch.float16, device="cuda"),
                torch.zeros((sh.layers, rows, sh.kv_width), dtype=torch.float16, device="cuda"))

    def forward(self, tokens, position, status=None):
        """Runs len(tokens) rows; returns (hidden, hidden_sums, priv_k, priv_v)."""
        sh = self.shape
        rows = tokens.numel()
        lib = hip.lib()
        lib.guffin_hip_forward_scratch_bytes.restype = C.c_uint64
        nbytes = lib.guffin_hip_forward_scratch_bytes(C.byref(self.desc), rows, position)
        if nbytes == 0:
            raise hip.GuffinError(-1, lib.guffin_hip_last_error().decode())
        scratch = torch.zeros(nbytes, dtype=torch.uint8, device="cuda")
        pk, pv = self.private_rows(rows)
        hidden = torch.zeros((rows, sh.hidden), dtype=torch.float32, device="cuda")
        sums = hip._receipt(rows, sh.hidden, "cuda")
        if status is None:
            status = hip.new_status()
        hip.check(lib.guffin_hip_forward_rows(hip._stream(), C.byref(self.desc), hip._p(tokens), rows, position,
                                              hip._p(scratch), C.c_uint64(nbytes), hip._p(pk), hip._p(pv),
                                              hip._p(hidden), hip._p(sums), hip._p(status)))
        return hidden, sums, pk, pv, status


    def prefill(self, tokens, position, status=None):
        """Ingests len(tokens) rows at `position` (rings are updated); returns the output-normed rows."""
        sh = self.shape
        rows = tokens.numel()
        lib = hip.lib()
        lib.guffin_hip_prefill_scratch_bytes.restype = C.c_uint64
        nbytes = lib.guffin_hip_prefill_scratch_bytes(C.byref(self.desc), rows)
        if nbytes == 0:
            raise hip.GuffinError(-1, lib.guffin_hip_last_error().decode())
        scratch = torch.zeros(nbytes, dtype=torch.uint8, device="cuda")
        hidden = torch.zeros((rows, sh.hidden), dtype=torch.float32, device="cuda")
        if status is None:
            status = hip.new_status()
        hip.check(lib.guffin_hip_prefill_rows(hip._stream(), C.byref(self.desc), hip._p(tokens), rows, position,
                                              hip._p(scratch), C.c_uint64(nbytes), hip._p(hidden), hip._p(status)))
        return hidden, status


class H1Plan:
    """One speculative cycle: buffers, descriptor and the call into guffin_hip_h1_step."""

    def __init__(self, target, drafter, target_position, drafter_position, temperature=1.0, top_k=64,
                 top_p=0.95, min_p=0.0, seed=0, publish=True, full_law=False, history=None, repetition_penalty=1.0,
                 draft_to_target=None, target_to_draft=None):
        self.target, self.drafter = target, drafter
        d = self.desc = H1Desc()
        d.target, d.drafter = C.pointer(target.desc), C.pointer(drafter.desc)
        d.target_position, d.drafter_position = target_position, drafter_position
        d.temperature, d.top_k, d.top_p, d.min_p = temperature, top_k, top_p, min_p
        d.seed, d.step = seed, 0
        d.full_law = 1 if full_law else 0
        if history is not None:
            self.history = torch.tensor(list(history), dtype=torch.int32, device="cuda")
            d.history, d.history_count, d.repetition_penalty = self.history.data_ptr(), len(history), repetition_penalty
        if draft_to_target is not None:
            self.draft_to_target = torch.as_tensor(draft_to_target, dtype=torch.int32).cuda()
            self.target_to_draft = torch.as_tensor(target_to_draft, dtype=torch.int32).cuda()
            d.draft_to_target, d.target_to_draft = self.draft_to_target.data_ptr(), self.target_to_draft.data_ptr()
        if publish:
            d.target_ring_k, d.target_ring_v = target.ring_k_table.data_ptr(), target.ring_v_table.data_ptr()
            d.drafter_ring_k, d.drafter_ring_v = drafter.ring_k_table.data_ptr(), drafter.ring_v_table.data_ptr()
        lib = hip.lib()
        lib.guffin_hip_h1_scratch_bytes.restype = C.c_uint64
        self.nbytes = lib.guffin_hip_h1_scratch_bytes(C.byref(d))
        if self.nbytes == 0:
            raise hip.GuffinError(-1, lib.guffin_hip_last_error().decode())
        self.scratch = torch.zeros(self.nbytes, dtype=torch.uint8, device="cuda")
        self.d_pk, self.d_pv = drafter.private_rows(1)
        self.t_pk, self.t_pv = target.private_rows(2)
        self.result = torch.zeros(hip.result_dtype.itemsize, dtype=torch.uint8, device="cuda")
        self.status = hip.new_status()
        self.root = torch.zeros(1, dtype=torch.int32, device="cuda")

    def step(self, step=None):
        if step is not None:
            self.desc.step = step
        hip.check(hip.lib().guffin_hip_h1_step(hip._stream(), C.byref(self.desc), hip._p(self.root),
                                               hip._p(self.scratch), C.c_uint64(self.nbytes), hip._p(self.d_pk),
                                               hip._p(self.d_pv), hip._p(self.t_pk), hip._p(self.t_pv),
                                               hip._p(self.result), hip._p(self.status)))

    def read_result(self):
        return self.result.cpu().numpy().view(hip.result_dtype)[0]

    def buffers(self):
        """Views of the step's intermediates inside the scratch arena."""
        ptrs = [C.c_void_p() for _ in range(7)]
        hip.check(hip.lib().guffin_hip_h1_buffers(C.byref(self.desc), hip._p(self.scratch),
                                                  *[C.byref(p) for p in ptrs]))
        base = self.scratch.data_ptr()
        T, D = self.target.shape, self.drafter.shape
        d_rows = 2 if self.desc.drafter_rows == 2 else 1

        def view(ptr, count, dtype):
            off = ptr.value - base
            return self.scratch[off:off + count * torch.tensor([], dtype=dtype).element_size()].view(dtype)

        full = C.c_void_p()
        hip.check(hip.lib().guffin_hip_h1_full_cdf(C.byref(self.desc), hip._p(self.scratch), C.byref(full)))
        return {
            "full_cdf": view(full, D.vocab + 1, torch.int64) if full.value else None,
            "drafter_hidden": view(ptrs[0], d_rows * D.hidden, torch.float32).view(d_rows, D.hidden)[d_rows - 1],
            "drafter_hidden_rows": view(ptrs[0], d_rows * D.hidden, torch.float32).view(d_rows, D.hidden),
            "target_hidden": view(ptrs[1], 2 * T.hidden, torch.float32).view(2, T.hidden),
            "q_logits": view(ptrs[2], D.vocab, torch.float32),
            "p_logits": view(ptrs[3], 2 * T.vocab, torch.float32).view(2, T.vocab),
            "law": view(ptrs[4], hip.law_dtype.itemsize, torch.uint8),
            "candidates": view(ptrs[5], 2 * hip.candidates_dtype.itemsize, torch.uint8),
            "tokens": view(ptrs[6], 10, torch.int32),
        }


class VerifyTicketDesc(C.Structure):
    _fields_ = [("target", C.POINTER(ModelDesc)), ("scratch", C.c_void_p), ("scratch_bytes", C.c_uint64),
                ("priv_k", C.c_void_p), ("priv_v", C.c_void_p), ("backup_k", C.c_void_p), ("backup_v", C.c_void_p),
                ("tokens", C.c_void_p), ("selected", C.c_void_p), ("candidates", C.c_void_p), ("status", C.c_void_p),
                ("retain", C.c_uint32), ("state", C.c_uint32), ("rows", C.c_uint32), ("position", C.c_uint32),
                ("provisional_count", C.c_uint32), ("provisional_path", C.c_uint32 * 4), ("row_tokens", C.c_uint32 * 4),
                ("parents", C.c_uint32 * 4), ("depths", C.c_uint32 * 4)]


TXN_IDLE, TXN_ENCODED, TXN_SUBMITTED, TXN_COMPLETED, TXN_PROVISIONAL, TXN_POISONED = range(6)


class VerifyTicket:
    """The target's verify pass as a transaction (guffin_hip_ticket_*): buffers and the calls."""

    def __init__(self, target, last_position, retain=64):
        self.target = target
        sh = target.shape
        t = self.desc = VerifyTicketDesc()
        t.target = C.pointer(target.desc)
        t.retain = retain
        lib = hip.lib()
        lib.guffin_hip_ticket_scratch_bytes.restype = C.c_uint64
        nbytes = lib.guffin_hip_ticket_scratch_bytes(C.byref(t), last_position)
        if nbytes == 0:
            raise hip.GuffinError(-1, "ticket: no arena size for this target")
        self.scratch = torch.zeros(nbytes, dtype=torch.uint8, device="cuda")
        self.priv_k, self.priv_v = target.private_rows(4)
        self.backup_k, self.backup_v = target.private_rows(4)
        self.tokens = torch.zeros(4, dtype=torch.int32, device="cuda")
        self.selected = torch.zeros(4, dtype=torch.int32, device="cuda")
        self.candidates = torch.zeros(4 * hip.candidates_dtype.itemsize, dtype=torch.uint8, device="cuda")
        self.status = torch.zeros(5, dtype=torch.int32, device="cuda")
        t.scratch, t.scratch_bytes = self.scratch.data_ptr(), nbytes
        t.priv_k, t.priv_v = self.priv_k.data_ptr(), self.priv_v.data_ptr()
        t.backup_k, t.backup_v = self.backup_k.data_ptr(), self.backup_v.data_ptr()
        t.tokens, t.selected = self.tokens.data_ptr(), self.selected.data_ptr()
        t.candidates, t.status = self.candidates.data_ptr(), self.status.data_ptr()
        t.state = TXN_IDLE

    @property
    def state(self):
        return int(self.desc.state)

    def encode(self, row_tokens, position):
        arr = (C.c_uint32 * len(row_tokens))(*row_tokens)
        hip.check(hip.lib().guffin_hip_ticket_encode(C.byref(self.desc), arr, len(row_tokens), position))

    ROOT = 0xFFFFFFFF

    def encode_tree(self, row_tokens, parents, position):
        """parents[r]: the row whose child row r is (None for the root)."""
        arr = (C.c_uint32 * len(row_tokens))(*row_tokens)
        par = (C.c_uint32 * len(parents))(*[self.ROOT if p is None else p for p in parents])
        hip.check(hip.lib().guffin_hip_ticket_encode_tree(C.byref(self.desc), arr, par, len(row_tokens), position))

    def submit(self):
        hip.check(hip.lib().guffin_hip_ticket_submit(hip._stream(), C.byref(self.desc)))

    def complete(self):
        raised = C.c_uint32(0)
        hip.check(hip.lib().guffin_hip_ticket_complete(hip._stream(), C.byref(self.desc), C.byref(raised)))
        return raised.value

    def provisional_commit(self, path):
        arr = (C.c_uint32 * max(1, len(path)))(*path)
        hip.check(hip.lib().guffin_hip_ticket_provisional_commit(hip._stream(), C.byref(self.desc), arr, len(path)))

    def finalize(self, retained):
        hip.check(hip.lib().guffin_hip_ticket_finalize(hip._stream(), C.byref(self.desc), retained))

    def discard(self):
        hip.check(hip.lib().guffin_hip_ticket_discard(hip._stream(), C.byref(self.desc)))

    def release(self):
        hip.check(hip.lib().guffin_hip_ticket_release(hip._stream(), C.byref(self.desc)))

    def read_candidates(self):
        return self.candidates.cpu().numpy().view(hip.candidates_dtype)


class Session:
    """Consecutive H1 cycles through guffin_hip_session_*: the library keeps positions, the drafter's
    pending token and the transaction state; this class owns the device memory it points at."""

    def __init__(self, target, drafter, root, target_position, drafter_position, cycles, temperature=1.0, top_k=64,
                 top_p=0.95, min_p=0.0, seed=0, full_law=False):
        self.target, self.drafter = target, drafter
        s = self.s = H1Session()
        d = s.desc
        d.target, d.drafter = C.pointer(target.desc), C.pointer(drafter.desc)
        d.temperature, d.top_k, d.top_p, d.min_p = temperature, top_k, top_p, min_p
        d.seed, d.full_law = seed, 1 if full_law else 0
        d.target_ring_k, d.target_ring_v = target.ring_k_table.data_ptr(), target.ring_v_table.data_ptr()
        d.drafter_ring_k, d.drafter_ring_v = drafter.ring_k_table.data_ptr(), drafter.ring_v_table.data_ptr()
        lib = hip.lib()
        lib.guffin_hip_session_scratch_bytes.restype = C.c_uint64
        nbytes = lib.guffin_hip_session_scratch_bytes(C.byref(s), target_position + 2 * cycles,
                                                      drafter_position + 2 * cycles)
        if nbytes == 0:
            raise hip.GuffinError(-1, lib.guffin_hip_last_error().decode())
        self.scratch = torch.zeros(nbytes, dtype=torch.uint8, device="cuda")
        self.d_pk, self.d_pv = drafter.private_rows(2)
        self.t_pk, self.t_pv = target.private_rows(2)
        self.tokens = torch.zeros(2, dtype=torch.int32, device="cuda")
        self.result = torch.zeros(hip.result_dtype.itemsize, dtype=torch.uint8, device="cuda")
        self.status = hip.new_status()
        s.scratch, s.scratch_bytes = self.scratch.data_ptr(), nbytes
        s.drafter_priv_k, s.drafter_priv_v = self.d_pk.data_ptr(), self.d_pv.data_ptr()
        s.target_priv_k, s.target_priv_v = self.t_pk.data_ptr(), self.t_pv.data_ptr()
        s.tokens, s.result, s.status = self.tokens.data_ptr(), self.result.data_ptr(), self.status.data_ptr()
        hip.check(lib.guffin_hip_session_start(C.byref(s), root, target_position, drafter_position))

    def submit(self):
        hip.check(hip.lib().guffin_hip_session_submit(hip._stream(), C.byref(self.s)))

    def complete(self):
        out = (C.c_uint32 * 2)()
        n = C.c_uint32()
        self._cycle_desc = H1Desc.from_buffer_copy(self.s.desc)   # the arena layout of the cycle in flight
        hip.check(hip.lib().guffin_hip_session_complete(hip._stream(), C.byref(self.s), out, C.byref(n)))
        return [int(out[i]) for i in range(n.value)]

    def buffers(self):
        plan = H1Plan.__new__(H1Plan)
        plan.desc, plan.scratch, plan.target, plan.drafter = self._cycle_desc, self.scratch, self.target, self.drafter
        return H1Plan.buffers(plan)

    def read_result(self):
        return self.result.cpu().numpy().view(hip.result_dtype)[0]


class DraftPlanDesc(C.Structure):
    _fields_ = [("model", C.c_void_p), ("workspace", C.c_void_p), ("workspace_bytes", C.c_uint64)] + \
               [(n, C.c_uint32) for n in
                ("position", "materialized", "pending_token", "has_pending", "transaction_active", "poisoned",
                 "checkpoint_position", "checkpoint_materialized", "checkpoint_pending", "checkpoint_has_pending",
                 "backup_end", "last_rows", "logits_valid", "hidden_valid", "checkpoint_hidden_valid",
                 "checkpoint_last_rows", "transaction_rows", "transaction_arena")]


class DraftPlan:
    """The drafter between cycles, with the method names of the reference's Gemma3DraftPlan
    (include/local_gguf_engine/engine/gemma3_draft.hpp:56-82) over guffin_hip_draft_plan_*.  State errors
    raise hip.GuffinError with the C code (GUFFIN_E_STATE = -6, capacity -4, argument -1)."""

    def __init__(self, drafter, transaction_rows=0):
        """transaction_rows: positions one transaction may write (the reference's constructor argument,
        src/engine/gemma3_draft.mm:648-657); 0 = 32."""
        self.drafter = drafter
        lib = hip.lib()
        lib.guffin_hip_draft_plan_bytes.restype = C.c_uint64
        need = lib.guffin_hip_draft_plan_bytes(C.byref(drafter.desc), C.c_uint32(transaction_rows))
        if need == 0:
            raise ValueError("the model cannot carry a draft plan of this transaction capacity (head tiles and rings "
                             "are required; a transaction holds 25 rows or more and fits the smallest ring)")
        self.workspace = torch.zeros(int(need), dtype=torch.uint8, device="cuda")
        self.desc = DraftPlanDesc()
        hip.check(lib.guffin_hip_draft_plan_init(hip._stream(), C.byref(self.desc), C.byref(drafter.desc),
                                                 hip._p(self.workspace), C.c_uint64(need), C.c_uint32(transaction_rows)))

    position = property(lambda self: self.desc.position)
    materialized_position = property(lambda self: self.desc.materialized)
    transaction_active = property(lambda self: bool(self.desc.transaction_active))
    poisoned = property(lambda self: bool(self.desc.poisoned))

    def reset(self):
        hip.check(hip.lib().guffin_hip_draft_plan_reset(hip._stream(), C.byref(self.desc)))

    def begin_transaction(self):
        hip.check(hip.lib().guffin_hip_draft_plan_begin_transaction(hip._stream(), C.byref(self.desc)))

    def commit_prefix(self, position):
        hip.check(hip.lib().guffin_hip_draft_plan_commit_prefix(hip._stream(), C.byref(self.desc), position))

    def abort_transaction(self):
        hip.check(hip.lib().guffin_hip_draft_plan_abort_transaction(hip._stream(), C.byref(self.desc)))

    def can_truncate(self, position):
        return bool(hip.lib().guffin_hip_draft_plan_can_truncate(C.byref(self.desc), position))

    def truncate(self, position):
        hip.check(hip.lib().guffin_hip_draft_plan_truncate(hip._stream(), C.byref(self.desc), position))

    def append(self, tokens):
        arr = (C.c_uint32 * len(tokens))(*[int(t) for t in tokens])
        hip.check(hip.lib().guffin_hip_draft_plan_append(hip._stream(), C.byref(self.desc), arr, len(tokens)))

    def restore_pending_token(self, token):
        hip.check(hip.lib().guffin_hip_draft_plan_restore_pending_token(C.byref(self.desc), int(token)))

    def propose(self, words, options, history=()):
        h = len(words)
        w = (C.c_uint32 * h)(*[int(x) for x in words])
        hist = (C.c_uint32 * max(1, len(history)))(*[int(x) for x in history])
        out = (C.c_uint32 * h)()
        hip.check(hip.lib().guffin_hip_draft_plan_propose(hip._stream(), C.byref(self.desc), w, h, C.byref(options),
                                                          hist if len(history) else None, len(history), out))
        return list(out)

    def read_logits(self):
        out = np.empty(self.drafter.shape.vocab, np.float32)
        hip.check(hip.lib().guffin_hip_draft_plan_read_logits(hip._stream(), C.byref(self.desc), out.ctypes.data_as(C.c_void_p)))
        return out

    def read_cache(self, layer, first_position, count):
        width = self.drafter.shape.kv_width
        k, v = np.empty((count, width), np.uint16), np.empty((count, width), np.uint16)
        hip.check(hip.lib().guffin_hip_draft_plan_read_cache(hip._stream(), C.byref(self.desc), layer, first_position, count,
                                                             k.ctypes.data_as(C.c_void_p), v.ctypes.data_as(C.c_void_p)))
        return k, v
