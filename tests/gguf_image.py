"""A HostModel written as a GGUF file image, the way a converter lays a Gemma 3 file out: tensor and metadata
names follow the reference (src/engine/gemma_model.cpp:36-116, src/engine/model.cpp:330-390)."""
import struct

import numpy as np

GGUF_TYPE = {0: 8, 1: 12, 2: 14}      # library dtype (Q8_0, Q4_K, Q6_K) -> GGUF tensor type id


def gguf_string(s):
    b = s.encode()
    return struct.pack("<Q", len(b)) + b


def write_gguf(host, alignment=64, drop=(), retype=None, reshape=None, extra=()):
    """drop: tensor names left out; retype / reshape: {name: GGUF type id} / {name: dims} written instead of the
    true ones; extra: (name, dims, type id, array) tensors appended (an output.weight of its own)."""
    sh = host.shape
    md = [("general.architecture", 8, "gemma3"), ("general.alignment", 4, alignment),
          ("gemma3.context_length", 4, 8192), ("gemma3.embedding_length", 4, sh.hidden),
          ("gemma3.block_count", 4, sh.layers), ("gemma3.feed_forward_length", 4, sh.ffn),
          ("gemma3.attention.head_count", 4, sh.q_heads), ("gemma3.attention.head_count_kv", 4, sh.kv_heads),
          ("gemma3.attention.key_length", 4, sh.head_dim), ("gemma3.attention.value_length", 4, sh.head_dim),
          ("gemma3.attention.sliding_window", 4, sh.sliding_window),
          ("gemma3.attention.layer_norm_rms_epsilon", 6, sh.eps), ("gemma3.rope.freq_base", 6, sh.global_base),
          ("gemma3.rope.scaling.type", 8, "linear"), ("gemma3.rope.scaling.factor", 6, 1.0 / sh.global_scale),
          ("tokenizer.ggml.tokens", 9, ["<s>", "</s>"])]
    tensors = [("token_embd.weight", [sh.hidden, sh.vocab], GGUF_TYPE[sh.embed_dtype], host.embed),
               ("output_norm.weight", [sh.hidden], 0, host.out_norm)]
    names = ("attn_q", "attn_k", "attn_v", "attn_output", "ffn_gate", "ffn_up", "ffn_down")
    norms = ("attn_norm", "attn_q_norm", "attn_k_norm", "post_attention_norm", "ffn_norm", "post_ffw_norm")
    for l in range(sh.layers):
        for i, (n, (K, N)) in enumerate(zip(names, sh.proj_shapes())):
            tensors.append(("blk.%d.%s.weight" % (l, n), [K, N], GGUF_TYPE[sh.dtypes_of(l)[i]], host.w[l][i]))
        for i, n in enumerate(norms):
            tensors.append(("blk.%d.%s.weight" % (l, n), [host.norm[l][i].size], 0, host.norm[l][i]))
    tensors += list(extra)
    tensors = [(n, (reshape or {}).get(n, d), (retype or {}).get(n, t), a) for n, d, t, a in tensors if n not in drop]
    out = bytearray(b"GGUF" + struct.pack("<IQQ", 3, len(tensors), len(md)))
    for key, t, v in md:
        out += gguf_string(key) + struct.pack("<I", t)
        if t == 8:
            out += gguf_string(v)
        elif t == 4:
            out += struct.pack("<I", v)
        elif t == 6:
            out += struct.pack("<f", v)
        else:
            out += struct.pack("<IQ", 8, len(v)) + b"".join(gguf_string(x) for x in v)
    offset, payloads = 0, []
    for name, dims, type_id, array in tensors:
        raw = np.ascontiguousarray(array).view(np.uint8).tobytes()
        out += gguf_string(name) + struct.pack("<I", len(dims)) + b"".join(struct.pack("<Q", d) for d in dims)
        out += struct.pack("<IQ", type_id, offset)
        payloads.append((offset, raw))
        offset = (offset + len(raw) + alignment - 1) // alignment * alignment
    out += b"\0" * (-len(out) % alignment)
    start = len(out)
    for off, raw in payloads:
        out += b"\0" * (start + off - len(out)) + raw
    return np.frombuffer(bytes(out), np.uint8)
