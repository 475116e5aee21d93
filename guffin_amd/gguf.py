"""ctypes binding of the GGUF container reader in libguffin_hip.so (host only: no GPU needed)."""
import ctypes as C
import struct

import numpy as np

from . import hip

STAGE_HEADER, STAGE_METADATA, STAGE_DIRECTORY, STAGE_MODEL = range(4)
ERRORS = ["truncated_header", "invalid_magic", "truncated_metadata", "invalid_metadata_value_type",
          "invalid_metadata_value", "unsupported_metadata_value_type", "truncated_tensor_directory",
          "invalid_tensor_dimension_count", "invalid_tensor_name", "invalid_alignment", "invalid_tensor_offset",
          "invalid_tensor_padding", "truncated_tensor_payload", "unsupported_tensor_type", "invalid_tensor_size"]


class Info(C.Structure):
    _fields_ = [("version", C.c_uint32), ("alignment", C.c_uint32), ("tensor_count", C.c_uint64),
                ("metadata_kv_count", C.c_uint64), ("metadata_end_offset", C.c_uint64),
                ("tensor_infos_end_offset", C.c_uint64), ("padding_byte_count", C.c_uint64),
                ("tensor_data_start_offset", C.c_uint64), ("parsed_entries", C.c_uint64),
                ("parsed_tensors", C.c_uint64)]


class EntryInfo(C.Structure):
    _fields_ = [("key", C.c_char_p), ("type", C.c_uint32), ("element_type", C.c_uint32), ("bits", C.c_uint64),
                ("text", C.c_void_p), ("text_bytes", C.c_uint64), ("count", C.c_uint64)]


class TensorInfo(C.Structure):
    _fields_ = [("name", C.c_char_p), ("n_dims", C.c_uint32), ("type_id", C.c_uint32), ("dims", C.c_uint64 * 4),
                ("offset", C.c_uint64), ("file_offset", C.c_uint64), ("byte_count", C.c_uint64)]


class Gemma3Config(C.Structure):
    """The GemmaModelConfig fields the weight validation reads (guffin_gemma3_config)."""
    _fields_ = [(n, C.c_uint32) for n in
                ("block_count", "embedding_length", "feed_forward_length", "vocab_size", "attention_head_count",
                 "attention_head_count_kv", "attention_key_length", "attention_value_length", "sliding_window",
                 "context_length", "attention_global_layer_period", "uses_qk_norm", "uses_tied_output_weight",
                 "target_geometry")] + \
               [(n, C.c_float) for n in ("rms_norm_epsilon", "attention_logit_softcap", "final_logit_softcap",
                                         "rope_freq_base", "local_rope_freq_base", "rope_freq_scale")]


class Gemma3Block(C.Structure):
    _fields_ = [("matrix", C.c_uint64 * 7), ("norm", C.c_uint64 * 6), ("type_id", C.c_uint32 * 7), ("pad", C.c_uint32)]


class Gemma3Binding(C.Structure):
    _fields_ = [("token_embedding", C.c_uint64), ("output_norm", C.c_uint64), ("output", C.c_uint64),
                ("tied_output", C.c_uint32), ("pad", C.c_uint32)]


class BindError(ValueError):
    """missing_tensor / invalid_tensor of the reference's EngineModelError, with its detail string."""
    def __init__(self, code, detail):
        self.code = {-120: "missing_tensor", -121: "invalid_tensor"}.get(code, code)
        self.detail = detail
        super().__init__("%s: %s" % (self.code, detail))


class ReadError(Exception):
    def __init__(self, code, expected, actual, magic):
        self.code = ERRORS[-100 - code] if -114 <= code <= -100 else code
        self.expected, self.actual, self.magic = expected, actual, magic
        super().__init__("%s (expected %d, actual %d)" % (self.code, expected, actual))


def _scalar(type_id, bits):
    fmt = {0: "B", 1: "b", 2: "H", 3: "h", 4: "I", 5: "i", 6: "f", 10: "Q", 11: "q", 12: "d"}
    if type_id == 7:
        return bool(bits)
    width = struct.calcsize(fmt[type_id])
    return struct.unpack("<" + fmt[type_id], int(bits).to_bytes(8, "little")[:width])[0]


class Reader:
    """A parsed GGUF buffer; `data` (bytes-like) is kept alive with the handle."""

    def __init__(self, data, stage=STAGE_MODEL):
        self._data = np.frombuffer(data, np.uint8) if not isinstance(data, np.ndarray) else data
        lib = hip.lib()
        lib.guffin_gguf_close.restype = None
        handle = C.c_void_p()
        rc = lib.guffin_gguf_open(self._data.ctypes.data_as(C.c_void_p), C.c_uint64(self._data.size), stage,
                                  C.byref(handle))
        if rc != 0:
            expected, actual, magic = C.c_uint64(), C.c_uint64(), (C.c_uint8 * 4)()
            lib.guffin_gguf_last_failure(C.byref(expected), C.byref(actual), magic)
            raise ReadError(rc, expected.value, actual.value, bytes(magic))
        self._h = handle
        self.info = Info()
        lib.guffin_gguf_summary(self._h, C.byref(self.info))

    def __del__(self):
        if getattr(self, "_h", None):
            hip.lib().guffin_gguf_close(self._h)
            self._h = None

    def entries(self):
        """[(key, type, value)]; arrays come back as lists."""
        lib, out = hip.lib(), []
        for i in range(self.info.parsed_entries):
            e = EntryInfo()
            assert lib.guffin_gguf_entry(self._h, C.c_uint64(i), C.byref(e)) == 0
            if e.type == 8:
                value = C.string_at(e.text, e.text_bytes).decode("utf-8", "replace")
            elif e.type == 9:
                value = []
                for k in range(e.count):
                    bits, text, n = C.c_uint64(), C.c_void_p(), C.c_uint64()
                    assert lib.guffin_gguf_entry_element(self._h, C.c_uint64(i), C.c_uint64(k), C.byref(bits),
                                                         C.byref(text), C.byref(n)) == 0
                    value.append(C.string_at(text, n.value).decode("utf-8", "replace") if e.element_type == 8
                                 else _scalar(e.element_type, bits.value))
            else:
                value = _scalar(e.type, e.bits)
            out.append((e.key.decode("utf-8", "replace"), e.type, value))
        return out

    def metadata(self):
        return {k: v for k, _, v in self.entries()}

    def tensors(self):
        lib, out = hip.lib(), []
        for i in range(self.info.parsed_tensors):
            t = TensorInfo()
            assert lib.guffin_gguf_tensor(self._h, C.c_uint64(i), C.byref(t)) == 0
            out.append({"name": t.name.decode("utf-8", "replace"), "dims": [int(t.dims[d]) for d in range(t.n_dims)], "type_id": t.type_id,
                        "offset": t.offset, "file_offset": t.file_offset, "byte_count": t.byte_count})
        return out

    def tensor(self, name):
        index, t = C.c_uint64(), TensorInfo()
        if hip.lib().guffin_gguf_find_tensor(self._h, name.encode(), C.byref(index)) != 0:
            raise KeyError(name)
        hip.lib().guffin_gguf_tensor(self._h, index, C.byref(t))
        return {"name": name, "dims": [int(t.dims[d]) for d in range(t.n_dims)], "type_id": t.type_id,
                "offset": t.offset, "file_offset": t.file_offset, "byte_count": t.byte_count}

    def has_tensor(self, name):
        index = C.c_uint64()
        return hip.lib().guffin_gguf_find_tensor(self._h, name.encode(), C.byref(index)) == 0

    def bind_gemma3(self, config):
        """guffin_gguf_bind_gemma3: (binding, blocks) of tensor indices, or BindError."""
        lib = hip.lib()
        lib.guffin_gguf_bind_detail.restype = C.c_char_p
        binding, blocks = Gemma3Binding(), (Gemma3Block * max(1, config.block_count))()
        rc = lib.guffin_gguf_bind_gemma3(self._h, C.byref(config), C.byref(binding), blocks)
        if rc != 0:
            raise BindError(rc, lib.guffin_gguf_bind_detail().decode())
        return binding, blocks

    def tensor_at(self, index):
        t = TensorInfo()
        assert hip.lib().guffin_gguf_tensor(self._h, C.c_uint64(index), C.byref(t)) == 0
        return {"name": t.name.decode("utf-8", "replace"), "dims": [int(t.dims[d]) for d in range(t.n_dims)], "type_id": t.type_id,
                "offset": t.offset, "file_offset": t.file_offset, "byte_count": t.byte_count}

    def payload(self, name):
        """Zero-copy view of a tensor's bytes."""
        t = self.tensor(name)
        return self._data[t["file_offset"]:t["file_offset"] + t["byte_count"]]
