"""The GGUF reader against the reference's own fixtures (tests/golden/gguf/*.hex are the data files
of the reference's tests/fixtures) and the values / error codes its tests expect for each
(tests/model_format/gguf_reader_tests.cpp:86-790).  The reference reader does not compile with this
image's g++ 11 (constexpr std::string comparison), so these expectations are what pins the reader."""
import os

import numpy as np
import pytest

HERE = os.path.dirname(os.path.abspath(__file__))


def fixture(name):
    text = open(os.path.join(HERE, "golden", "gguf", name + ".hex")).read()
    data = bytearray()
    for line in text.splitlines():
        line = line.split("#")[0]
        data += bytes.fromhex("".join(line.split()))
    return np.frombuffer(bytes(data), np.uint8)


@pytest.fixture(scope="module")
def gguf():
    from guffin_amd import gguf as module
    return module


def failure(gguf, name, stage):
    with pytest.raises(gguf.ReadError) as info:
        gguf.Reader(fixture(name), stage)
    return info.value


def test_fixed_header(gguf):
    r = gguf.Reader(fixture("valid-header-v3"), gguf.STAGE_HEADER)
    assert (r.info.version, r.info.tensor_count, r.info.metadata_kv_count) == (3, 2, 5)
    raw = bytes([0x47, 0x47, 0x55, 0x46, 3, 0, 0, 0, 8, 7, 6, 5, 4, 3, 2, 1, 0x88, 0x77, 0x66, 0x55, 0x44, 0x33, 0x22, 0x11])
    r = gguf.Reader(np.frombuffer(raw, np.uint8), gguf.STAGE_HEADER)
    assert (r.info.tensor_count, r.info.metadata_kv_count) == (0x0102030405060708, 0x1122334455667788)


def test_header_failures(gguf):
    e = failure(gguf, "invalid-magic", gguf.STAGE_HEADER)
    assert e.code == "invalid_magic" and e.magic == bytes([0x42, 0x41, 0x44, 0x21])
    e = failure(gguf, "truncated-header", gguf.STAGE_HEADER)
    assert (e.code, e.expected, e.actual) == ("truncated_header", 24, 3)
    e = failure(gguf, "truncated-count-data", gguf.STAGE_HEADER)
    assert (e.code, e.expected, e.actual) == ("truncated_header", 24, 16)


def test_metadata_scalars(gguf):
    data = fixture("valid-metadata-scalars")
    r = gguf.Reader(data, gguf.STAGE_METADATA)
    assert (r.info.version, r.info.tensor_count, r.info.metadata_kv_count) == (3, 0, 4)
    assert r.info.metadata_end_offset == data.size
    assert r.entries() == [("general.architecture", 8, "dummy"), ("general.alignment", 4, 32),
                           ("model.context_length", 10, 4096), ("model.use_parallel_residual", 7, True)]


def test_metadata_every_scalar_type(gguf):
    data = fixture("valid-metadata-all-scalars")
    r = gguf.Reader(data, gguf.STAGE_METADATA)
    assert r.info.metadata_end_offset == data.size
    got = r.entries()
    assert [k for k, _, _ in got] == ["test.u8", "test.i8", "test.u16", "test.i16", "test.u32", "test.i32", "test.f32",
                                      "test.bool", "test.string", "test.u64", "test.i64", "test.f64"]
    assert [t for _, t, _ in got] == [0, 1, 2, 3, 4, 5, 6, 7, 8, 10, 11, 12]
    values = [v for _, _, v in got]
    assert values[0] == 0x7F and values[1] == -1 and values[2] == 0x1234 and values[3] == -2
    assert values[4] == 0x12345678 and values[5] == -1 and values[6] == 3.5 and values[8] == "ok"
    assert values[9] == 0x0102030405060708 and values[10] == -2 and values[11] == 3.5


def test_metadata_string_array(gguf):
    r = gguf.Reader(fixture("valid-metadata-string-array"), gguf.STAGE_METADATA)
    assert r.entries() == [("tokenizer.ggml.tokens", 9, ["<s>", "</s>"])]


def test_metadata_failures(gguf):
    assert failure(gguf, "invalid-metadata-type", gguf.STAGE_METADATA).code == "invalid_metadata_value_type"
    assert failure(gguf, "invalid-metadata-bool", gguf.STAGE_METADATA).code == "invalid_metadata_value"
    assert failure(gguf, "unsupported-nested-metadata-array", gguf.STAGE_METADATA).code == "unsupported_metadata_value_type"
    assert failure(gguf, "truncated-metadata-value", gguf.STAGE_METADATA).code == "truncated_metadata"


def test_tensor_directory(gguf):
    data = fixture("valid-tensor-directory")
    r = gguf.Reader(data, gguf.STAGE_DIRECTORY)
    i = r.info
    assert (i.version, i.tensor_count, i.metadata_kv_count) == (3, 2, 1)
    assert r.entries() == [("general.alignment", 4, 32)]
    assert (i.alignment, i.tensor_infos_end_offset, i.padding_byte_count, i.tensor_data_start_offset) == (32, 171, 21, 192)
    assert i.tensor_data_start_offset == data.size
    t = r.tensors()
    assert (t[0]["name"], t[0]["dims"], t[0]["type_id"], t[0]["offset"], t[0]["file_offset"]) == \
        ("tok_embeddings.weight", [4, 8], 0, 0, 192)
    assert (t[1]["name"], t[1]["dims"], t[1]["type_id"], t[1]["offset"], t[1]["file_offset"]) == \
        ("output.weight", [8, 4], 8, 128, 320)
    data = fixture("valid-tensor-directory-default-alignment")
    r = gguf.Reader(data, gguf.STAGE_DIRECTORY)
    i = r.info
    assert (i.tensor_count, i.metadata_kv_count, i.alignment) == (1, 0, 32)
    assert (i.tensor_infos_end_offset, i.padding_byte_count, i.tensor_data_start_offset) == (64, 0, 64) and data.size == 64
    t = r.tensors()[0]
    assert (t["name"], t["dims"], t["offset"], t["file_offset"]) == ("abcdefgh", [8], 0, 64)


def test_tensor_directory_failures(gguf):
    e = failure(gguf, "invalid-tensor-dimension-count", gguf.STAGE_DIRECTORY)
    assert (e.code, e.expected, e.actual) == ("invalid_tensor_dimension_count", 4, 5)
    e = failure(gguf, "invalid-tensor-name", gguf.STAGE_DIRECTORY)
    assert e.code == "invalid_tensor_name" and e.expected == 64 and e.actual > 64
    e = failure(gguf, "invalid-alignment-value", gguf.STAGE_DIRECTORY)
    assert (e.code, e.expected, e.actual) == ("invalid_alignment", 8, 12)
    assert failure(gguf, "invalid-alignment-type", gguf.STAGE_DIRECTORY).code == "invalid_alignment"
    e = failure(gguf, "invalid-tensor-offset-alignment", gguf.STAGE_DIRECTORY)
    assert (e.code, e.expected, e.actual) == ("invalid_tensor_offset", 32, 16)
    assert failure(gguf, "invalid-tensor-padding", gguf.STAGE_DIRECTORY).code == "invalid_tensor_padding"
    assert failure(gguf, "truncated-tensor-directory", gguf.STAGE_DIRECTORY).code == "truncated_tensor_directory"


@pytest.mark.parametrize("name,tensor,dims,type_id,nbytes,first,last", [
    ("valid-tensor-payload-view", "ab", None, 0, 8, 0x00, 0x40),
    ("valid-q8-0-tensor-payload-view", "q8", [32], 8, 34, 0x00, 0x21),
    ("valid-q4-k-tensor-payload-view", "q4", [256], 12, 144, 0x00, 0x7F),
    ("valid-q6-k-tensor-payload-view", "q6", [256], 14, 210, 0x00, 0x40),
    ("valid-f16-tensor-payload-view", "h2", [2], 1, 4, 0x00, 0x40),
])
def test_payload_views(gguf, name, tensor, dims, type_id, nbytes, first, last):
    data = fixture(name)
    r = gguf.Reader(data, gguf.STAGE_MODEL)
    assert r.info.tensor_data_start_offset == 64 and len(r.tensors()) == 1
    t = r.tensor(tensor)
    assert (t["type_id"], t["file_offset"], t["byte_count"]) == (type_id, 64, nbytes)
    if dims is not None:
        assert t["dims"] == dims
    view = r.payload(tensor)
    assert view.size == nbytes and view.ctypes.data == data.ctypes.data + 64      # a view, not a copy
    assert (int(view[0]), int(view[-1])) == (first, last)
    if name == "valid-tensor-payload-view":
        assert int(view[2]) == 0x80 and int(view[6]) == 0x00


def test_payload_failures(gguf):
    assert failure(gguf, "truncated-tensor-payload", gguf.STAGE_MODEL).code == "truncated_tensor_payload"
    gguf.Reader(fixture("truncated-tensor-payload"), gguf.STAGE_DIRECTORY)     # the directory alone is well-formed
    assert failure(gguf, "unsupported-tensor-payload-type", gguf.STAGE_MODEL).code == "unsupported_tensor_type"
    e = failure(gguf, "invalid-q4-k-row-size", gguf.STAGE_MODEL)
    assert (e.code, e.expected, e.actual) == ("invalid_tensor_size", 256, 128)
    assert failure(gguf, "invalid-quantized-tensor-payload-size", gguf.STAGE_MODEL).code == "invalid_tensor_size"


def test_q6_k_row_matrix_fixture(gguf):
    """A whole Q6_K matrix in GGUF row order (tests/tensor/tensor_tests.cpp uses the same file)."""
    r = gguf.Reader(fixture("valid-q6-k-gguf-row-matrix"), gguf.STAGE_MODEL)
    t = r.tensors()
    assert len(t) == 1 and t[0]["type_id"] == 14 and t[0]["byte_count"] == (np.prod(t[0]["dims"]) // 256) * 210


def test_arguments(gguf):
    import ctypes as C
    from guffin_amd import hip
    handle = C.c_void_p()
    assert hip.lib().guffin_gguf_open(None, C.c_uint64(8), 0, C.byref(handle)) == -1
    assert hip.lib().guffin_gguf_open(None, C.c_uint64(0), 7, C.byref(handle)) == -1
    with pytest.raises(gguf.ReadError):
        gguf.Reader(np.zeros(0, np.uint8), gguf.STAGE_HEADER)


def test_damaged_images_end_in_a_defined_error(gguf):
    """The reader validates every count and offset before it uses it (src/model_format/gguf_reader.cpp walks the
    file the same way): flipped bytes, truncations and oversized counts anywhere in the header, metadata and
    tensor directory of a small model image give one of the 15 error codes or a parse that can be listed and bound
    (or refused) - never a fault."""
    from dataclasses import replace
    from guffin_amd import model
    from gguf_image import write_gguf
    shape = replace(model.GEMMA3_270M, layers=1, vocab=256, hidden=64, ffn=128)
    image = np.array(write_gguf(model.HostModel(shape, seed=1, position=0)))
    meta_end = int(gguf.Reader(image).info.metadata_end_offset)
    config = gguf.Gemma3Config()
    config.block_count, config.embedding_length, config.feed_forward_length, config.vocab_size = 1, 64, 128, 256
    config.attention_head_count, config.attention_head_count_kv = 4, 1
    config.attention_key_length = config.attention_value_length = 256
    config.sliding_window, config.context_length, config.attention_global_layer_period, config.uses_qk_norm = 512, 8192, 6, 1
    config.rms_norm_epsilon, config.rope_freq_base, config.local_rope_freq_base, config.rope_freq_scale = 1e-6, 1e6, 1e4, 1.0
    gguf.Reader(image).bind_gemma3(config)
    rng = np.random.default_rng(0)
    seen = set()
    for case in range(3000):
        data = image.copy()
        kind = case % 4
        if kind == 0:
            for _ in range(rng.integers(1, 4)):
                data[rng.integers(0, meta_end + 4096)] = rng.integers(0, 256)
        elif kind == 1:
            data = data[:rng.integers(0, meta_end + 8192)]
        elif kind == 2:
            at = int(rng.integers(0, meta_end))
            data[at:at + 8] = 0xFF
        else:
            data[rng.integers(0, meta_end)] = rng.integers(0, 256)
            data = data[:rng.integers(meta_end // 2, data.size)]
        try:
            reader = gguf.Reader(np.ascontiguousarray(data))
        except gguf.ReadError as error:
            assert error.code in gguf.ERRORS, error.code
            seen.add(error.code)
            continue
        assert len(reader.entries()) == reader.info.parsed_entries and len(reader.tensors()) == reader.info.parsed_tensors
        try:
            reader.bind_gemma3(config)
        except gguf.BindError as error:
            assert error.code in ("missing_tensor", "invalid_tensor")
            seen.add(error.code)
    assert {"truncated_metadata", "truncated_tensor_payload", "invalid_metadata_value_type", "truncated_tensor_directory"} <= seen
