// GGUF container reader (host only): header, metadata, tensor directory and payload views.
//
// Follows the reference's validating reader: field order, limits and the error taxonomy of
// src/model_format/gguf_reader.cpp:60-870 with the types of
// include/local_gguf_engine/model_format/{gguf_header,gguf_metadata,gguf_tensor,gguf_reader}.hpp.
// One cursor walks the bytes once; `stage` says how far (the reference exposes the same four
// depths as read_gguf_header / _metadata_section / _tensor_directory / _model_view).  Nothing is
// copied out of the caller's bytes except keys, names and scalar values: payload views are
// offsets into the same buffer, which must outlive the handle.
#include <cstdint>
#include <cstring>
#include <limits>
#include <new>
#include <cmath>
#include <string>
#include <vector>

#include "../../include/guffin_hip.h"

namespace {

constexpr uint64_t kSizeMax = std::numeric_limits<uint64_t>::max();

struct ReadFailure { int code; uint64_t expected, actual; uint8_t magic[4]; };

struct Entry {
    std::string key;
    uint32_t type = 0;           // GGUF metadata value type
    uint32_t element_type = 0;   // for arrays
    uint64_t bits = 0;           // scalar payload, little-endian widened (floats by bit pattern)
    std::string text;            // string payload
    uint64_t count = 0;          // array length
    std::vector<uint64_t> numbers;     // array of scalars (bit patterns)
    std::vector<std::string> strings;  // array of strings
};

struct Tensor {
    std::string name;
    uint32_t n_dims = 0;
    uint64_t dims[4] = {0, 0, 0, 0};
    uint32_t type_id = 0;
    uint64_t offset = 0, file_offset = 0, byte_count = 0;
};

}  // namespace

struct guffin_gguf {
    const uint8_t* bytes = nullptr;
    uint64_t size = 0;
    uint32_t version = 0;
    uint64_t tensor_count = 0, kv_count = 0;
    std::vector<Entry> entries;
    uint64_t metadata_end = 0;
    std::vector<Tensor> tensors;
    uint32_t alignment = 32;
    uint64_t infos_end = 0, padding = 0, data_start = 0;
};

namespace {

class Cursor {
public:
    Cursor(const uint8_t* bytes, uint64_t size) : bytes_(bytes), size_(size) {}
    uint64_t at = 0;

    void need(uint64_t count, int code) const {
        if (at <= size_ && count <= size_ - at) return;
        throw ReadFailure {code, count > kSizeMax - at ? kSizeMax : at + count, size_, {}};
    }
    uint64_t left() const { return at > size_ ? 0 : size_ - at; }
    uint64_t take(unsigned width, int code) {  // little-endian unsigned of 1, 2, 4 or 8 bytes
        need(width, code);
        uint64_t v = 0;
        for (unsigned i = 0; i < width; ++i) v |= uint64_t(bytes_[at + i]) << (8 * i);
        at += width;
        return v;
    }
    std::string text(int code) {
        const uint64_t length = take(8, code);
        need(length, code);
        std::string s(reinterpret_cast<const char*>(bytes_ + at), static_cast<size_t>(length));
        at += length;
        return s;
    }
    uint8_t byte_at(uint64_t i) const { return bytes_[i]; }

private:
    const uint8_t* bytes_;
    uint64_t size_;
};

unsigned scalar_width(uint32_t type) {
    switch (type) {
        case 0: case 1: case 7: return 1;
        case 2: case 3: return 2;
        case 4: case 5: case 6: return 4;
        case 10: case 11: case 12: return 8;
        default: return 0;
    }
}

uint32_t value_type(Cursor& c) {
    const uint32_t raw = static_cast<uint32_t>(c.take(4, GUFFIN_GGUF_TRUNCATED_METADATA));
    if (raw > 12) throw ReadFailure {GUFFIN_GGUF_INVALID_METADATA_VALUE_TYPE, 0, raw, {}};
    return raw;
}

uint64_t scalar(Cursor& c, uint32_t type) {
    const uint64_t v = c.take(scalar_width(type), GUFFIN_GGUF_TRUNCATED_METADATA);
    if (type == 7 && v > 1) throw ReadFailure {GUFFIN_GGUF_INVALID_METADATA_VALUE, 1, v, {}};
    return v;
}

void read_value(Cursor& c, Entry& e) {
    if (e.type == 8) { e.text = c.text(GUFFIN_GGUF_TRUNCATED_METADATA); return; }
    if (e.type != 9) { e.bits = scalar(c, e.type); return; }
    e.element_type = value_type(c);
    e.count = c.take(8, GUFFIN_GGUF_TRUNCATED_METADATA);
    if (e.element_type == 9) throw ReadFailure {GUFFIN_GGUF_UNSUPPORTED_METADATA_VALUE_TYPE, 0, 9, {}};
    const uint64_t reserve = e.count < c.left() ? e.count : c.left();  // a hostile count cannot reserve beyond the file
    if (e.element_type == 8) {
        e.strings.reserve(static_cast<size_t>(reserve));
        for (uint64_t i = 0; i < e.count; ++i) e.strings.push_back(c.text(GUFFIN_GGUF_TRUNCATED_METADATA));
    } else {
        e.numbers.reserve(static_cast<size_t>(reserve));
        for (uint64_t i = 0; i < e.count; ++i) e.numbers.push_back(scalar(c, e.element_type));
    }
}

void parse_header(guffin_gguf& g) {
    if (g.size < 24) throw ReadFailure {GUFFIN_GGUF_TRUNCATED_HEADER, 24, g.size, {}};
    static const uint8_t magic[4] = {0x47, 0x47, 0x55, 0x46};
    if (std::memcmp(g.bytes, magic, 4) != 0) {
        ReadFailure f {GUFFIN_GGUF_INVALID_MAGIC, 4, 4, {}};
        std::memcpy(f.magic, g.bytes, 4);
        throw f;
    }
    Cursor c(g.bytes, g.size);
    c.at = 4;
    g.version = static_cast<uint32_t>(c.take(4, GUFFIN_GGUF_TRUNCATED_HEADER));
    g.tensor_count = c.take(8, GUFFIN_GGUF_TRUNCATED_HEADER);
    g.kv_count = c.take(8, GUFFIN_GGUF_TRUNCATED_HEADER);
}

void parse_metadata(guffin_gguf& g) {
    Cursor c(g.bytes, g.size);
    c.at = 24;
    g.entries.reserve(static_cast<size_t>(g.kv_count < c.left() ? g.kv_count : c.left()));
    for (uint64_t i = 0; i < g.kv_count; ++i) {
        Entry e;
        e.key = c.text(GUFFIN_GGUF_TRUNCATED_METADATA);
        e.type = value_type(c);
        read_value(c, e);
        g.entries.push_back(std::move(e));
    }
    g.metadata_end = c.at;
}

void parse_directory(guffin_gguf& g) {
    Cursor c(g.bytes, g.size);
    c.at = g.metadata_end;
    g.tensors.reserve(static_cast<size_t>(g.tensor_count < c.left() ? g.tensor_count : c.left()));
    for (uint64_t i = 0; i < g.tensor_count; ++i) {
        Tensor t;
        t.name = c.text(GUFFIN_GGUF_TRUNCATED_TENSOR_DIRECTORY);
        if (t.name.size() > 64) throw ReadFailure {GUFFIN_GGUF_INVALID_TENSOR_NAME, 64, t.name.size(), {}};
        t.n_dims = static_cast<uint32_t>(c.take(4, GUFFIN_GGUF_TRUNCATED_TENSOR_DIRECTORY));
        if (t.n_dims > 4) throw ReadFailure {GUFFIN_GGUF_INVALID_TENSOR_DIMENSION_COUNT, 4, t.n_dims, {}};
        for (uint32_t d = 0; d < t.n_dims; ++d) t.dims[d] = c.take(8, GUFFIN_GGUF_TRUNCATED_TENSOR_DIRECTORY);
        t.type_id = static_cast<uint32_t>(c.take(4, GUFFIN_GGUF_TRUNCATED_TENSOR_DIRECTORY));
        t.offset = c.take(8, GUFFIN_GGUF_TRUNCATED_TENSOR_DIRECTORY);
        g.tensors.push_back(std::move(t));
    }
    // general.alignment: the first entry of that name decides; it must be a uint32, non-zero, a multiple of 8
    g.alignment = 32;
    for (const Entry& e : g.entries) {
        if (e.key != "general.alignment") continue;
        if (e.type != 4) throw ReadFailure {GUFFIN_GGUF_INVALID_ALIGNMENT, 4, 0, {}};
        const uint32_t a = static_cast<uint32_t>(e.bits);
        if (a == 0 || a % 8 != 0) throw ReadFailure {GUFFIN_GGUF_INVALID_ALIGNMENT, 8, a, {}};
        g.alignment = a;
        break;
    }
    g.infos_end = c.at;
    const uint64_t rest = g.infos_end % g.alignment;
    g.padding = rest ? g.alignment - rest : 0;
    if (g.padding > kSizeMax - g.infos_end) throw ReadFailure {GUFFIN_GGUF_INVALID_ALIGNMENT, g.alignment, 0, {}};
    g.data_start = g.infos_end + g.padding;
    c.need(g.padding, GUFFIN_GGUF_TRUNCATED_TENSOR_DIRECTORY);
    for (uint64_t i = 0; i < g.padding; ++i)
        if (c.byte_at(g.infos_end + i) != 0)
            throw ReadFailure {GUFFIN_GGUF_INVALID_TENSOR_PADDING, 0, c.byte_at(g.infos_end + i), {}};
    for (Tensor& t : g.tensors) {
        if (t.offset % g.alignment != 0) throw ReadFailure {GUFFIN_GGUF_INVALID_TENSOR_OFFSET, g.alignment, t.offset, {}};
        if (t.offset > kSizeMax - g.data_start) throw ReadFailure {GUFFIN_GGUF_INVALID_TENSOR_OFFSET, 0, 0, {}};
        t.file_offset = g.data_start + t.offset;
    }
}

uint64_t checked_product(uint64_t a, uint64_t b) {
    if (a != 0 && b > kSizeMax / a) throw ReadFailure {GUFFIN_GGUF_INVALID_TENSOR_SIZE, 0, 0, {}};
    return a * b;
}

void parse_payloads(guffin_gguf& g) {
    for (Tensor& t : g.tensors) {
        uint64_t block_elems = 0, block_bytes = 0;
        switch (t.type_id) {  // F32, F16, Q8_0, Q4_K, Q6_K
            case 0: block_elems = 1; block_bytes = 4; break;
            case 1: block_elems = 1; block_bytes = 2; break;
            case 8: block_elems = 32; block_bytes = 34; break;
            case 12: block_elems = 256; block_bytes = 144; break;
            case 14: block_elems = 256; block_bytes = 210; break;
            default: throw ReadFailure {GUFFIN_GGUF_UNSUPPORTED_TENSOR_TYPE, 0, t.type_id, {}};
        }
        uint64_t elements = 1;
        for (uint32_t d = 0; d < t.n_dims; ++d) elements = checked_product(elements, t.dims[d]);
        const uint64_t row = t.n_dims ? t.dims[0] : elements;  // blocks never straddle rows
        if (row % block_elems != 0) throw ReadFailure {GUFFIN_GGUF_INVALID_TENSOR_SIZE, block_elems, row, {}};
        if (elements % block_elems != 0) throw ReadFailure {GUFFIN_GGUF_INVALID_TENSOR_SIZE, block_elems, elements, {}};
        t.byte_count = checked_product(elements / block_elems, block_bytes);
        Cursor c(g.bytes, g.size);
        c.at = t.file_offset;
        c.need(t.byte_count, GUFFIN_GGUF_TRUNCATED_TENSOR_PAYLOAD);
    }
}

thread_local ReadFailure g_last_failure {};

const Entry* entry_at(const guffin_gguf* g, uint64_t index) {
    return g && index < g->entries.size() ? &g->entries[static_cast<size_t>(index)] : nullptr;
}

}  // namespace

extern "C" int guffin_gguf_open(const void* bytes, uint64_t size, int stage, guffin_gguf** out) {
    if (!out || (!bytes && size) || stage < GUFFIN_GGUF_STAGE_HEADER || stage > GUFFIN_GGUF_STAGE_MODEL) return GUFFIN_E_ARG;
    *out = nullptr;
    guffin_gguf* g = new (std::nothrow) guffin_gguf;
    if (!g) return GUFFIN_E_CAPACITY;
    g->bytes = static_cast<const uint8_t*>(bytes);
    g->size = size;
    try {
        parse_header(*g);
        if (stage >= GUFFIN_GGUF_STAGE_METADATA) parse_metadata(*g);
        if (stage >= GUFFIN_GGUF_STAGE_DIRECTORY) parse_directory(*g);
        if (stage >= GUFFIN_GGUF_STAGE_MODEL) parse_payloads(*g);
    } catch (const ReadFailure& f) {
        g_last_failure = f;
        delete g;
        return f.code;
    } catch (const std::bad_alloc&) {
        delete g;
        return GUFFIN_E_CAPACITY;
    }
    *out = g;
    return GUFFIN_OK;
}

extern "C" void guffin_gguf_close(guffin_gguf* g) { delete g; }

extern "C" void guffin_gguf_last_failure(uint64_t* expected, uint64_t* actual, uint8_t magic[4]) {
    if (expected) *expected = g_last_failure.expected;
    if (actual) *actual = g_last_failure.actual;
    if (magic) std::memcpy(magic, g_last_failure.magic, 4);
}

extern "C" int guffin_gguf_summary(const guffin_gguf* g, guffin_gguf_info* out) {
    if (!g || !out) return GUFFIN_E_ARG;
    out->version = g->version;
    out->tensor_count = g->tensor_count;
    out->metadata_kv_count = g->kv_count;
    out->metadata_end_offset = g->metadata_end;
    out->alignment = g->alignment;
    out->tensor_infos_end_offset = g->infos_end;
    out->padding_byte_count = g->padding;
    out->tensor_data_start_offset = g->data_start;
    out->parsed_entries = g->entries.size();
    out->parsed_tensors = g->tensors.size();
    return GUFFIN_OK;
}

extern "C" int guffin_gguf_entry(const guffin_gguf* g, uint64_t index, guffin_gguf_entry_info* out) {
    const Entry* e = entry_at(g, index);
    if (!e || !out) return GUFFIN_E_ARG;
    out->key = e->key.c_str();
    out->type = e->type;
    out->element_type = e->element_type;
    out->bits = e->bits;
    out->text = e->type == 8 ? e->text.c_str() : nullptr;
    out->text_bytes = e->type == 8 ? e->text.size() : 0;
    out->count = e->count;
    return GUFFIN_OK;
}

extern "C" int guffin_gguf_entry_element(const guffin_gguf* g, uint64_t index, uint64_t element, uint64_t* bits,
                                         const char** text, uint64_t* text_bytes) {
    const Entry* e = entry_at(g, index);
    if (!e || e->type != 9 || element >= e->count) return GUFFIN_E_ARG;
    if (e->element_type == 8) {
        const std::string& s = e->strings[static_cast<size_t>(element)];
        if (text) *text = s.c_str();
        if (text_bytes) *text_bytes = s.size();
        if (bits) *bits = 0;
    } else {
        if (bits) *bits = e->numbers[static_cast<size_t>(element)];
        if (text) *text = nullptr;
        if (text_bytes) *text_bytes = 0;
    }
    return GUFFIN_OK;
}

extern "C" int guffin_gguf_find_entry(const guffin_gguf* g, const char* key, uint64_t* index) {
    if (!g || !key || !index) return GUFFIN_E_ARG;
    for (size_t i = 0; i < g->entries.size(); ++i)
        if (g->entries[i].key == key) { *index = i; return GUFFIN_OK; }
    return GUFFIN_E_ARG;
}

extern "C" int guffin_gguf_tensor(const guffin_gguf* g, uint64_t index, guffin_gguf_tensor_info* out) {
    if (!g || !out || index >= g->tensors.size()) return GUFFIN_E_ARG;
    const Tensor& t = g->tensors[static_cast<size_t>(index)];
    out->name = t.name.c_str();
    out->n_dims = t.n_dims;
    for (int d = 0; d < 4; ++d) out->dims[d] = t.dims[d];
    out->type_id = t.type_id;
    out->offset = t.offset;
    out->file_offset = t.file_offset;
    out->byte_count = t.byte_count;
    return GUFFIN_OK;
}

extern "C" int guffin_gguf_find_tensor(const guffin_gguf* g, const char* name, uint64_t* index) {
    if (!g || !name || !index) return GUFFIN_E_ARG;
    for (size_t i = 0; i < g->tensors.size(); ++i)
        if (g->tensors[i].name == name) { *index = i; return GUFFIN_OK; }
    return GUFFIN_E_ARG;
}

// ---- weight binding ---------------------------------------------------------------------------
// bind_gemma_model_weights + validate_gemma3_model_weights (src/engine/gemma_model.cpp:72-177): every tensor
// a Gemma 3 block graph needs is looked up by its GGUF name and checked against the configuration before
// anything is uploaded.  The detail string of a refusal follows the reference's wording.
namespace {
thread_local std::string g_bind_detail;

int refuse(int code, std::string detail) {
    g_bind_detail = std::move(detail);
    return code;
}

constexpr const char* kMatrixNames[7] = {"attn_q", "attn_k", "attn_v", "attn_output", "ffn_gate", "ffn_up", "ffn_down"};
constexpr const char* kNormNames[6] = {"attn_norm", "attn_q_norm", "attn_k_norm", "post_attention_norm", "ffn_norm", "post_ffw_norm"};
constexpr uint32_t kTypeF32 = 0, kTypeQ8 = 8, kTypeQ4K = 12, kTypeQ6K = 14;

std::string block_name(uint32_t block, const char* suffix) {
    return "blk." + std::to_string(block) + "." + suffix + ".weight";
}
}  // namespace

extern "C" const char* guffin_gguf_bind_detail(void) { return g_bind_detail.c_str(); }

extern "C" int guffin_gguf_bind_gemma3(const guffin_gguf* g, const guffin_gemma3_config* c, guffin_gemma3_binding* out,
                                       guffin_gemma3_block* blocks) {
    if (!g || !c || !out || !blocks) return GUFFIN_E_ARG;
    g_bind_detail.clear();
    const auto find = [&](const std::string& name, uint64_t* index) {
        for (size_t i = 0; i < g->tensors.size(); ++i)
            if (g->tensors[i].name == name) { *index = i; return true; }
        return false;
    };
    // bind_gemma_model_weights (:72-103): every tensor is looked up before anything is validated, the blocks first
    // and inside a block in the order of the reference's initialisers (:38-68), so the first name that is absent in
    // that order is the refusal whatever else is wrong with the file or the configuration.
    enum { kAttnNorm = 0, kQNorm = 1, kKNorm = 2, kPostAttnNorm = 3, kFfnNorm = 4, kPostFfwNorm = 5 };
    for (uint32_t b = 0; b < c->block_count; ++b) {
        guffin_gemma3_block& blk = blocks[b];
        const auto need_norm = [&](int i) { return find(block_name(b, kNormNames[i]), &blk.norm[i]) ? 0 : refuse(GUFFIN_BIND_MISSING_TENSOR, block_name(b, kNormNames[i])); };
        const auto need_matrix = [&](int i) { return find(block_name(b, kMatrixNames[i]), &blk.matrix[i]) ? 0 : refuse(GUFFIN_BIND_MISSING_TENSOR, block_name(b, kMatrixNames[i])); };
        if (int rc = need_norm(kAttnNorm)) return rc;
        if (int rc = need_norm(kPostAttnNorm)) return rc;
        for (int i = 0; i < 4; ++i)
            if (int rc = need_matrix(i)) return rc;
        if (c->uses_qk_norm) {
            if (int rc = need_norm(kQNorm)) return rc;
            if (int rc = need_norm(kKNorm)) return rc;
        }
        if (int rc = need_norm(kFfnNorm)) return rc;
        if (int rc = need_norm(kPostFfwNorm)) return rc;
        for (int i = 4; i < 7; ++i)
            if (int rc = need_matrix(i)) return rc;
    }
    if (!find("token_embd.weight", &out->token_embedding)) return refuse(GUFFIN_BIND_MISSING_TENSOR, "token_embd.weight");
    if (!find("output_norm.weight", &out->output_norm)) return refuse(GUFFIN_BIND_MISSING_TENSOR, "output_norm.weight");
    // output_weight_or_tied_embedding (:26-34): output.weight when the file has one, else the embedding
    out->tied_output = find("output.weight", &out->output) ? 0u : 1u;
    if (out->tied_output) out->output = out->token_embedding;

    // validate_gemma3_model_weights (:105-177), in its order.  The execution configuration (:106-119):
    const auto finite_positive = [](float v) { return std::isfinite(v) && v > 0.0f; };
    if (!c->uses_qk_norm || c->attention_global_layer_period != 6 || c->embedding_length == 0 || c->feed_forward_length == 0
        || c->block_count == 0 || c->vocab_size == 0 || c->attention_head_count == 0 || c->attention_head_count_kv == 0
        || c->attention_head_count % c->attention_head_count_kv != 0 || c->attention_key_length == 0
        || c->attention_key_length % 2 != 0 || c->attention_key_length != c->attention_value_length
        || !finite_positive(c->rms_norm_epsilon) || c->attention_logit_softcap != 0.0f || c->final_logit_softcap != 0.0f
        || !finite_positive(c->rope_freq_base) || !finite_positive(c->local_rope_freq_base) || !finite_positive(c->rope_freq_scale))
        return refuse(GUFFIN_BIND_INVALID_TENSOR, "Gemma 3 execution configuration");
    // the target's geometry (:120-124); the drafter (4 query heads on 1 KV head, Q8_0 blocks) is bound without it
    if (c->target_geometry
        && (c->attention_key_length != 256 || uint64_t(c->attention_head_count) != 2 * uint64_t(c->attention_head_count_kv)
            || c->block_count > 64))
        return refuse(GUFFIN_BIND_INVALID_TENSOR, "Gemma 3 target requires 256-wide paired GQA heads and at most 64 layers");
    if (c->context_length < c->sliding_window)
        return refuse(GUFFIN_BIND_INVALID_TENSOR, "Gemma 3 runtime context must cover the local attention window");
    const uint64_t query_width = uint64_t(c->attention_head_count) * c->attention_key_length;
    const uint64_t kv_width = uint64_t(c->attention_head_count_kv) * c->attention_key_length;
    if (query_width > 0xFFFFFFFFull || kv_width > 0xFFFFFFFFull)   // the reference's wording, whatever the device
        return refuse(GUFFIN_BIND_INVALID_TENSOR, "Gemma 3 attention width exceeds Metal indexing range");

    const auto norm = [&](uint64_t index, uint64_t width, const std::string& name) {
        const Tensor& t = g->tensors[static_cast<size_t>(index)];
        if (t.n_dims != 1 || t.dims[0] != width || t.type_id != kTypeF32)
            return refuse(GUFFIN_BIND_INVALID_TENSOR, name + ": expected F32 norm with width " + std::to_string(width));
        return 0;
    };
    const auto matrix = [&](uint64_t index, uint64_t input, uint64_t output, const std::string& name, bool head) {
        const Tensor& t = g->tensors[static_cast<size_t>(index)];
        const bool kquant = head && c->target_geometry ? t.type_id == kTypeQ6K : (t.type_id == kTypeQ4K || t.type_id == kTypeQ6K);
        const bool q8 = !c->target_geometry && t.type_id == kTypeQ8;
        if (t.n_dims != 2 || t.dims[0] != input || t.dims[1] != output || !(kquant || q8) || input % (q8 ? 32 : 256) != 0)
            return refuse(GUFFIN_BIND_INVALID_TENSOR, name + ": expected native " + (c->target_geometry ? (head ? "Q6_K" : "Q4_K/Q6_K") : "Q8_0/Q4_K/Q6_K")
                              + " GGUF matrix [" + std::to_string(input) + ", " + std::to_string(output) + "]");
        return 0;
    };
    if (int rc = matrix(out->token_embedding, c->embedding_length, c->vocab_size, "token_embd.weight", true)) return rc;
    if (int rc = matrix(out->output, c->embedding_length, c->vocab_size, "output.weight", true)) return rc;
    if (c->uses_tied_output_weight && !out->tied_output)
        return refuse(GUFFIN_BIND_INVALID_TENSOR, "Gemma 3 tied output must alias token_embd.weight");
    if (int rc = norm(out->output_norm, c->embedding_length, "output_norm.weight")) return rc;
    const uint64_t in_out[7][2] = {{c->embedding_length, query_width}, {c->embedding_length, kv_width}, {c->embedding_length, kv_width},
                                   {query_width, c->embedding_length}, {c->embedding_length, c->feed_forward_length},
                                   {c->embedding_length, c->feed_forward_length}, {c->feed_forward_length, c->embedding_length}};
    for (uint32_t b = 0; b < c->block_count; ++b) {
        guffin_gemma3_block& blk = blocks[b];
        const auto check_norm = [&](int i, uint64_t width) { return norm(blk.norm[i], width, block_name(b, kNormNames[i])); };
        const auto check_matrix = [&](int i) { return matrix(blk.matrix[i], in_out[i][0], in_out[i][1], block_name(b, kMatrixNames[i]), false); };
        if (int rc = check_norm(kAttnNorm, c->embedding_length)) return rc;
        if (int rc = check_norm(kPostAttnNorm, c->embedding_length)) return rc;
        if (int rc = check_norm(kQNorm, c->attention_key_length)) return rc;
        if (int rc = check_norm(kKNorm, c->attention_key_length)) return rc;
        for (int i = 0; i < 4; ++i)
            if (int rc = check_matrix(i)) return rc;
        if (int rc = check_norm(kFfnNorm, c->embedding_length)) return rc;
        if (int rc = check_norm(kPostFfwNorm, c->embedding_length)) return rc;
        for (int i = 4; i < 7; ++i)
            if (int rc = check_matrix(i)) return rc;
        bool any_q8 = false, any_kquant = false;
        for (int i = 0; i < 7; ++i) {
            blk.type_id[i] = g->tensors[static_cast<size_t>(blk.matrix[i])].type_id;
            (blk.type_id[i] == kTypeQ8 ? any_q8 : any_kquant) = true;
        }
        // the kernels of one block share an activation image: 32-weight and 256-weight formats do not mix in it
        if (any_q8 && any_kquant)
            return refuse(GUFFIN_BIND_INVALID_TENSOR, block_name(b, "attn_q") + ": a block mixes 32-weight and 256-weight formats");
    }
    return GUFFIN_OK;
}
