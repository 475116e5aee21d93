// Host-only driver for the GGUF reader and the weight binding under AddressSanitizer and
// UndefinedBehaviorSanitizer: a small model image is damaged in many ways (flipped bytes, truncations, counts set
// to all ones) in an exactly sized heap copy, so that any read past the end of the file is a heap overflow the
// sanitizer reports, parsed at every depth, listed, and bound.  Built and run by tests/test_gguf_sanitized.py.
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <random>
#include <vector>
#include "guffin_hip.h"
int main(int argc, char** argv) {
    if (argc < 3) { puts("usage: gguf_damage_run IMAGE CASES"); return 2; }
    FILE* f = fopen(argv[1], "rb");
    if (!f) { puts("cannot open the image"); return 2; }
    const int cases = atoi(argv[2]);
    std::vector<uint8_t> image;
    uint8_t buf[65536]; size_t n;
    while ((n = fread(buf, 1, sizeof buf, f)) > 0) image.insert(image.end(), buf, buf + n);
    fclose(f);
    guffin_gguf* g = nullptr;
    if (guffin_gguf_open(image.data(), image.size(), GUFFIN_GGUF_STAGE_MODEL, &g) != 0) { puts("base image refused"); return 1; }
    guffin_gguf_info info; guffin_gguf_summary(g, &info);
    const uint64_t meta_end = info.metadata_end_offset;
    guffin_gguf_close(g);
    std::mt19937_64 rng(1);
    guffin_gemma3_config c {};
    c.block_count = 1; c.embedding_length = 64; c.feed_forward_length = 128; c.vocab_size = 256;
    c.attention_head_count = 4; c.attention_head_count_kv = 1; c.attention_key_length = c.attention_value_length = 256;
    c.sliding_window = 512; c.context_length = 8192; c.attention_global_layer_period = 6; c.uses_qk_norm = 1;
    c.rms_norm_epsilon = 1e-6f; c.rope_freq_base = 1e6f; c.local_rope_freq_base = 1e4f; c.rope_freq_scale = 1.f;
    long ok = 0, bad = 0, bound = 0;
    for (int it = 0; it < cases; ++it) {
        // an exactly sized heap copy, so that a read past the end is a heap overflow the sanitizer sees
        size_t len = image.size();
        const int kind = it % 4;
        if (kind == 1) len = rng() % (meta_end + 8192);
        if (kind == 3) len = meta_end / 2 + rng() % (image.size() - meta_end / 2);
        uint8_t* data = static_cast<uint8_t*>(malloc(len ? len : 1));
        memcpy(data, image.data(), len);
        if (kind == 0) for (int k = 0, m = 1 + rng() % 3; k < m; ++k) { size_t at = rng() % (meta_end + 4096); if (at < len) data[at] = rng(); }
        if (kind == 2) { size_t at = rng() % meta_end; for (int k = 0; k < 8 && at + k < len; ++k) data[at + k] = 0xFF; }
        if (kind == 3) { size_t at = rng() % meta_end; if (at < len) data[at] = rng(); }
        guffin_gguf* h = nullptr;
        const int stage = it % 7 == 0 ? int(rng() % 4) : GUFFIN_GGUF_STAGE_MODEL;
        const int rc = guffin_gguf_open(data, len, stage, &h);
        if (rc == 0) {
            ++ok;
            guffin_gguf_info in; guffin_gguf_summary(h, &in);
            for (uint64_t i = 0; i < in.parsed_entries; ++i) {
                guffin_gguf_entry_info e; guffin_gguf_entry(h, i, &e);
                if (e.type == 9) for (uint64_t k = 0; k < e.count && k < 64; ++k) { uint64_t bits; const char* t; uint64_t tn; guffin_gguf_entry_element(h, i, k, &bits, &t, &tn); if (t && tn) { volatile uint8_t x = t[tn - 1]; (void)x; } }
                if (e.type == 8 && e.text_bytes) { volatile uint8_t x = e.text[e.text_bytes - 1]; (void)x; }
            }
            for (uint64_t i = 0; i < in.parsed_tensors; ++i) {
                guffin_gguf_tensor_info t; guffin_gguf_tensor(h, i, &t);
                if (stage == GUFFIN_GGUF_STAGE_MODEL && t.byte_count) { volatile uint8_t x = data[t.file_offset + t.byte_count - 1]; (void)x; }
            }
            if (stage >= GUFFIN_GGUF_STAGE_DIRECTORY) {
                guffin_gemma3_binding b; guffin_gemma3_block blk[1];
                if (guffin_gguf_bind_gemma3(h, &c, &b, blk) == 0) ++bound;
            }
            guffin_gguf_close(h);
        } else ++bad;
        free(data);
    }
    printf("ok %ld refused %ld bound %ld\n", ok, bad, bound);
    return 0;
}
