// Host side of the H1 step above the kernel C ABI: the Gemma-3 block graph for a few
// contiguous rows, and one speculative cycle (draft 1 token, verify 2 rows, accept).
//
// Mirrors, in structure and operator order:
//   encode_gemma_target_blocks            src/engine/gemma_target_runtime.cpp:13-221
//   stage_contiguous_rows                 src/engine/gemma_target_runtime.cpp:238-271
//   run_gemma_target_width_two_verifier   src/engine/gemma_target_runtime.cpp:457-519
//   Gemma3DraftPlan forward / project     src/engine/gemma3_draft.mm:888-993
//   one H1 cycle                          src/engine/standalone_chat.cpp:508-615,
//                                         src/engine/chain_chat.mm:245-543
// Like the reference's command context it allocates nothing: weights, KV rings and the
// scratch arena are the caller's; everything is enqueued in order on one HIP stream, so a
// caller can capture a whole step into a HIP graph.
#include <cstddef>
#include "common.hpp"
#include "selection_request.hpp"
#include "receipt.hpp"

#include <algorithm>
#include <vector>
#include <cmath>
#include <cstring>

namespace guffin {
namespace {

// history window of the reference's sampler (token_sampler history, 64 tokens)
constexpr uint32_t kHistoryWindow = 64;

struct Arena {
    uint8_t* base; uint64_t used, capacity;
    template <typename T> T* take(uint64_t count) {
        used = (used + 255) & ~uint64_t{255};
        T* p = base ? reinterpret_cast<T*>(base + used) : nullptr;
        used += count * sizeof(T);
        return p;
    }
};

// private rows a verify tree may hold (rows of one pass are at most 2; a tree takes several passes)
constexpr uint32_t kMaxTreeSlots = 8;

struct Scratch {
    float *x, *x1, *u, *us, *q, *a, *as, *h, *hs;
    float *part_a, *part_b, *part_c;          // GEMV partial planes (largest users: gate / up / down)
    float *attn_out, *attn_ml;
    float *rope_local, *rope_global;          // [rows][head_dim/2][2] cos/sin per frequency base
    uint32_t *positions, *ancestors, *schedule;
    uint8_t* exchange;        // the resident pass's exchange buffers (models it covers)
    uint32_t* sync;           // its barrier counters, cleared by the row-staging kernel
    uint32_t sync_words;
    uint64_t bytes;
};

uint32_t slices(int dtype, uint32_t K, uint32_t N) { return guffin_hip_gemv_packed_slices(dtype, K, N); }
// floats in the activation receipt of `rows` rows of `width`
uint64_t receipt_floats(uint32_t rows, uint32_t width) { return receipt_layout(rows, width).bytes / 4; }
// floats from the start of a [rows][width] block to its receipt (256-byte aligned) and the total
uint64_t hidden_receipt_offset(uint32_t rows, uint32_t width) { return (uint64_t(rows) * width + 63) & ~uint64_t{63}; }
uint64_t hidden_with_receipt(uint32_t rows, uint32_t width) { return hidden_receipt_offset(rows, width) + receipt_floats(rows, width); }
uint32_t qkv_slices(const guffin_layer_desc& L, uint32_t H, uint32_t QW, uint32_t KW) {
    const uint32_t n[3] = {QW, KW, KW};
    return guffin_hip_gemv_packed_multi_slices(3, L.dtype, n, H);
}
uint32_t ffn_slices(const guffin_layer_desc& L, uint32_t H, uint32_t F) {
    const uint32_t n[2] = {F, F};
    return guffin_hip_gemv_packed_multi_slices(2, L.dtype + 4, n, H);
}

bool is_local(const guffin_model_desc& m, uint32_t layer) { return layer_is_local(m.global_period, layer); }

// longest token list an attention call of this model can see at `position` with `rows` rows
uint32_t max_tokens_for(const guffin_model_desc& m, uint32_t layer, uint32_t position, uint32_t rows) {
    if (is_local(m, layer)) {
        const uint32_t w = m.sliding_window;
        return (position < w ? position : w) + rows;
    }
    return position + rows;
}

Scratch layout(const guffin_model_desc& m, uint32_t rows, uint32_t position, uint8_t* base) {
    Arena ar {base, 0, 0};
    const uint32_t H = m.hidden, F = m.ffn, QW = m.q_heads * m.head_dim, KW = m.kv_heads * m.head_dim;
    Scratch s {};
    s.x = ar.take<float>(uint64_t(rows) * H);
    s.x1 = ar.take<float>(uint64_t(rows) * H);
    s.u = ar.take<float>(uint64_t(rows) * H);
    s.us = ar.take<float>(receipt_floats(rows, H));
    s.q = ar.take<float>(uint64_t(rows) * QW);
    s.a = ar.take<float>(uint64_t(rows) * QW);
    s.as = ar.take<float>(receipt_floats(rows, QW));
    s.h = ar.take<float>(uint64_t(rows) * F);
    s.hs = ar.take<float>(receipt_floats(rows, F));
    // partial planes: a <- q / o / gate / down, b <- k / up, c <- v
    uint64_t pa = 0, pb = 0, pc = 0;
    for (uint32_t l = 0; l < m.layer_count; ++l) {
        const guffin_layer_desc& L = m.layers[l];
        auto need = [&](int i, uint32_t K, uint32_t N) { return uint64_t(slices(L.dtype[i], K, N)) * rows * N; };
        const uint64_t sq = qkv_slices(L, H, QW, KW), sf = ffn_slices(L, H, F);
        pa = std::max({pa, sq * rows * QW, need(3, QW, H), sf * rows * F, need(6, F, H)});
        pb = std::max({pb, sq * rows * KW, sf * rows * F});
        pc = std::max(pc, sq * rows * KW);
    }
    s.part_a = ar.take<float>(pa);
    s.part_b = ar.take<float>(pb);
    s.part_c = ar.take<float>(pc);
    // partitions of the longest token list, and of any shorter one: the partition length shrinks with the list
    // (down to 16 tokens, while fewer than 256 workgroups would run), so a shorter list can have more of them
    uint32_t max_parts = 1;
    for (uint32_t l = 0; l < m.layer_count; ++l) {
        const uint32_t longest = max_tokens_for(m, l, position, rows);
        const uint32_t shorter = std::min((512u + m.kv_heads - 1) / m.kv_heads, (longest + 15) / 16);
        max_parts = std::max({max_parts, guffin_hip_attention_partitions(longest, m.kv_heads), shorter});
    }
    s.attn_out = ar.take<float>(uint64_t(rows) * m.q_heads * max_parts * m.head_dim);
    s.attn_ml = ar.take<float>(uint64_t(rows) * m.q_heads * max_parts * 2);
    s.rope_local = ar.take<float>(uint64_t(rows) * m.head_dim);
    s.rope_global = ar.take<float>(uint64_t(rows) * m.head_dim);
    s.positions = ar.take<uint32_t>(rows);
    s.ancestors = ar.take<uint32_t>(uint64_t(rows) * kMaxTreeSlots);   // a chain uses `rows` of them, a tree pass one list per row
    s.schedule = ar.take<uint32_t>(uint64_t(m.layer_count) * rows * 4);
    if (resident_fits(m, rows)) {
        s.exchange = ar.take<uint8_t>(resident_scratch_bytes(m, rows));
        s.sync_words = resident_sync_words(m);
        s.sync = ar.take<uint32_t>(s.sync_words);
    }
    s.bytes = (ar.used + 255) & ~uint64_t{255};
    return s;
}

// The schedule words of row `row` of a pass of contiguous rows at `position`: first ring position, ring count,
// first private row, private row count.
__host__ __device__ inline void row_schedule_words(bool local, uint32_t window, uint32_t position, uint32_t row, uint32_t (&s)[4]) {
    const uint32_t p = position + row;
    const uint32_t window_start = (local && p >= window) ? p + 1 - window : 0;
    const uint32_t base_start = position < window_start ? position : window_start;
    const uint32_t private_start = window_start > position ? window_start - position : 0;
    s[0] = base_start; s[1] = position - base_start; s[2] = private_start; s[3] = row + 1 - private_start;
}
// the same on the host, with a bit per private row the row attends (a contiguous pass's ancestor list is 0, 1, 2, ..)
void row_schedule(const guffin_model_desc& m, uint32_t layer, uint32_t position, uint32_t row, uint32_t (&s)[4], uint32_t& amask) {
    row_schedule_words(layer_is_local(m.global_period, layer), m.sliding_window, position, row, s);
    amask = 0;
    for (uint32_t i = 0; i < s[3]; ++i) amask |= 1u << (s[2] + i);
}

// positions, ancestors, the per-layer attention schedule of `rows` contiguous rows and the two
// rotation tables (local and global frequency base) of the pass
__global__ void stage_rows_kernel(uint32_t* positions, uint32_t* ancestors, uint32_t* schedule, uint32_t rows,
                                  uint32_t position, uint32_t layers, uint32_t window, uint32_t global_period,
                                  float2* rope_local, float2* rope_global, uint32_t rope_dim, float local_base,
                                  float global_base, float global_scale, uint32_t* sync, uint32_t sync_words) {
    const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < sync_words) sync[i] = 0u;   // barrier counters of the resident pass start at zero
    const uint32_t half = rope_dim / 2;
    if (i < rows * half) {
        float c, s;
        if (global_period > 1) {  // a model without local blocks has no local base
            rope_sincos(position + i / half, i % half, rope_dim, local_base, 1.0f, c, s);
            rope_local[i] = make_float2(c, s);
        }
        rope_sincos(position + i / half, i % half, rope_dim, global_base, global_scale, c, s);
        rope_global[i] = make_float2(c, s);
    }
    if (i < rows) { positions[i] = position + i; ancestors[i] = i; }
    if (i >= layers * rows) return;
    const uint32_t layer = i / rows, row = i % rows;
    uint32_t words[4];
    row_schedule_words(layer_is_local(global_period, layer), window, position, row, words);
    uint32_t* s = schedule + 4 * i;
    s[0] = words[0]; s[1] = words[1]; s[2] = words[2]; s[3] = words[3];
}

int validate_model(const guffin_model_desc* m) {
    if (!m || !m->layers || !m->embed_rows || !m->out_norm) return fail(GUFFIN_E_ARG, "forward: null model field");
    if (m->head_dim != 256) return fail(GUFFIN_E_SHAPE, "forward: head_dim must be 256");
    if (m->layer_count == 0) return fail(GUFFIN_E_SHAPE, "forward: the model has no blocks");
    if (m->hidden % 64 || m->ffn % 64 || m->kv_heads == 0 || m->q_heads % m->kv_heads)
        return fail(GUFFIN_E_SHAPE, "forward: widths must be multiples of 64 and q_heads a multiple of kv_heads");
    if ((m->ring_local & (m->ring_local - 1)) || (m->ring_global & (m->ring_global - 1)) || !m->ring_local || !m->ring_global)
        return fail(GUFFIN_E_ARG, "forward: ring capacities must be powers of two");
    return GUFFIN_OK;
}

#define GUFFIN_TRY(expr) do { if (int rc_ = (expr)) return rc_; } while (0)

// The rows of a pass at `position` must fit the rings they are published to and read from: global
// layers address [0, position + rows) through the mask, so the global rings must hold all of it; a
// local layer reads the window - 1 positions before a row from its ring.
int check_ring_capacity(const guffin_model_desc& m, uint32_t position, uint32_t rows, const char* what) {
    if (uint64_t(position) + rows > m.ring_global) return fail(GUFFIN_E_CAPACITY, what);
    if (m.global_period > 1 && m.sliding_window > 0 && m.sliding_window - 1 > m.ring_local) return fail(GUFFIN_E_CAPACITY, what);
    return GUFFIN_OK;
}

// A block after its attention: o-projection, the two norm joints, gate/up with GeGLU, down.  s.a / s.as hold
// the attention rows and their receipt, s.x the residual rows; leaves the next block's normalised rows in
// s.u / s.us (the last block: the output-normed rows in out_hidden / out_hidden_sums).
int block_tail(void* st, const guffin_model_desc& m, uint32_t l, const Scratch& s, uint32_t rows, float* out_hidden,
               float* out_hidden_sums, uint32_t* status) {
    const guffin_layer_desc& L = m.layers[l];
    const uint32_t H = m.hidden, F = m.ffn, QW = m.q_heads * m.head_dim;
    GUFFIN_TRY(guffin_hip_gemv_packed(st, L.dtype[3], L.tiles[3], s.a, s.as, s.part_a, nullptr, rows, QW, H));
    // x1 = x + rms(o, post_attention_norm); u = rms(x1, ffn_norm)
    GUFFIN_TRY(guffin_hip_rms_norm_add_norm(st, s.part_a, slices(L.dtype[3], QW, H), uint64_t(rows) * H, L.norm[3],
                                            s.x, s.x1, L.norm[4], s.u, s.us, rows, H, m.eps, status));
    if (L.dtype[4] == L.dtype[5] && L.dtype[4] != GUFFIN_Q6_K) {
        GUFFIN_TRY(guffin_hip_gateup_geglu(st, L.dtype[4], L.tiles[4], L.tiles[5], s.u, s.us, s.h, s.hs, rows, H, F));
    } else {
        const int dt[2] = {L.dtype[4], L.dtype[5]};
        const void* tl[2] = {L.tiles[4], L.tiles[5]};
        const uint32_t n[2] = {F, F};
        float* parts[2] = {s.part_a, s.part_b};
        GUFFIN_TRY(guffin_hip_gemv_packed_multi(st, 2, dt, tl, n, parts, s.u, s.us, rows, H));
        GUFFIN_TRY(guffin_hip_geglu(st, s.part_a, s.part_b, ffn_slices(L, H, F), uint64_t(rows) * F, s.h, s.hs, rows, F));
    }
    GUFFIN_TRY(guffin_hip_gemv_packed(st, L.dtype[6], L.tiles[6], s.h, s.hs, s.part_a, nullptr, rows, F, H));
    // x = x1 + rms(down, post_ffw_norm); u = rms(x, next block's attn_norm | output_norm)
    const bool last = l + 1 == m.layer_count;
    const float* gamma_next = last ? m.out_norm : m.layers[l + 1].norm[0];
    GUFFIN_TRY(guffin_hip_rms_norm_add_norm(st, s.part_a, slices(L.dtype[6], F, H), uint64_t(rows) * H, L.norm[5],
                                            s.x1, s.x, gamma_next, last ? out_hidden : s.u,
                                            last ? out_hidden_sums : s.us, rows, H, m.eps, status));
    return GUFFIN_OK;
}

int forward_rows(hipStream_t stream, const guffin_model_desc& m, const uint32_t* tokens, uint32_t rows,
                 uint32_t position, const Scratch& s, void* priv_k, void* priv_v, float* out_hidden,
                 float* out_hidden_sums, uint32_t* status) {
    void* st = stream;
    const uint32_t H = m.hidden, F = m.ffn, QW = m.q_heads * m.head_dim, KW = m.kv_heads * m.head_dim;
    const float attn_scale = 1.0f / std::sqrt(static_cast<float>(m.head_dim));
    // the resident pass is the default where it is the faster one: models with a single KV head (the drafter's
    // small blocks); it can be forced for any model it covers
    const bool resident = s.exchange != nullptr && resident_chosen(m, rows);
    if (g_forward_mode == 2 && !resident) return fail(GUFFIN_E_SHAPE, "forward: the resident pass does not cover this model");
    const uint32_t sync_words = resident ? s.sync_words : 0u;
    const uint32_t n_stage = std::max({m.layer_count * rows, rows * (m.head_dim / 2), sync_words});
    launch(stage_rows_kernel, dim3((n_stage + 63) / 64), dim3(64), 0, stream, s.positions, s.ancestors,
                       s.schedule, rows, position, m.layer_count, m.sliding_window, m.global_period,
                       reinterpret_cast<float2*>(s.rope_local), reinterpret_cast<float2*>(s.rope_global), m.head_dim,
                       m.local_base, m.global_base, m.global_scale, s.sync, sync_words);
    GUFFIN_TRY(check_launch("stage_rows"));
    GUFFIN_TRY(guffin_hip_embed(st, m.embed_dtype, m.embed_rows, tokens, s.x, rows, H,
                                std::sqrt(static_cast<float>(H)), m.vocab, status));
    GUFFIN_TRY(guffin_hip_rms_norm(st, s.x, 1, 0, m.layers[0].norm[0], nullptr, s.u, s.us, rows, H, m.eps, status));
    if (resident) {
        // groups of blocks, each one launch whose workgroups stay on the chip; the residual rows and the
        // normalised rows' receipt pass from launch to launch through s.x / s.us
        uint32_t ring_tokens = 0;
        for (uint32_t l = 0; l < m.layer_count; ++l) ring_tokens = std::max(ring_tokens, max_tokens_for(m, l, position, rows) - rows);
        const uint32_t words_per_launch = s.sync_words / ((m.layer_count + kResidentLayers - 1) / kResidentLayers);
        for (uint32_t first = 0, n = 0; first < m.layer_count; first += kResidentLayers, ++n) {
            const uint32_t count = std::min(kResidentLayers, m.layer_count - first);
            const bool last = first + count == m.layer_count;
            GUFFIN_TRY(resident_launch(stream, m, rows, first, count, s.exchange, s.sync + size_t(n) * words_per_launch,
                                       s.rope_local, s.rope_global, s.schedule, s.ancestors, priv_k, priv_v, s.x, s.us, s.x,
                                       last ? out_hidden : s.u, last ? static_cast<void*>(out_hidden_sums) : static_cast<void*>(s.us),
                                       ring_tokens, status));
        }
        return GUFFIN_OK;
    }
    for (uint32_t l = 0; l < m.layer_count; ++l) {
        const guffin_layer_desc& L = m.layers[l];
        const bool local = is_local(m, l);
        const uint32_t ring_mask = (local ? m.ring_local : m.ring_global) - 1;
        uint16_t* pk = static_cast<uint16_t*>(priv_k) + size_t(l) * rows * KW;
        uint16_t* pv = static_cast<uint16_t*>(priv_v) + size_t(l) * rows * KW;
        {   // q, k, v projections of the normalised rows
            const int dt[3] = {L.dtype[0], L.dtype[1], L.dtype[2]};
            const void* tl[3] = {L.tiles[0], L.tiles[1], L.tiles[2]};
            const uint32_t n[3] = {QW, KW, KW};
            float* parts[3] = {s.part_a, s.part_b, s.part_c};
            GUFFIN_TRY(guffin_hip_gemv_packed_multi(st, 3, dt, tl, n, parts, s.u, s.us, rows, H));
            const uint32_t sq = qkv_slices(L, H, QW, KW);
            if (sq == 0) return fail(GUFFIN_E_SHAPE, "forward: q, k and v must share the block length");
            // head norms, rotation, fp16 K/V rows and the attention itself in one pass over the planes; the
            // rows are contiguous and the position is the host's, so the schedule words stage_rows_kernel
            // writes are known here too and travel with the launch
            uint32_t host_schedule[2][4], host_amask[2];
            for (uint32_t row = 0; row < rows; ++row) row_schedule(m, l, position, row, host_schedule[row], host_amask[row]);
            GUFFIN_TRY(qkv_attention_scheduled(st, s.part_a, s.part_b, s.part_c, sq, uint64_t(rows) * QW, uint64_t(rows) * KW,
                                               uint64_t(rows) * KW, L.norm[1], L.norm[2],
                                               local ? s.rope_local : s.rope_global, m.eps, L.ring_k, L.ring_v, pk, pv,
                                               s.schedule + size_t(l) * rows * 4, s.ancestors, &host_schedule[0][0], host_amask,
                                               s.a, s.as, s.attn_out, s.attn_ml, rows, max_tokens_for(m, l, position, rows),
                                               ring_mask, m.q_heads, m.kv_heads, m.head_dim, attn_scale, status));
        }
        GUFFIN_TRY(block_tail(st, m, l, s, rows, out_hidden, out_hidden_sums, status));
    }
    return GUFFIN_OK;
}

// publishes the verified rows: row 0 always, row 1 if the proposal was accepted
__global__ void commit_rows_kernel(const uint16_t* priv_k, const uint16_t* priv_v, uint16_t* const* ring_k,
                                   uint16_t* const* ring_v, const uint32_t* accepted, uint32_t position, uint32_t rows,
                                   uint32_t row_width, uint32_t mask_local, uint32_t mask_global, uint32_t global_period) {
    const uint32_t layer = blockIdx.y, row = blockIdx.z;
    const uint32_t publish = accepted ? 1u + (*accepted != 0u) : rows;
    if (row >= publish || row >= rows) return;
    const bool local = layer_is_local(global_period, layer);
    const uint32_t mask = local ? mask_local : mask_global;
    const size_t src = (size_t(layer) * rows + row) * row_width, dst = size_t((position + row) & mask) * row_width;
    for (uint32_t c = blockIdx.x * blockDim.x + threadIdx.x; c < row_width; c += gridDim.x * blockDim.x) {
        ring_k[layer][dst + c] = priv_k[src + c];
        ring_v[layer][dst + c] = priv_v[src + c];
    }
}

// the caller's history (target ids) in the drafter's ids; a token without a draft id matches nothing
__global__ void draft_history_kernel(const uint32_t* history, uint32_t count, const int32_t* target_to_draft, uint32_t vocab,
                                     uint32_t* out) {
    const uint32_t t = threadIdx.x;
    if (t >= count) return;
    const uint32_t token = history[t];
    const int32_t d = token < vocab ? target_to_draft[token] : -1;
    out[t] = d < 0 ? 0xFFFFFFFFu : static_cast<uint32_t>(d);
}

// The two verify rows' selection requests: row 0 sees the caller's history, row 1 the same after the
// proposal has been observed (a full window drops its oldest token), each without duplicates as the
// sampler lists them (src/engine/sampling.cpp:352-378).  out: two resolved records, then the two lists
// [2][64], then the two counts.  A history token outside the vocabulary is skipped and flagged.
constexpr uint32_t kHistLists = 2 * sizeof(ResolvedRow) / 4, kHistCounts = kHistLists + 2 * kHistoryWindow,
                   kHistDraft = kHistCounts + 2, kHistWords = kHistDraft + kHistoryWindow;
__global__ void __launch_bounds__(128)
build_history_kernel(const uint32_t* history, uint32_t count, const uint32_t* proposal, uint32_t vocab, uint32_t top_k,
                     uint32_t* out, uint32_t* status) {
    __shared__ uint32_t suffix[1];
    const uint32_t row = threadIdx.x >> 6, lane = threadIdx.x & 63;
    if (threadIdx.x == 0) suffix[0] = *proposal;
    __syncthreads();
    uint32_t token = 0, st = 0;
    const uint32_t kept = resolve_history(history, 0, count, kHistoryWindow, suffix, row, vocab, true, lane, token, st);
    ResolvedRow& record = reinterpret_cast<ResolvedRow*>(out)[row];
    record.history_token_ids[lane] = token;
    out[kHistLists + row * kHistoryWindow + lane] = token;
    if (lane == 0) {
        record.top_k = top_k;
        record.base_candidate_count = top_k + kept;
        record.history_count = kept;
        record.reserved = 0;
        out[kHistCounts + row] = kept;
        if (st && status) atomicOr(status, GUFFIN_STATUS_BAD_TOKEN);
    }
}

// the step's token slots: [0] root, [1] proposal (written later), [8..] the drafter's input rows
// With a vocabulary map the drafter's rows are the same tokens in its own ids; a token it does not
// have raises GUFFIN_STATUS_BAD_TOKEN (the reference refuses such a root on the host).
__global__ void set_step_tokens_kernel(const uint32_t* root, const uint32_t* pending, uint32_t* words,
                                       const int32_t* target_to_draft, uint32_t target_vocab, uint32_t* status) {
    auto drafter_id = [&](uint32_t token) {
        if (!target_to_draft) return token;
        const int32_t d = token < target_vocab ? target_to_draft[token] : -1;
        if (d < 0) { atomicOr(status, GUFFIN_STATUS_BAD_TOKEN); return 0u; }
        return static_cast<uint32_t>(d);
    };
    words[0] = *root;
    if (pending) { words[8] = drafter_id(*pending); words[9] = drafter_id(*root); } else { words[8] = drafter_id(*root); }
}

}  // namespace
}  // namespace guffin

using namespace guffin;

extern "C" uint64_t guffin_hip_forward_scratch_bytes(const guffin_model_desc* model, uint32_t rows, uint32_t position) {
    if (validate_model(model) || rows == 0 || rows > 2) return 0;
    return layout(*model, rows, position, nullptr).bytes;
}

extern "C" int guffin_hip_forward_rows(void* stream, const guffin_model_desc* model, const uint32_t* tokens,
                                       uint32_t rows, uint32_t position, void* scratch, uint64_t scratch_bytes,
                                       void* priv_k, void* priv_v, float* out_hidden, float* out_hidden_sums,
                                       uint32_t* status) {
    GUFFIN_TRY(validate_model(model));
    if (!tokens || !scratch || !priv_k || !priv_v || !out_hidden || !status) return fail(GUFFIN_E_ARG, "forward_rows: null pointer");
    if (rows == 0 || rows > 2) return fail(GUFFIN_E_SHAPE, "forward_rows: rows must be 1 or 2");
    GUFFIN_TRY(check_ring_capacity(*model, position, rows, "forward_rows: the rows do not fit the KV rings"));
    if (reinterpret_cast<uintptr_t>(scratch) & 255u) return fail(GUFFIN_E_ALIGN, "forward_rows: scratch must be 256-byte aligned");
    const Scratch s = layout(*model, rows, position, static_cast<uint8_t*>(scratch));
    if (s.bytes > scratch_bytes) return fail(GUFFIN_E_CAPACITY, "forward_rows: scratch arena too small");
    return forward_rows(as_stream(stream), *model, tokens, rows, position, s, priv_k, priv_v, out_hidden,
                        out_hidden_sums, status);
}

// ---- rows of a verify tree -------------------------------------------------------------------
// One pass of 1 or 2 rows whose parents may be any earlier row of the tree: a row's token list is the ring
// below `base_position` (through the layer's window) followed by its ancestors among the tree's private
// rows, itself last.  The rows' own K/V go to consecutive private slots; attention reads every slot an
// ancestor list names, also those an earlier pass of the same tree wrote.
extern "C" int guffin_hip_forward_tree_rows(void* stream, const guffin_model_desc* model, const uint32_t* tokens, uint32_t rows,
                                            uint32_t base_position, const uint32_t* depths, const uint32_t* ancestor_lists,
                                            const uint32_t* ancestor_counts, uint32_t first_slot, uint32_t slot_count,
                                            void* scratch, uint64_t scratch_bytes, void* priv_k, void* priv_v,
                                            float* out_hidden, float* out_hidden_sums, uint32_t* status) {
    GUFFIN_TRY(validate_model(model));
    if (!tokens || !depths || !ancestor_lists || !ancestor_counts || !scratch || !priv_k || !priv_v || !out_hidden || !status)
        return fail(GUFFIN_E_ARG, "forward_tree_rows: null pointer");
    if (rows == 0 || rows > 2) return fail(GUFFIN_E_SHAPE, "forward_tree_rows: a pass has 1 or 2 rows");
    if (slot_count == 0 || slot_count > kMaxTreeSlots || first_slot + rows > slot_count)
        return fail(GUFFIN_E_SHAPE, "forward_tree_rows: at most 8 private rows, the pass's slots among them");
    const guffin_model_desc& m = *model;
    if (m.global_period > 1 && m.sliding_window <= slot_count)
        return fail(GUFFIN_E_SHAPE, "forward_tree_rows: the sliding window must exceed the tree's depth");
    if (reinterpret_cast<uintptr_t>(scratch) & 255u) return fail(GUFFIN_E_ALIGN, "forward_tree_rows: scratch must be 256-byte aligned");
    // host staging: positions, per-layer schedules, the concatenated ancestor lists
    uint32_t positions[2] = {0, 0}, offsets[2] = {0, 0}, total = 0, deepest = 0;
    for (uint32_t r = 0; r < rows; ++r) {
        if (depths[r] >= slot_count) return fail(GUFFIN_E_ARG, "forward_tree_rows: a row lies deeper than the tree has rows");
        const uint32_t n = ancestor_counts[r];
        if (n == 0 || n > slot_count) return fail(GUFFIN_E_ARG, "forward_tree_rows: an ancestor list holds the row itself and at most every slot");
        for (uint32_t i = 0; i < n; ++i)
            if (ancestor_lists[total + i] >= slot_count) return fail(GUFFIN_E_ARG, "forward_tree_rows: ancestor outside the private rows");
        if (ancestor_lists[total + n - 1] != first_slot + r) return fail(GUFFIN_E_ARG, "forward_tree_rows: a row's list ends with its own slot");
        if (n != depths[r] + 1) return fail(GUFFIN_E_ARG, "forward_tree_rows: a row at depth d has d ancestors and itself");
        positions[r] = base_position + depths[r];
        offsets[r] = total;
        total += n;
        deepest = std::max(deepest, depths[r]);
    }
    GUFFIN_TRY(check_ring_capacity(m, base_position, deepest + 1, "forward_tree_rows: the rows do not fit the KV rings"));
    // the arena of a chain pass at the deepest position covers this pass: its longest token list is the same
    const Scratch s = layout(m, rows, base_position + slot_count, static_cast<uint8_t*>(scratch));
    if (s.bytes > scratch_bytes) return fail(GUFFIN_E_CAPACITY, "forward_tree_rows: scratch arena too small");
    std::vector<uint32_t> schedule(size_t(m.layer_count) * rows * 4);
    for (uint32_t l = 0; l < m.layer_count; ++l)
        for (uint32_t r = 0; r < rows; ++r) {
            const bool local = is_local(m, l);
            const uint32_t p = positions[r];
            const uint32_t window_start = (local && p >= m.sliding_window) ? p + 1 - m.sliding_window : 0;
            const uint32_t base_first = std::min(window_start, base_position);
            uint32_t* e = schedule.data() + (size_t(l) * rows + r) * 4;
            e[0] = base_first; e[1] = base_position - base_first; e[2] = offsets[r]; e[3] = ancestor_counts[r];
        }
    hipStream_t hs = as_stream(stream);
    if (hipMemcpyWithStream(s.positions, positions, rows * 4, hipMemcpyHostToDevice, hs) != hipSuccess
        || hipMemcpyWithStream(s.ancestors, ancestor_lists, total * 4, hipMemcpyHostToDevice, hs) != hipSuccess
        || hipMemcpyWithStream(s.schedule, schedule.data(), schedule.size() * 4, hipMemcpyHostToDevice, hs) != hipSuccess)
        return fail(GUFFIN_E_HIP, "forward_tree_rows: upload failed");
    const uint32_t H = m.hidden, QW = m.q_heads * m.head_dim, KW = m.kv_heads * m.head_dim;
    const float attn_scale = 1.0f / std::sqrt(static_cast<float>(m.head_dim));
    if (m.global_period > 1) GUFFIN_TRY(guffin_hip_rope_table(stream, s.positions, s.rope_local, rows, m.head_dim, m.local_base, 1.0f));
    GUFFIN_TRY(guffin_hip_rope_table(stream, s.positions, s.rope_global, rows, m.head_dim, m.global_base, m.global_scale));
    GUFFIN_TRY(guffin_hip_embed(stream, m.embed_dtype, m.embed_rows, tokens, s.x, rows, H, std::sqrt(static_cast<float>(H)), m.vocab, status));
    GUFFIN_TRY(guffin_hip_rms_norm(stream, s.x, 1, 0, m.layers[0].norm[0], nullptr, s.u, s.us, rows, H, m.eps, status));
    for (uint32_t l = 0; l < m.layer_count; ++l) {
        const guffin_layer_desc& L = m.layers[l];
        const bool local = is_local(m, l);
        const uint32_t ring_mask = (local ? m.ring_local : m.ring_global) - 1;
        uint16_t* layer_k = static_cast<uint16_t*>(priv_k) + size_t(l) * slot_count * KW;
        uint16_t* layer_v = static_cast<uint16_t*>(priv_v) + size_t(l) * slot_count * KW;
        const int dt[3] = {L.dtype[0], L.dtype[1], L.dtype[2]};
        const void* tl[3] = {L.tiles[0], L.tiles[1], L.tiles[2]};
        const uint32_t n[3] = {QW, KW, KW};
        float* parts[3] = {s.part_a, s.part_b, s.part_c};
        GUFFIN_TRY(guffin_hip_gemv_packed_multi(stream, 3, dt, tl, n, parts, s.u, s.us, rows, H));
        const uint32_t sq = qkv_slices(L, H, QW, KW);
        if (sq == 0) return fail(GUFFIN_E_SHAPE, "forward_tree_rows: q, k and v must share the block length");
        // head norms, rotation and fp16 narrowing into the rows' own slots, then attention over ring and slots
        GUFFIN_TRY(guffin_hip_qkv_post(stream, s.part_a, s.part_b, s.part_c, sq, sq, sq, uint64_t(rows) * QW, uint64_t(rows) * KW,
                                       uint64_t(rows) * KW, L.norm[1], L.norm[2], s.positions, s.q, layer_k + size_t(first_slot) * KW,
                                       layer_v + size_t(first_slot) * KW, rows, m.q_heads, m.kv_heads, m.head_dim, m.head_dim,
                                       local ? m.local_base : m.global_base, local ? 1.0f : m.global_scale, m.eps,
                                       local ? s.rope_local : s.rope_global, status));
        const uint32_t ring_tokens = max_tokens_for(m, l, base_position + deepest, 1) - 1;   // the widest ring range of the pass
        GUFFIN_TRY(guffin_hip_attention_decode(stream, s.q, L.ring_k, L.ring_v, layer_k, layer_v, s.schedule + size_t(l) * rows * 4,
                                               s.ancestors, s.a, s.as, s.attn_out, s.attn_ml, rows, slot_count,
                                               std::min(ring_tokens, base_position) + slot_count, ring_mask, m.q_heads, m.kv_heads,
                                               m.head_dim, attn_scale, status));
        GUFFIN_TRY(block_tail(stream, m, l, s, rows, out_hidden, out_hidden_sums, status));
    }
    return GUFFIN_OK;
}

extern "C" int guffin_hip_commit_rows(void* stream, const guffin_model_desc* model, const void* priv_k,
                                      const void* priv_v, void* const* ring_k_table, void* const* ring_v_table,
                                      const uint32_t* accepted, uint32_t position, uint32_t rows) {
    GUFFIN_TRY(validate_model(model));
    if (!priv_k || !priv_v || !ring_k_table || !ring_v_table) return fail(GUFFIN_E_ARG, "commit_rows: null pointer");
    if (rows == 0 || rows > 2) return fail(GUFFIN_E_SHAPE, "commit_rows: rows must be 1 or 2");
    const uint32_t KW = model->kv_heads * model->head_dim;
    launch(commit_rows_kernel, dim3((KW + 255) / 256, model->layer_count, rows), dim3(256), 0,
                       as_stream(stream), static_cast<const uint16_t*>(priv_k), static_cast<const uint16_t*>(priv_v),
                       reinterpret_cast<uint16_t* const*>(ring_k_table), reinterpret_cast<uint16_t* const*>(ring_v_table),
                       accepted, position, rows, KW, model->ring_local - 1, model->ring_global - 1, model->global_period);
    return check_launch("commit_rows");
}

// ---- prefill: a run of rows through every block --------------------------------------------
namespace guffin {
namespace {

struct PrefillScratch {
    float *x, *x1, *u, *q, *kraw, *vraw, *a, *gate, *up, *h, *o;
    float *rope_local, *rope_global;
    uint16_t *run_k, *run_v;
    uint8_t* attn_ws;   // transposed values of the matrix-core attention
    uint8_t* image;
    uint32_t* positions;
    uint64_t bytes;
};

PrefillScratch prefill_layout(const guffin_model_desc& m, uint32_t rows, uint8_t* base) {
    Arena ar {base, 0, 0};
    const uint64_t H = m.hidden, F = m.ffn, QW = uint64_t(m.q_heads) * m.head_dim, KW = uint64_t(m.kv_heads) * m.head_dim;
    PrefillScratch s {};
    s.x = ar.take<float>(rows * H); s.x1 = ar.take<float>(rows * H); s.u = ar.take<float>(rows * H);
    s.o = ar.take<float>(rows * H);
    s.q = ar.take<float>(rows * QW); s.a = ar.take<float>(rows * QW);
    s.kraw = ar.take<float>(rows * KW); s.vraw = ar.take<float>(rows * KW);
    s.gate = ar.take<float>(rows * F); s.up = ar.take<float>(rows * F); s.h = ar.take<float>(rows * F);
    s.rope_local = ar.take<float>(uint64_t(rows) * m.head_dim);
    s.rope_global = ar.take<float>(uint64_t(rows) * m.head_dim);
    s.run_k = ar.take<uint16_t>(rows * KW); s.run_v = ar.take<uint16_t>(rows * KW);
    // V^T of every token a row may see: at most a full global ring plus the run, in whole 32-token tiles
    s.attn_ws = ar.take<uint8_t>(uint64_t(m.kv_heads) * m.head_dim * 2 * ((uint64_t(m.ring_global) + rows + 63) & ~uint64_t{31}));
    const uint32_t widest = std::max({m.hidden, m.ffn, m.q_heads * m.head_dim});
    s.image = ar.take<uint8_t>(guffin_hip_prefill_image_bytes(rows, widest));
    s.positions = ar.take<uint32_t>(rows);
    s.bytes = (ar.used + 255) & ~uint64_t{255};
    return s;
}

__global__ void fill_positions_kernel(uint32_t* positions, uint32_t rows, uint32_t position) {
    const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < rows) positions[i] = position + i;
}

}  // namespace
}  // namespace guffin

extern "C" uint64_t guffin_hip_prefill_scratch_bytes(const guffin_model_desc* model, uint32_t rows) {
    if (!model || rows == 0 || guffin::validate_model(model)) return 0;
    return guffin::prefill_layout(*model, rows, nullptr).bytes;
}

extern "C" int guffin_hip_prefill_rows(void* stream, const guffin_model_desc* model, const uint32_t* tokens,
                                       uint32_t rows, uint32_t position, void* scratch, uint64_t scratch_bytes,
                                       float* out_hidden, uint32_t* status) {
    using namespace guffin;
    if (!tokens || !scratch || !out_hidden || !status) return fail(GUFFIN_E_ARG, "prefill_rows: null pointer");
    GUFFIN_TRY(validate_model(model));
    if (rows == 0) return fail(GUFFIN_E_SHAPE, "prefill_rows: no rows");
    GUFFIN_TRY(check_ring_capacity(*model, position, rows, "prefill_rows: the rows do not fit the KV rings"));
    if (reinterpret_cast<uintptr_t>(scratch) & 255u) return fail(GUFFIN_E_ALIGN, "prefill_rows: scratch must be 256-byte aligned");
    const guffin_model_desc& m = *model;
    const PrefillScratch s = prefill_layout(m, rows, static_cast<uint8_t*>(scratch));
    if (s.bytes > scratch_bytes) return fail(GUFFIN_E_CAPACITY, "prefill_rows: scratch arena too small");
    hipStream_t hs = as_stream(stream);
    const uint32_t H = m.hidden, F = m.ffn, QW = m.q_heads * m.head_dim, KW = m.kv_heads * m.head_dim;
    const float attn_scale = 1.0f / std::sqrt(static_cast<float>(m.head_dim));
    launch(fill_positions_kernel, dim3((rows + 255) / 256), dim3(256), 0, hs, s.positions, rows, position);
    GUFFIN_TRY(check_launch("prefill positions"));
    GUFFIN_TRY(guffin_hip_rope_table(stream, s.positions, s.rope_local, rows, m.head_dim, m.local_base, 1.0f));
    GUFFIN_TRY(guffin_hip_rope_table(stream, s.positions, s.rope_global, rows, m.head_dim, m.global_base, m.global_scale));
    GUFFIN_TRY(guffin_hip_embed(stream, m.embed_dtype, m.embed_rows, tokens, s.x, rows, H,
                                std::sqrt(static_cast<float>(H)), m.vocab, status));
    GUFFIN_TRY(guffin_hip_rms_norm(stream, s.x, 1, 0, m.layers[0].norm[0], nullptr, s.u, nullptr, rows, H, m.eps, status));
    for (uint32_t l = 0; l < m.layer_count; ++l) {
        const guffin_layer_desc& L = m.layers[l];
        const bool local = is_local(m, l);
        const float base = local ? m.local_base : m.global_base, scale = local ? 1.0f : m.global_scale;
        const uint32_t ring_mask = (local ? m.ring_local : m.ring_global) - 1;
        GUFFIN_TRY(guffin_hip_prefill_pack(stream, s.u, s.image, rows, H));
        GUFFIN_TRY(guffin_hip_prefill_gemm(stream, L.dtype[0], L.tiles[0], s.image, s.q, rows, H, QW));
        GUFFIN_TRY(guffin_hip_prefill_gemm(stream, L.dtype[1], L.tiles[1], s.image, s.kraw, rows, H, KW));
        GUFFIN_TRY(guffin_hip_prefill_gemm(stream, L.dtype[2], L.tiles[2], s.image, s.vraw, rows, H, KW));
        GUFFIN_TRY(guffin_hip_qkv_post(stream, s.q, s.kraw, s.vraw, 1, 1, 1, 0, 0, 0, L.norm[1], L.norm[2], s.positions,
                                       s.q, s.run_k, s.run_v, rows, m.q_heads, m.kv_heads, m.head_dim, m.head_dim, base,
                                       scale, m.eps, local ? s.rope_local : s.rope_global, status));
        GUFFIN_TRY(guffin_hip_prefill_attention(stream, s.q, L.ring_k, L.ring_v, s.run_k, s.run_v, s.a, rows, position,
                                                local ? m.sliding_window : 0u, ring_mask, m.q_heads, m.kv_heads,
                                                m.head_dim, attn_scale, s.attn_ws));
        GUFFIN_TRY(guffin_hip_publish_run(stream, s.run_k, s.run_v, L.ring_k, L.ring_v, rows, position, ring_mask, KW));
        GUFFIN_TRY(guffin_hip_prefill_pack(stream, s.a, s.image, rows, QW));
        GUFFIN_TRY(guffin_hip_prefill_gemm(stream, L.dtype[3], L.tiles[3], s.image, s.o, rows, QW, H));
        GUFFIN_TRY(guffin_hip_rms_norm_add_norm(stream, s.o, 1, 0, L.norm[3], s.x, s.x1, L.norm[4], s.u, nullptr, rows, H,
                                                m.eps, status));
        GUFFIN_TRY(guffin_hip_prefill_pack(stream, s.u, s.image, rows, H));
        GUFFIN_TRY(guffin_hip_prefill_gemm(stream, L.dtype[4], L.tiles[4], s.image, s.gate, rows, H, F));
        GUFFIN_TRY(guffin_hip_prefill_gemm(stream, L.dtype[5], L.tiles[5], s.image, s.up, rows, H, F));
        GUFFIN_TRY(guffin_hip_geglu(stream, s.gate, s.up, 1, 0, s.h, nullptr, rows, F));
        GUFFIN_TRY(guffin_hip_prefill_pack(stream, s.h, s.image, rows, F));
        GUFFIN_TRY(guffin_hip_prefill_gemm(stream, L.dtype[6], L.tiles[6], s.image, s.o, rows, F, H));
        const bool last = l + 1 == m.layer_count;
        GUFFIN_TRY(guffin_hip_rms_norm_add_norm(stream, s.o, 1, 0, L.norm[5], s.x1, s.x,
                                                last ? m.out_norm : m.layers[l + 1].norm[0], last ? out_hidden : s.u,
                                                nullptr, rows, H, m.eps, status));
    }
    return GUFFIN_OK;
}

// ---- one H1 cycle ---------------------------------------------------------------------
namespace guffin {
namespace {
// the step's buffers inside the caller's scratch arena; scratch == nullptr only measures
struct StepBuffers {
    uint64_t d_bytes, t_bytes, bytes;
    uint8_t *d_scratch, *t_scratch;
    float *d_hidden, *t_hidden, *q_parts, *q_logits, *p_parts, *p_logits;
    uint8_t *law_ws, *sel_ws, *law, *cands, *any_ws;
    uint32_t* words;
    uint32_t* hist;      // [2][64] sampler history of the two verify rows, then their two counts
    uint64_t* full_cdf;
};
// rows the drafter ingests: the root alone, or the accepted proposal it still owes and the root
uint32_t drafter_rows(const guffin_h1_desc* d) { return d->drafter_rows == 2 ? 2u : 1u; }

StepBuffers carve_step(const guffin_h1_desc* d, void* scratch) {
    const guffin_model_desc& T = *d->target;
    const guffin_model_desc& D = *d->drafter;
    const uint64_t V = T.vocab;
    Arena ar {static_cast<uint8_t*>(scratch), 0, 0};
    StepBuffers b {};
    const uint32_t dr = drafter_rows(d);
    b.d_bytes = guffin_hip_forward_scratch_bytes(&D, dr, d->drafter_position);
    b.t_bytes = guffin_hip_forward_scratch_bytes(&T, 2, d->target_position);
    b.d_scratch = ar.take<uint8_t>(b.d_bytes);
    b.t_scratch = ar.take<uint8_t>(b.t_bytes);
    b.d_hidden = ar.take<float>(hidden_with_receipt(dr, D.hidden));
    b.t_hidden = ar.take<float>(hidden_with_receipt(2, T.hidden));
    b.q_parts = ar.take<float>(uint64_t(slices(D.head_dtype, D.hidden, D.vocab)) * dr * D.vocab);
    b.q_logits = ar.take<float>(uint64_t(dr) * D.vocab);
    b.p_parts = ar.take<float>(uint64_t(slices(T.head_dtype, T.hidden, V)) * 2 * V);
    b.p_logits = ar.take<float>(2 * V);
    b.law_ws = ar.take<uint8_t>(guffin_hip_draft_law_workspace_bytes(D.vocab));
    b.sel_ws = ar.take<uint8_t>(guffin_hip_select_workspace_bytes(2, V, d->top_k + kHistoryWindow));
    b.law = ar.take<uint8_t>(4096 + 2 * 3088);  // the compact law, then the two candidate rows
    b.cands = b.law ? b.law + 4096 : nullptr;
    b.words = ar.take<uint32_t>(16);
    b.hist = ar.take<uint32_t>(kHistWords);  // resolved requests, lists, counts, then the history in the drafter's ids
    if (d->full_law) {
        b.any_ws = ar.take<uint8_t>(guffin_hip_draft_law_any_workspace_bytes(D.vocab));
        b.full_cdf = ar.take<uint64_t>(uint64_t(D.vocab) + 1);
    }
    b.bytes = (ar.used + 255) & ~uint64_t{255};
    return b;
}

}  // namespace
}  // namespace guffin
using namespace guffin;

extern "C" uint64_t guffin_hip_h1_scratch_bytes(const guffin_h1_desc* d) {
    if (!d || validate_model(d->target) || validate_model(d->drafter)) return 0;
    return carve_step(d, nullptr).bytes;
}

extern "C" int guffin_hip_h1_step(void* stream, const guffin_h1_desc* d, const uint32_t* root_token, void* scratch,
                                  uint64_t scratch_bytes, void* drafter_priv_k, void* drafter_priv_v,
                                  void* target_priv_k, void* target_priv_v, void* result, uint32_t* status) {
    if (!d || !root_token || !scratch || !result || !status) return fail(GUFFIN_E_ARG, "h1_step: null pointer");
    GUFFIN_TRY(validate_model(d->target));
    GUFFIN_TRY(validate_model(d->drafter));
    if (!d->target->head_tiles || !d->drafter->head_tiles) return fail(GUFFIN_E_ARG, "h1_step: models need packed head weights");
    if (d->drafter->vocab != d->target->vocab && !(d->draft_to_target && d->target_to_draft))
        return fail(GUFFIN_E_SHAPE, "h1_step: drafter and target vocabularies must coincide unless a vocabulary map is given");
    GUFFIN_TRY(check_ring_capacity(*d->target, d->target_position, 2, "h1_step: the verify rows do not fit the target's KV rings"));
    GUFFIN_TRY(check_ring_capacity(*d->drafter, d->drafter_position, d->drafter_rows == 2 ? 2u : 1u,
                                   "h1_step: the drafter's rows do not fit its KV rings"));
    if (reinterpret_cast<uintptr_t>(scratch) & 255u) return fail(GUFFIN_E_ALIGN, "h1_step: scratch must be 256-byte aligned");
    const guffin_model_desc& T = *d->target;
    const guffin_model_desc& D = *d->drafter;
    const uint64_t V = T.vocab;
    const StepBuffers B = carve_step(d, scratch);
    if (B.bytes > scratch_bytes) return fail(GUFFIN_E_CAPACITY, "h1_step: scratch arena too small");
    const uint64_t d_bytes = B.d_bytes, t_bytes = B.t_bytes;
    uint8_t *d_scratch = B.d_scratch, *t_scratch = B.t_scratch, *law_ws = B.law_ws, *sel_ws = B.sel_ws, *any_ws = B.any_ws;
    float *d_hidden = B.d_hidden, *t_hidden = B.t_hidden, *q_parts = B.q_parts, *q_logits = B.q_logits;
    float *p_parts = B.p_parts, *p_logits = B.p_logits;
    uint64_t* full_cdf = B.full_cdf;
    void* law = B.law;
    void* cands = B.cands;
    uint32_t* tokens = B.words;          // [root, proposal]
    uint32_t* sel_status = B.words + 4;  // per-row selection status
    hipStream_t s = as_stream(stream);

    const bool with_history = d->history != nullptr && d->history_count > 0;
    if (d->history_count > kHistoryWindow) return fail(GUFFIN_E_CAPACITY, "h1_step: at most 64 history tokens");
    if (with_history && !(d->repetition_penalty > 0.f)) return fail(GUFFIN_E_ARG, "h1_step: the repetition penalty must be positive");
    struct { float temperature; uint32_t top_k; float top_p, min_p, repetition_penalty; } opt
        = {d->temperature, d->top_k, d->top_p, d->min_p, with_history ? d->repetition_penalty : 1.0f};

    // 1. drafter: ingest (the pending proposal and) the root, project, build the proposal law, pick x
    const uint32_t dr = drafter_rows(d);
    if (dr == 2 && !d->pending_token) return fail(GUFFIN_E_ARG, "h1_step: two drafter rows need the pending token");
    const bool mapped = d->draft_to_target != nullptr;
    if (mapped != (d->target_to_draft != nullptr)) return fail(GUFFIN_E_ARG, "h1_step: the vocabulary map needs its inverse");
    launch(set_step_tokens_kernel, dim3(1), dim3(1), 0, s, root_token, dr == 2 ? d->pending_token : nullptr, tokens,
                       d->target_to_draft, T.vocab, status);
    GUFFIN_TRY(check_launch("set_step_tokens"));
    GUFFIN_TRY(guffin_hip_forward_rows(stream, &D, tokens + 8, dr, d->drafter_position, d_scratch, d_bytes, drafter_priv_k,
                                       drafter_priv_v, d_hidden, d_hidden + hidden_receipt_offset(dr, D.hidden), status));
    GUFFIN_TRY(guffin_hip_gemv_packed(stream, D.head_dtype, D.head_tiles, d_hidden, d_hidden + hidden_receipt_offset(dr, D.hidden), q_parts,
                                      q_logits, dr, D.hidden, D.vocab));
    q_logits += uint64_t(dr - 1) * D.vocab;  // the law comes from the last ingested row (the root)
    if (mapped) {
        // gd_process -> compact law -> proposal, through the map: tokens[2] keeps the proposal in the
        // drafter's ids, tokens[1] carries it to the verify pass in the target's
        const uint32_t* draft_hist = nullptr;
        if (with_history) {
            launch(draft_history_kernel, dim3(1), dim3(64), 0, s, d->history, d->history_count, d->target_to_draft,
                               T.vocab, B.hist + kHistDraft);
            GUFFIN_TRY(check_launch("draft_history"));
            draft_hist = B.hist + kHistDraft;
        }
        if (d->full_law)
            GUFFIN_TRY(guffin_hip_draft_law_any_mapped(stream, q_logits, D.vocab, d->draft_to_target, draft_hist,
                                                       with_history ? d->history_count : 0u, &opt, d->seed, d->step, nullptr, any_ws,
                                                       q_parts, law, full_cdf, tokens + 2, tokens + 1, status));
        else
            GUFFIN_TRY(guffin_hip_draft_law_mapped(stream, q_logits, D.vocab, d->draft_to_target, draft_hist,
                                                   with_history ? d->history_count : 0u, &opt, d->seed, d->step, nullptr, law_ws,
                                                   q_parts, law, tokens + 2, tokens + 1, status));
    } else if (with_history && d->repetition_penalty != 1.0f) {
        // the proposal law sees the same history as the verify pass's first row (the head's partial
        // planes are summed by now: their buffer takes the penalised scores)
        GUFFIN_TRY(guffin_hip_draft_process(stream, q_logits, D.vocab, d->history, d->history_count, d->repetition_penalty, q_parts));
        q_logits = q_parts;
    }
    if (mapped) {
        // built above
    } else if (d->full_law) {
        GUFFIN_TRY(guffin_hip_draft_law_any(stream, q_logits, D.vocab, &opt, d->seed, d->step, nullptr, any_ws, law,
                                            full_cdf, tokens + 1, status));
    } else {
        GUFFIN_TRY(guffin_hip_draft_law(stream, q_logits, D.vocab, &opt, d->seed, d->step, nullptr, law_ws, law,
                                        tokens + 1, status));
    }
    // 2. target: rows [root, x] together, head, candidates of both rows
    GUFFIN_TRY(guffin_hip_forward_rows(stream, &T, tokens, 2, d->target_position, t_scratch, t_bytes, target_priv_k,
                                       target_priv_v, t_hidden, t_hidden + hidden_receipt_offset(2, T.hidden), status));
    GUFFIN_TRY(guffin_hip_gemv_packed(stream, T.head_dtype, T.head_tiles, t_hidden, t_hidden + hidden_receipt_offset(2, T.hidden), p_parts,
                                      p_logits, 2, T.hidden, V));
    // candidates: the top_k best plus one per history token (a penalised token can fall out of the
    // top_k, src/engine/sampling.cpp:430-446), then the history tokens' own logits
    const uint32_t* hist = nullptr;
    if (with_history) {
        launch(build_history_kernel, dim3(1), dim3(128), 0, s, d->history, d->history_count, tokens + 1, V,
                           d->top_k, B.hist, status);
        GUFFIN_TRY(check_launch("build_history"));
        hist = B.hist + kHistLists;
        // capacity of the launch; each row retains top_k + its own deduplicated count
        const uint32_t capacity = std::min<uint64_t>(V, uint64_t(d->top_k) + std::min(d->history_count + 1, kHistoryWindow));
        GUFFIN_TRY(guffin_hip_select_candidates_resolved(stream, p_logits, 2, V, capacity, B.hist, sel_ws, cands, sel_status));
    } else {
        GUFFIN_TRY(guffin_hip_select_candidates(stream, p_logits, 2, V, d->top_k, nullptr, nullptr, sel_ws, cands, sel_status));
    }
    // 3. accept x or draw from the residual; on acceptance draw the next root from row 1
    GUFFIN_TRY(guffin_hip_spec_accept_mapped(stream, cands, law, full_cdf, D.vocab, d->target_to_draft, hist,
                                             hist ? B.hist + kHistCounts : nullptr, tokens + 1, &opt, d->seed, d->step,
                                             nullptr, result, status));
    // 4. publish: the target keeps row 0, and row 1 if x was accepted; the drafter keeps the root
    if (d->target_ring_k && d->target_ring_v) {
        GUFFIN_TRY(guffin_hip_commit_rows(stream, &T, target_priv_k, target_priv_v, d->target_ring_k, d->target_ring_v,
                                          static_cast<const uint32_t*>(result), d->target_position, 2));
    }
    if (d->drafter_ring_k && d->drafter_ring_v) {
        GUFFIN_TRY(guffin_hip_commit_rows(stream, &D, drafter_priv_k, drafter_priv_v, d->drafter_ring_k,
                                          d->drafter_ring_v, nullptr, d->drafter_position, dr));
    }
    return GUFFIN_OK;
}

// debug / test access to the intermediate buffers of the last step laid out in `scratch`
extern "C" int guffin_hip_h1_buffers(const guffin_h1_desc* d, void* scratch, float** drafter_hidden,
                                     float** target_hidden, float** q_logits, float** p_logits, void** law,
                                     void** candidates, uint32_t** tokens) {
    if (!d || !scratch) return fail(GUFFIN_E_ARG, "h1_buffers: null pointer");
    GUFFIN_TRY(validate_model(d->target));
    GUFFIN_TRY(validate_model(d->drafter));
    const StepBuffers B = carve_step(d, scratch);
    if (drafter_hidden) *drafter_hidden = B.d_hidden;
    if (target_hidden) *target_hidden = B.t_hidden;
    if (q_logits) *q_logits = B.q_logits + uint64_t(drafter_rows(d) - 1) * d->drafter->vocab;
    if (p_logits) *p_logits = B.p_logits;
    if (law) *law = B.law;
    if (candidates) *candidates = B.cands;
    if (tokens) *tokens = B.words;
    return GUFFIN_OK;
}

extern "C" int guffin_hip_h1_full_cdf(const guffin_h1_desc* d, void* scratch, uint64_t** full_cdf) {
    if (!d || !scratch || !full_cdf) return fail(GUFFIN_E_ARG, "h1_full_cdf: null pointer");
    GUFFIN_TRY(validate_model(d->target));
    GUFFIN_TRY(validate_model(d->drafter));
    *full_cdf = carve_step(d, scratch).full_cdf;
    return GUFFIN_OK;
}

// ---- consecutive cycles ---------------------------------------------------------------------
// Host-side lifecycle around guffin_hip_h1_step: positions, the drafter's pending token and the
// transaction state of the verify pass.  States follow VerifierTransactionState
// (include/local_gguf_engine/engine/gemma2_metal_plan.hpp:208-215); the pending token follows
// Gemma3DraftPlan (include/local_gguf_engine/engine/gemma3_draft.hpp:61-63,
// src/engine/gemma3_draft.mm:1430-1486): the drafter's last emission is materialised together with
// the next root, and only if the target accepted it.
namespace guffin {
namespace {
struct StepResultHead { uint32_t accepted, token, next_root, status; };

int session_ready(const guffin_h1_session* s, const char* what) {
    if (!s || !s->scratch || !s->drafter_priv_k || !s->drafter_priv_v || !s->target_priv_k || !s->target_priv_v
        || !s->tokens || !s->result || !s->status)
        return fail(GUFFIN_E_ARG, what);
    return GUFFIN_OK;
}
}  // namespace
}  // namespace guffin

extern "C" uint64_t guffin_hip_session_scratch_bytes(const guffin_h1_session* s, uint32_t last_target_position,
                                                     uint32_t last_drafter_position) {
    if (!s) return 0;
    guffin_h1_desc d = s->desc;  // the largest arena any cycle up to the given positions needs
    d.target_position = last_target_position;
    d.drafter_position = last_drafter_position;
    d.drafter_rows = 2;
    return guffin_hip_h1_scratch_bytes(&d);
}

extern "C" int guffin_hip_session_start(guffin_h1_session* s, uint32_t root_token, uint32_t target_position,
                                        uint32_t drafter_position) {
    GUFFIN_TRY(session_ready(s, "session_start: null pointer"));
    if (!s->desc.target_ring_k || !s->desc.target_ring_v || !s->desc.drafter_ring_k || !s->desc.drafter_ring_v)
        return fail(GUFFIN_E_ARG, "session_start: a session publishes its rows: ring tables are required");
    s->desc.target_position = target_position;
    s->desc.drafter_position = drafter_position;
    s->desc.step = 0;
    s->root = root_token; s->pending = 0; s->has_pending = 0;
    s->cycles = 0; s->accepted = 0;
    s->state = GUFFIN_TXN_IDLE;
    return GUFFIN_OK;
}

extern "C" int guffin_hip_session_submit(void* stream, guffin_h1_session* s) {
    GUFFIN_TRY(session_ready(s, "session_submit: null pointer"));
    if (s->state == GUFFIN_TXN_POISONED) return fail(GUFFIN_E_STATE, "session_submit: the session is poisoned");
    if (s->state != GUFFIN_TXN_IDLE) return fail(GUFFIN_E_STATE, "session_submit: a cycle is already in flight");
    hipStream_t hs = as_stream(stream);
    // sources that outlive the call: root and pending are adjacent fields of the session
    static const uint32_t kZero = 0;
    static_assert(offsetof(guffin_h1_session, pending) == offsetof(guffin_h1_session, root) + sizeof(uint32_t),
                  "root and pending are uploaded as one pair");
    if (hipMemcpyAsync(s->tokens, &s->root, 2 * sizeof(uint32_t), hipMemcpyHostToDevice, hs) != hipSuccess
        || hipMemcpyAsync(s->status, &kZero, sizeof(kZero), hipMemcpyHostToDevice, hs) != hipSuccess)
        return fail(GUFFIN_E_HIP, "session_submit: upload failed");
    s->desc.drafter_rows = s->has_pending ? 2u : 1u;
    s->desc.pending_token = s->tokens + 1;
    if (int rc = guffin_hip_h1_step(stream, &s->desc, s->tokens, s->scratch, s->scratch_bytes, s->drafter_priv_k,
                                    s->drafter_priv_v, s->target_priv_k, s->target_priv_v, s->result, s->status))
        return rc;  // nothing was enqueued that changes the caches: still idle
    s->state = GUFFIN_TXN_SUBMITTED;
    return GUFFIN_OK;
}

extern "C" int guffin_hip_session_complete(void* stream, guffin_h1_session* s, uint32_t* emitted, uint32_t* emitted_count) {
    GUFFIN_TRY(session_ready(s, "session_complete: null pointer"));
    if (!emitted || !emitted_count) return fail(GUFFIN_E_ARG, "session_complete: null pointer");
    if (s->state != GUFFIN_TXN_SUBMITTED) return fail(GUFFIN_E_STATE, "session_complete: no cycle in flight");
    StepResultHead r {};
    uint32_t status = 0;
    if (hipStreamSynchronize(as_stream(stream)) != hipSuccess
        || hipMemcpy(&r, s->result, sizeof(r), hipMemcpyDeviceToHost) != hipSuccess
        || hipMemcpy(&status, s->status, sizeof(status), hipMemcpyDeviceToHost) != hipSuccess) {
        s->state = GUFFIN_TXN_POISONED;
        return fail(GUFFIN_E_HIP, "session_complete: read-back failed");
    }
    *emitted_count = 0;
    resident_note_status(status);   // a wait that gave up: later cycles of this process run one launch per operator
    if (status != 0 || r.status != 0) {
        // a numerical fault or a refused law: the rows of this cycle may already be in the caches
        s->state = GUFFIN_TXN_POISONED;
        return fail(GUFFIN_E_STATE, "session_complete: device status raised, the session is poisoned");
    }
    // row 0 (the root) is published; row 1 (the proposal) too if it was accepted
    const uint32_t proposal = r.accepted ? r.token : 0;
    s->desc.target_position += 1 + (r.accepted ? 1u : 0u);
    s->desc.drafter_position += s->desc.drafter_rows == 2 ? 2u : 1u;
    s->desc.step += 1;
    s->cycles += 1;
    s->accepted += r.accepted ? 1u : 0u;
    if (r.accepted) { emitted[0] = proposal; emitted[1] = r.next_root; *emitted_count = 2; }
    else { emitted[0] = r.token; *emitted_count = 1; }
    s->has_pending = r.accepted ? 1u : 0u;   // the drafter has not seen the accepted proposal yet
    s->pending = proposal;
    s->root = r.next_root;
    s->state = GUFFIN_TXN_IDLE;
    return GUFFIN_OK;
}
