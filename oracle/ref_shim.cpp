// C-ABI wrapper around the REFERENCE's own CPU sources (test infrastructure only).
//
// oracle/Makefile compiles the reference translation units where they lie under the
// reference checkout and links them with this file into oracle/_ref/libguffin_ref.so.
// Nothing from the reference is copied into this repository: this file only calls the
// reference's public functions through their headers.  It is used to validate the
// restatement in gfo_*.cpp and, when present, as the "reference" CPU baseline.
//
// Not wrapped, and why: backends::cpu::matmul_f32_quantized_gguf_weight
// (src/tensor/backends/cpu_backend.cpp:301-323) links only together with
// backend_buffer.mm (Objective-C++, Metal); its arithmetic is reached instead through
// dot_q4_k_row_f32 / dot_q6_k_row_f32 (src/tensor/quantization.cpp:706-713, 826-833),
// which dequantise one column and take the same ascending fp32 inner product from 0.0f.
#include "local_gguf_engine/engine/sampling.hpp"
#include "local_gguf_engine/tensor/f16.hpp"
#include "local_gguf_engine/tensor/ops/attention.hpp"
#include "local_gguf_engine/tensor/ops/elementwise.hpp"
#include "local_gguf_engine/tensor/ops/normalization.hpp"
#include "local_gguf_engine/tensor/ops/reduction.hpp"
#include "local_gguf_engine/tensor/ops/rope.hpp"
#include "local_gguf_engine/tensor/ops/softmax.hpp"
#include "local_gguf_engine/tensor/quantization.hpp"
#include "local_gguf_engine/tensor/tensor.hpp"

#include "gfo.h"

#include <cstring>
#include <span>
#include <vector>

namespace t = local_gguf_engine::tensor;
namespace e = local_gguf_engine::engine;

namespace {

t::DType to_dtype(int dtype) {
    return dtype == GFO_Q8_0 ? t::DType::q8_0 : dtype == GFO_Q4_K ? t::DType::q4_k : t::DType::q6_k;
}

t::TensorStorage f32_matrix(const float* data, uint64_t rows, uint64_t cols) {
    const auto d = t::TensorDescriptor::from(t::Shape::from({rows, cols}), t::DType::f32);
    return t::TensorStorage::from_bytes(
        d, std::span<const uint8_t>(reinterpret_cast<const uint8_t*>(data), d.byte_count));
}

t::TensorStorage f32_vector(const float* data, uint64_t n) {
    const auto d = t::TensorDescriptor::from(t::Shape::from({n}), t::DType::f32);
    return t::TensorStorage::from_bytes(
        d, std::span<const uint8_t>(reinterpret_cast<const uint8_t*>(data), d.byte_count));
}

void copy_out(const t::TensorStorage& s, float* out) {
    std::memcpy(out, s.bytes().data(), s.bytes().size());
}

// rows of `cols` quantised weights, each row contiguous: the row helpers' convention
t::TensorStorage quant_rows(int dtype, const uint8_t* bytes, uint64_t rows, uint64_t cols) {
    const auto d = t::TensorDescriptor::from(t::Shape::from({rows, cols}), to_dtype(dtype));
    return t::TensorStorage::from_bytes(d, std::span<const uint8_t>(bytes, d.byte_count));
}

e::TokenSamplerOptions to_options(const gfo_sampler_options& o) {
    e::TokenSamplerOptions r;
    r.temperature = o.temperature;
    r.top_k = o.top_k;
    r.top_p = o.top_p;
    r.min_p = o.min_p;
    r.repetition_penalty = o.repetition_penalty;
    r.seed = 1;
    r.repetition_window = 64;
    return r;
}

void to_plain(const e::PreparedTokenDistribution& p, gfo_prepared* out) {
    std::memset(out, 0, sizeof(*out));
    out->count = p.count;
    out->total_sampling_weight = p.total_sampling_weight;
    for (uint32_t i = 0; i < p.count; ++i) {
        out->token[i] = p.values[i].token;
        out->probability[i] = p.values[i].probability;
        out->sampling_weight[i] = p.values[i].sampling_weight;
    }
}

e::PreparedTokenDistribution prepare(const gfo_token_logit* cands, uint32_t n,
                                     const gfo_sampler_options& opt, const uint32_t* history,
                                     uint32_t history_count) {
    const auto options = to_options(opt);
    e::TokenSelectionRequest request;
    request.top_k = options.temperature == 0.0F ? 1U : static_cast<uint32_t>(options.top_k);
    request.history_token_count = history_count;
    for (uint32_t i = 0; i < history_count; ++i) request.history_token_ids[i] = history[i];
    request.base_candidate_count = request.top_k + history_count;
    std::vector<e::TokenLogit> values(n);
    for (uint32_t i = 0; i < n; ++i) values[i] = {cands[i].token, cands[i].logit};
    return e::prepare_token_distribution(values, options, request);
}

}  // namespace

extern "C" {

float gfr_f16_to_f32(uint16_t bits) { return t::f16_bits_to_f32(bits); }

int gfr_dequant(int dtype, const uint8_t* blocks, uint64_t n_blocks, float* out) try {
    const uint64_t be = dtype == GFO_Q8_0 ? 32 : 256;
    const auto s = quant_rows(dtype, blocks, 1, n_blocks * be);
    for (uint64_t b = 0; b < n_blocks; ++b)
        for (uint64_t i = 0; i < be; ++i) {
            float v;
            if (dtype == GFO_Q8_0) v = t::q8_0_block_view(s, b).dequantized_value(i);
            else if (dtype == GFO_Q4_K) v = t::q4_k_block_view(s, b).dequantized_value(i);
            else v = t::q6_k_block_view(s, b).dequantized_value(i);
            out[b * be + i] = v;
        }
    return 0;
} catch (...) { return -1; }

// y[r, n] = dot(row n of W, x[r]) through the reference's own row dot (Q4_K, Q6_K);
// Q8_0 has no row helper, so its blocks are decoded by the reference and summed here
// in the CPU backend's order.
int gfr_gemv(int dtype, const uint8_t* w, const float* x, float* y, uint32_t rows, uint32_t K,
             uint32_t N) try {
    const auto s = quant_rows(dtype, w, N, K);
    for (uint32_t r = 0; r < rows; ++r) {
        const std::span<const float> xr(x + size_t(r) * K, K);
        for (uint32_t n = 0; n < N; ++n) {
            float v;
            if (dtype == GFO_Q4_K) v = t::dot_q4_k_row_f32(s, n, xr);
            else if (dtype == GFO_Q6_K) v = t::dot_q6_k_row_f32(s, n, xr);
            else {
                v = 0.0F;
                for (uint32_t k = 0; k < K; ++k)
                    v += xr[k] * t::q8_0_block_view(s, uint64_t(n) * (K / 32) + k / 32).dequantized_value(k % 32);
            }
            y[size_t(r) * N + n] = v;
        }
    }
    return 0;
} catch (...) { return -1; }

int gfr_rms_norm(const float* x, const float* gamma, float* y, uint32_t rows, uint32_t width,
                 float eps) try {
    copy_out(t::ops::rms_norm_f32(f32_matrix(x, rows, width), f32_vector(gamma, width), eps), y);
    return 0;
} catch (...) { return -1; }

int gfr_rope_neox(const float* in, float* out, uint64_t position_start, uint32_t rows,
                  uint32_t heads, uint32_t head_dim, uint32_t rope_dim, float base) try {
    copy_out(t::ops::rope_neox_f32_by_heads_with_position_start(
                 f32_matrix(in, rows, uint64_t(heads) * head_dim), position_start, heads, head_dim,
                 rope_dim, base), out);
    return 0;
} catch (...) { return -1; }

int gfr_gelu_mul(const float* gate, const float* up, float* out, uint64_t n) try {
    const auto g = t::ops::gelu_tanh_f32(f32_vector(gate, n));
    copy_out(t::ops::multiply_f32(g, f32_vector(up, n)), out);
    return 0;
} catch (...) { return -1; }

// scores -> softmax -> values exactly as the CPU operators compose them.  Keys and values
// are fp32 rows for positions 0..key_rows-1; `window` is attention_token_count.
int gfr_attention(const float* q, const float* k, const float* v, float* out,
                  uint64_t query_position_start, uint32_t rows, uint32_t key_rows, uint32_t heads,
                  uint32_t kv_heads, uint32_t head_dim, uint32_t window, float scale,
                  float softcap) try {
    const auto query = f32_matrix(q, rows, uint64_t(heads) * head_dim);
    const auto key = f32_matrix(k, key_rows, uint64_t(kv_heads) * head_dim);
    const auto value = f32_matrix(v, key_rows, uint64_t(kv_heads) * head_dim);
    const auto scores = t::ops::causal_grouped_attention_scores_f32(
        query, key, query_position_start, heads, kv_heads, head_dim, window, scale, softcap);
    const auto probabilities = t::ops::softmax_f32(scores);
    copy_out(t::ops::causal_grouped_attention_values_f32(
                 probabilities, value, query_position_start, heads, kv_heads, head_dim, window), out);
    return 0;
} catch (...) { return -1; }

uint32_t gfr_argmax(const float* logits, uint32_t vocab) {
    return t::ops::top_logit_f32(f32_vector(logits, vocab)).token;
}

int gfr_prepare_token_distribution(const gfo_token_logit* cands, uint32_t n,
                                   const gfo_sampler_options* opt, const uint32_t* history,
                                   uint32_t history_count, gfo_prepared* out) try {
    to_plain(prepare(cands, n, *opt, history, history_count), out);
    return 0;
} catch (...) { return -1; }

uint32_t gfr_select_draft_token(const uint32_t* tokens, const uint64_t* masses, uint32_t count,
                                uint32_t word, int* status) try {
    e::DraftTokenDistribution d;
    d.count = count;
    for (uint32_t i = 0; i < count; ++i) d.values[i] = {tokens[i], masses[i]};
    *status = 0;
    return e::select_draft_token(d, word);
} catch (...) { *status = -1; return 0; }

// Gathered-law acceptance exactly as TokenSamplerFork::sample_speculative composes it
// (sampling.cpp:896-934), with the draws injected.  q is given as the compact law.
int gfr_spec_accept(const gfo_token_logit* row0, uint32_t n0, const gfo_token_logit* row1,
                    uint32_t n1, const gfo_draft_law* law, uint32_t proposal,
                    const gfo_sampler_options* opt, double u_accept, double u_residual,
                    double u_next, gfo_spec_result* out) try {
    std::memset(out, 0, sizeof(*out));
    const auto target = prepare(row0, n0, *opt, nullptr, 0);
    e::DraftProbabilityLeaseOwner owner;
    owner.begin_epoch();
    e::GatheredDraftTokenDistribution gathered;
    gathered.lease = owner.lease(0);
    gathered.count = target.count;
    auto mass = [&](uint32_t token, uint64_t* begin) -> uint64_t {
        for (uint32_t i = 0; i < law->count; ++i)
            if (law->ids[i] == token) { if (begin) *begin = law->cdf[i]; return law->cdf[i + 1] - law->cdf[i]; }
        if (begin) *begin = 0;
        return 0;
    };
    uint64_t begin = 0;
    gathered.proposal = {proposal, mass(proposal, &begin)};
    gathered.proposal_cdf_begin = begin;
    for (uint32_t i = 0; i < target.count; ++i)
        gathered.target_values[i] = {target.values[i].token, mass(target.values[i].token, nullptr)};
    const auto distribution = e::prepare_speculative_distribution(proposal, gathered, target);
    out->acceptance_probability = distribution.acceptance_probability;
    out->residual_total = distribution.residual.total_sampling_weight;
    out->residual_count = distribution.residual.count;
    const auto selected = e::sample_speculative_token(proposal, distribution, u_accept, u_residual);
    out->accepted = selected.accepted ? 1 : 0;
    out->token = selected.token;
    out->next_root = selected.token;
    if (selected.accepted) {
        // next root: an ordinary draw from row 1's prepared law.  select_prepared_token is
        // internal, so reach it through the residual branch of sample_speculative_token.
        e::PreparedSpeculativeDistribution next;
        next.proposal_token = proposal;
        next.acceptance_probability = 0.0;
        next.residual = prepare(row1, n1, *opt, nullptr, 0);
        out->next_root = e::sample_speculative_token(proposal, next, 0.0, u_next).token;
    }
    return 0;
} catch (...) { return -1; }

// make_token_selection_request(options, DeviceSelectionRequest) (sampling.cpp:380-392): the host
// definition the device request resolver must reproduce.  Returns -1 where the reference throws.
int gfr_selection_request(const gfo_selection_row* raw, uint32_t top_k, int repetition_enabled,
                          gfo_resolved_row* out) try {
    std::memset(out, 0, sizeof(*out));
    e::TokenSamplerOptions options;
    options.temperature = 0.8F;
    options.top_k = top_k;
    options.top_p = 1.0F;
    options.min_p = 0.0F;
    options.repetition_penalty = repetition_enabled ? 1.1F : 1.0F;
    options.seed = 1;
    options.repetition_window = raw->history_window_limit;
    e::DeviceSelectionRequest request;
    for (uint32_t i = 0; i < 64; ++i) request.history.token_ids[i] = raw->history_token_ids[i];
    request.history.head = raw->history_head;
    request.history.length = raw->history_length;
    request.history.window_limit = raw->history_window_limit;
    for (uint32_t i = 0; i < 23; ++i) request.suffix_token_ids[i] = raw->suffix_token_ids[i];
    request.suffix_count = raw->suffix_count;
    const auto resolved = e::make_token_selection_request(options, request);
    out->top_k = resolved.top_k;
    out->base_candidate_count = resolved.base_candidate_count;
    out->history_count = resolved.history_token_count;
    for (uint32_t i = 0; i < resolved.history_token_count; ++i) out->history_token_ids[i] = resolved.history_token_ids[i];
    return 0;
} catch (...) { return -1; }

}  // extern "C"
