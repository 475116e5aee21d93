// CPU oracle (test infrastructure only, see gfo.h): the sampling laws of one H1 cycle.
//
// Follows:
//   src/engine/sampling.cpp:25-30     candidate order (logit desc, token asc)
//   src/engine/sampling.cpp:394-499   prepare_token_distribution: dedup -> repetition ->
//                                     sort -> top-k -> top-p on T=1 weights -> min-p ->
//                                     temperature re-weight -> normalise (all double)
//   src/engine/sampling.cpp:117-158   validate_prepared_distribution: Neumaier total
//   src/engine/sampling.cpp:561-630   gathered speculative law: a=min(1,p/q), residual
//                                     max(p-q,0) on p's support in p's order, q not renormalised
//   src/engine/sampling.cpp:632-656   accept iff u_a < a, else inverse-CDF on the residual
//   src/engine/sampling.cpp:247-257   select_prepared_token: first i with draw < cumsum
//   src/engine/sampling.cpp:501-514   select_draft_token: first bin with word < cdf_end
//   src/engine/sampling.cpp:896-934   draw order: acceptance draw, residual draw only on reject
//   src/engine/gemma3_draft.mm:191-294  compact proposal law (score = logit/T, support = all
//                                     scores >= k-th best, descending sort, tail top-p / min-p,
//                                     id sort, f32 prefix / total * 2^32 -> u64 bins)
//   src/engine/gemma3_draft.mm:296-379  full-vocabulary law (256-token tiles, f32 prefix)
//   src/engine/gemma3_draft.mm:1528-1581 gather: q mass of each target-support token
//   src/engine/chain_chat.mm:524-533  after a full accept, row 1's candidates seed the next root
//
// The reference draws from std::mt19937_64; this build feeds both sides from
// Philox4x32-10 keyed (seed, step) while keeping the consumption pattern.
#include "gfo.h"

#include <algorithm>
#include <array>
#include <cmath>
#include <cstring>
#include <limits>
#include <vector>

namespace {

constexpr uint32_t kMaxTopK = 256, kMaxCandidates = 384, kMaxHistory = 64;
constexpr uint64_t kMassTotal = uint64_t{1} << 32;

inline bool better(const gfo_token_logit& a, const gfo_token_logit& b) {
    if (a.logit != b.logit) return a.logit > b.logit;
    return a.token < b.token;
}

bool options_valid(const gfo_sampler_options& o) {
    if (!std::isfinite(o.temperature) || o.temperature < 0.0f) return false;
    if (o.top_k == 0 || o.top_k > kMaxTopK) return false;
    if (!std::isfinite(o.top_p) || o.top_p <= 0.0f || o.top_p > 1.0f) return false;
    if (!std::isfinite(o.min_p) || o.min_p < 0.0f || o.min_p > 1.0f) return false;
    if (!std::isfinite(o.repetition_penalty) || o.repetition_penalty <= 0.0f) return false;
    return true;
}

// Returns the compensated total, or a negative value when the reference would throw.
double validated_total(const gfo_prepared& p) {
    if (p.count == 0 || p.count > kMaxTopK || !std::isfinite(p.total_sampling_weight)
        || p.total_sampling_weight <= 0.0)
        return -1.0;
    double total = 0.0, correction = 0.0;
    for (uint32_t i = 0; i < p.count; ++i) {
        const double prob = p.probability[i], w = p.sampling_weight[i];
        if (!std::isfinite(prob) || prob < 0.0 || prob > 1.0 || !std::isfinite(w) || w < 0.0) return -1.0;
        const double expected = w / p.total_sampling_weight;
        const double tol = 4.0 * std::numeric_limits<double>::epsilon() * std::max(expected, prob);
        if (std::abs(prob - expected) > tol) return -1.0;
        for (uint32_t e = 0; e < i; ++e)
            if (p.token[e] == p.token[i]) return -1.0;
        const double sum = total + w;
        correction += total >= w ? (total - sum) + w : (w - sum) + total;
        total = sum;
    }
    total += correction;
    const double tol = static_cast<double>(p.count) * std::numeric_limits<double>::epsilon() * total;
    if (!std::isfinite(total) || total <= 0.0 || std::abs(total - p.total_sampling_weight) > tol) return -1.0;
    return total;
}

uint32_t select_prepared(const gfo_prepared& p, double draw) {
    double cumulative = 0.0;
    for (uint32_t i = 0; i < p.count; ++i) {
        cumulative += p.sampling_weight[i];
        if (draw < cumulative) return p.token[i];
    }
    return p.token[p.count - 1];
}

// q mass of `token` under a compact law (ids ascending); 0 outside the support.
uint64_t law_mass(const gfo_draft_law& law, uint32_t token, uint64_t* begin) {
    const uint32_t* end = law.ids + law.count;
    const uint32_t* it = std::lower_bound(law.ids, end, token);
    if (it == end || *it != token) { if (begin) *begin = 0; return 0; }
    const size_t i = static_cast<size_t>(it - law.ids);
    if (begin) *begin = law.cdf[i];
    return law.cdf[i + 1] - law.cdf[i];
}

// a law as the gather sees it: compact receipt or full table (gemma3_draft.mm:1538-1556)
// target_to_draft: the inverse of the drafter's vocabulary map (src/engine/gemma3_draft.mm:659-671), -1
// for a target token no draft token maps to; null when both sides share one vocabulary.  The law lives in
// draft ids; masses are looked up by target id (Gemma3DraftPlan::gather, :1570-1578).
struct LawView { const gfo_draft_law* compact; const uint64_t* full; uint32_t vocab; const int32_t* target_to_draft = nullptr; };
uint64_t law_mass(const LawView& law, uint32_t token, uint64_t* begin) {
    if (law.target_to_draft) {
        const int32_t draft = law.target_to_draft[token];
        if (draft < 0) { if (begin) *begin = 0; return 0; }
        token = static_cast<uint32_t>(draft);
    }
    if (law.compact) return law_mass(*law.compact, token, begin);
    if (token >= law.vocab) { if (begin) *begin = 0; return 0; }
    if (begin) *begin = law.full[token];
    return law.full[token + 1] - law.full[token];
}

struct Scored { uint32_t token; float score; };
inline bool better_scored(const Scored& a, const Scored& b) {
    return a.score > b.score || (a.score == b.score && a.token < b.token);
}

}  // namespace

extern "C" {

// exp for the draft law's f32 weights, built only from IEEE-exact float operations
// (multiply, add, fused multiply-add, floor, exponent-field scaling) so that any
// conforming machine reproduces every bit.  Arguments are <= 0 in the law; results
// below 2^-126 flush to zero.  Accuracy ~1 ulp against exp.
float gfo_exp_f32(float x) {
    if (!(x > -86.0f)) return x != x ? x : 0.0f;
    if (x > 88.0f) return std::numeric_limits<float>::infinity();
    const float kf = std::floor(std::fma(x, 1.44269502162933349609375f, 0.5f));
    float r = std::fma(kf, -0.693145751953125f, x);            // ln2 high part (product is exact)
    r = std::fma(kf, -1.428606765330187045037746429443359375e-06f, r);  // ln2 low part
    float p = 1.0f / 5040.0f;                                  // Taylor, |r| <= 0.347: error < 6e-9
    p = std::fma(p, r, 1.0f / 720.0f);
    p = std::fma(p, r, 1.0f / 120.0f);
    p = std::fma(p, r, 1.0f / 24.0f);
    p = std::fma(p, r, 1.0f / 6.0f);
    p = std::fma(p, r, 0.5f);
    p = std::fma(p, r, 1.0f);
    p = std::fma(p, r, 1.0f);
    const int k = static_cast<int>(kf);                        // k in [-124, 127] here
    uint32_t bits = static_cast<uint32_t>(k + 127) << 23;
    float two_k;
    std::memcpy(&two_k, &bits, 4);
    return p * two_k;
}

int gfo_prepare_token_distribution(const gfo_token_logit* cands, uint32_t n,
                                   const gfo_sampler_options* opt, const uint32_t* history,
                                   uint32_t history_count, gfo_prepared* out) {
    if (!options_valid(*opt)) return -1;
    if (n == 0 || n > kMaxCandidates) return -2;
    if (history_count > kMaxHistory) return -3;
    // request.top_k is 1 for greedy, options.top_k otherwise (sampling.cpp:363-365)
    const uint32_t request_top_k = opt->temperature == 0.0f ? 1u : opt->top_k;

    std::array<gfo_token_logit, kMaxCandidates> c {};
    size_t count = 0;
    for (uint32_t i = 0; i < n; ++i) {
        if (!std::isfinite(cands[i].logit)) return -4;
        size_t e = 0;
        for (; e < count; ++e)
            if (c[e].token == cands[i].token) break;
        if (e == count) c[count++] = cands[i];
        else if (cands[i].logit != c[e].logit) return -5;
    }
    if (count < request_top_k) return -6;
    for (size_t i = 0; i < count; ++i) {
        if (std::find(history, history + history_count, c[i].token) != history + history_count)
            c[i].logit = c[i].logit < 0.0f ? c[i].logit * opt->repetition_penalty
                                           : c[i].logit / opt->repetition_penalty;
    }
    std::sort(c.begin(), c.begin() + count, better);
    count = std::min<size_t>(count, request_top_k);

    std::memset(out, 0, sizeof(*out));
    if (opt->temperature == 0.0f) {
        out->token[0] = c[0].token;
        out->probability[0] = 1.0;
        out->sampling_weight[0] = 1.0;
        out->count = 1;
        out->total_sampling_weight = 1.0;
        return 0;
    }
    std::array<double, kMaxTopK> w {};
    const float max_logit = c[0].logit;
    for (size_t i = 0; i < count; ++i) w[i] = std::exp(static_cast<double>(c[i].logit - max_logit));
    double total = 0.0;
    for (size_t i = 0; i < count; ++i) total += w[i];
    double retained = 0.0;
    size_t kept = 0;
    do {
        retained += w[kept++];
    } while (kept < count && retained / total < static_cast<double>(opt->top_p));
    count = kept;
    if (opt->min_p > 0.0f) {
        size_t m = 1;
        while (m < count && w[m] >= static_cast<double>(opt->min_p)) ++m;
        count = m;
    }
    double norm = 0.0;
    for (size_t i = 0; i < count; ++i) {
        w[i] = std::exp(static_cast<double>(c[i].logit - max_logit) / static_cast<double>(opt->temperature));
        norm += w[i];
    }
    if (!std::isfinite(norm) || norm <= 0.0) return -7;
    out->count = static_cast<uint32_t>(count);
    out->total_sampling_weight = norm;
    for (size_t i = 0; i < count; ++i) {
        out->token[i] = c[i].token;
        out->probability[i] = w[i] / norm;
        out->sampling_weight[i] = w[i];
    }
    return 0;
}

static int compact_law(const float* logits, uint32_t vocab, const gfo_sampler_options* opt,
                       const int32_t* draft_to_target, gfo_draft_law* out);

int gfo_draft_law_compact(const float* logits, uint32_t vocab, const gfo_sampler_options* opt,
                          gfo_draft_law* out) {
    return compact_law(logits, vocab, opt, nullptr, out);
}

// with the drafter's vocabulary map: a draft token without a target token (map < 0) is suppressed, its
// raw logit is still validated (gd_process, gd_compact_collect: src/engine/gemma3_draft.mm:191-204, 237-243)
int gfo_draft_law_compact_mapped(const float* logits, uint32_t vocab, const gfo_sampler_options* opt,
                                 const int32_t* draft_to_target, gfo_draft_law* out) {
    return compact_law(logits, vocab, opt, draft_to_target, out);
}

static int compact_law(const float* logits, uint32_t vocab, const gfo_sampler_options* opt,
                       const int32_t* draft_to_target, gfo_draft_law* out) {
    if (!options_valid(*opt) || opt->temperature <= 0.0f || opt->top_k > 64) return -1;
    std::memset(out, 0, sizeof(*out));
    // gd_process: validate, score = logit / T (repetition penalty handled by the caller's logits)
    std::vector<float> score(vocab);
    for (uint32_t i = 0; i < vocab; ++i) {
        if (!std::isfinite(logits[i])) return -10;
        if (draft_to_target && draft_to_target[i] < 0) { score[i] = -std::numeric_limits<float>::infinity(); continue; }
        float s = logits[i];
        s /= opt->temperature;
        if (!std::isfinite(s)) return -11;
        score[i] = s;
    }
    // k-th best by (score desc, token asc)
    const uint32_t k = std::min(opt->top_k, vocab);
    std::vector<Scored> all(vocab);
    for (uint32_t i = 0; i < vocab; ++i) all[i] = {i, score[i]};
    std::partial_sort(all.begin(), all.begin() + k, all.end(), better_scored);
    const float cutoff = all[k - 1].score;
    // gd_compact_collect: every token whose score >= the k-th best (ties included)
    std::vector<Scored> v;
    for (uint32_t i = 0; i < vocab; ++i)
        if (!(draft_to_target && draft_to_target[i] < 0) && !(score[i] < cutoff)) v.push_back({i, score[i]});
    if (v.empty()) return -12;
    if (v.size() > 256) return 1;
    const uint32_t n = static_cast<uint32_t>(v.size());
    std::sort(v.begin(), v.end(), better_scored);
    std::array<float, 256> w {};
    for (uint32_t i = 0; i < n; ++i) w[i] = gfo_exp_f32(v[i].score - v[0].score);
    float total = 0.0f, tail = 0.0f;
    for (uint32_t j = n; j > 0; --j) total += w[j - 1];
    for (uint32_t j = n; j > 0; --j) {
        const uint32_t i = j - 1;
        tail += w[i];
        const bool keep = i == 0
            || ((opt->top_p >= 1.0f || tail / total > 1.0f - opt->top_p)
                && (opt->min_p <= 0.0f || w[i] >= opt->min_p));
        if (!keep) v[i].score = -std::numeric_limits<float>::infinity();
    }
    std::sort(v.begin(), v.end(), [](const Scored& a, const Scored& b) { return a.token < b.token; });
    float maximum = -std::numeric_limits<float>::infinity();
    for (uint32_t i = 0; i < n; ++i) maximum = std::max(maximum, v[i].score);
    total = 0.0f;
    for (uint32_t i = 0; i < n; ++i) {
        w[i] = gfo_exp_f32(v[i].score - maximum);
        total += w[i];
    }
    if (!(total > 0.0f) || !std::isfinite(total)) return -13;
    float prefix = 0.0f;
    uint64_t last = 0;
    out->count = n;
    out->cdf[0] = 0;
    for (uint32_t i = 0; i < n; ++i) {
        out->ids[i] = v[i].token;
        prefix += w[i];
        float scaled = (prefix / total) * 4294967296.0f;
        scaled = std::min(std::max(scaled, 0.0f), 4294967296.0f);
        const uint64_t next = static_cast<uint64_t>(scaled);
        out->cdf[i + 1] = next;
        if (next < last || next > kMassTotal) return -14;
        last = next;
    }
    if (last != kMassTotal) return -15;
    return 0;
}

static int full_law(const float* logits, uint32_t vocab, const gfo_sampler_options* opt,
                    const int32_t* draft_to_target, uint64_t* cdf);

int gfo_draft_law_full(const float* logits, uint32_t vocab, const gfo_sampler_options* opt,
                       uint64_t* cdf) {
    return full_law(logits, vocab, opt, nullptr, cdf);
}

// with the drafter's vocabulary map: gd_process gives a token without a target id the score -inf before
// either law is built (src/engine/gemma3_draft.mm:191-204), so it sorts last, weighs nothing and keeps an
// empty bin; its raw logit is validated all the same
int gfo_draft_law_full_mapped(const float* logits, uint32_t vocab, const gfo_sampler_options* opt,
                              const int32_t* draft_to_target, uint64_t* cdf) {
    return full_law(logits, vocab, opt, draft_to_target, cdf);
}

static int full_law(const float* logits, uint32_t vocab, const gfo_sampler_options* opt,
                    const int32_t* draft_to_target, uint64_t* cdf) {
    // Full-vocabulary law (gemma3_draft.mm:295-395 in the dispatch order of :1040-1166), entered
    // when top_k > 64, when drafting greedily, or when the compact support overflows:
    // tiles of 256 tokens, f32 prefix inside a tile, f32 running offsets across tiles.
    if (!options_valid(*opt) || opt->temperature < 0.0f || vocab == 0 || vocab % 256 != 0) return -1;
    if (opt->temperature == 0.0f) {
        // greedy drafting: no transform, no filter; all mass on the lowest-id maximum
        // (gd_max / gd_max_finish, then gd_cdf's step function, gemma3_draft.mm:338-379)
        uint32_t best = 0xFFFFFFFFu;
        for (uint32_t i = 0; i < vocab; ++i) {
            if (!std::isfinite(logits[i])) return -10;
            if (draft_to_target && draft_to_target[i] < 0) continue;
            if (best == 0xFFFFFFFFu || logits[i] > logits[best]) best = i;
        }
        if (best == 0xFFFFFFFFu) return -6;
        for (uint32_t i = 0; i <= vocab; ++i) cdf[i] = i <= best ? 0 : kMassTotal;
        return 0;
    }
    std::vector<float> score(vocab);
    for (uint32_t i = 0; i < vocab; ++i) {
        if (!std::isfinite(logits[i])) return -10;
        if (draft_to_target && draft_to_target[i] < 0) { score[i] = -std::numeric_limits<float>::infinity(); continue; }
        score[i] = logits[i] / opt->temperature;
        if (!std::isfinite(score[i])) return -11;
    }
    // sorted view for top-k cutoff and the descending-tail top-p / min-p filter
    std::vector<Scored> sorted(vocab);
    for (uint32_t i = 0; i < vocab; ++i) sorted[i] = {i, score[i]};
    std::sort(sorted.begin(), sorted.end(), better_scored);
    const float cutoff = opt->top_k ? sorted[std::min(opt->top_k, vocab) - 1].score
                                    : -std::numeric_limits<float>::infinity();
    const uint32_t tiles = vocab / 256;
    std::vector<float> prefix(vocab), offsets(tiles + 1);
    std::vector<float> totals(tiles);
    for (uint32_t g = 0; g < tiles; ++g) {  // gd_filter_prefix: ascending tail order
        float t = 0.0f;
        for (uint32_t j = 0; j < 256; ++j) {
            const Scored item = sorted[vocab - 1 - (g * 256 + j)];
            const float w = item.score >= cutoff ? gfo_exp_f32(item.score - sorted[0].score) : 0.0f;
            t += w;
            prefix[g * 256 + j] = t;
        }
        totals[g] = t;
    }
    float s = 0.0f;
    offsets[0] = 0.0f;
    for (uint32_t g = 0; g < tiles; ++g) { s += totals[g]; offsets[g + 1] = s; }
    std::vector<uint8_t> eligible(vocab, 0);
    for (uint32_t i = 0; i < vocab; ++i) {  // gd_filter_apply
        const Scored item = sorted[vocab - 1 - i];
        bool keep = item.score >= cutoff;
        const float tail = (offsets[i / 256] + prefix[i]) / offsets[tiles];
        if (opt->top_p < 1.0f && tail <= 1.0f - opt->top_p && i != vocab - 1) keep = false;
        if (opt->min_p > 0.0f && gfo_exp_f32(item.score - sorted[0].score) < opt->min_p && i != vocab - 1)
            keep = false;
        eligible[item.token] = keep ? 1 : 0;
        if (!keep) score[item.token] = -std::numeric_limits<float>::infinity();
    }
    float maximum = -std::numeric_limits<float>::infinity();
    for (uint32_t i = 0; i < vocab; ++i)
        if (eligible[i] && score[i] > maximum) maximum = score[i];
    if (!std::isfinite(maximum)) return -6;
    for (uint32_t g = 0; g < tiles; ++g) {  // gd_prefix (temperature already folded: divide by 1)
        float t = 0.0f;
        for (uint32_t j = 0; j < 256; ++j) {
            const uint32_t i = g * 256 + j;
            t += eligible[i] ? gfo_exp_f32((score[i] - maximum) / 1.0f) : 0.0f;
            prefix[i] = t;
        }
        totals[g] = t;
    }
    s = 0.0f;
    for (uint32_t g = 0; g < tiles; ++g) { s += totals[g]; offsets[g + 1] = s; }
    if (!(s > 0.0f) || !std::isfinite(s)) return -7;
    for (uint32_t i = 0; i <= vocab; ++i) {  // gd_cdf
        if (i == 0) { cdf[i] = 0; continue; }
        if (i == vocab) { cdf[i] = kMassTotal; continue; }
        const uint32_t b = i / 256;
        const float sum = (i % 256 == 0) ? offsets[b] : offsets[b] + prefix[i - 1];
        float scaled = (sum / offsets[tiles]) * 4294967296.0f;
        scaled = std::min(std::max(scaled, 0.0f), 4294967296.0f);
        cdf[i] = static_cast<uint64_t>(scaled);
    }
    for (uint32_t i = 0; i < vocab; ++i) {  // gd_select's validation
        if (cdf[i] > cdf[i + 1] || cdf[i + 1] > kMassTotal) return -8;
        if (cdf[i] < cdf[i + 1] && !eligible[i]) return -9;
    }
    return 0;
}

uint32_t gfo_draft_select(const gfo_draft_law* law, uint32_t word) {
    for (uint32_t i = 0; i < law->count; ++i)
        if (uint64_t(word) >= law->cdf[i] && uint64_t(word) < law->cdf[i + 1]) return law->ids[i];
    return 0xFFFFFFFFu;
}

uint32_t gfo_draft_select_full(const uint64_t* cdf, uint32_t vocab, uint32_t word) {
    for (uint32_t i = 0; i < vocab; ++i)
        if (uint64_t(word) >= cdf[i] && uint64_t(word) < cdf[i + 1]) return i;
    return 0xFFFFFFFFu;
}

namespace {
int spec_from_prepared(const gfo_prepared* target_in, const LawView& view,
                       uint32_t proposal, double u_accept, double u_residual,
                       gfo_spec_result* out) {
    const LawView* law = &view;
    const gfo_prepared& target = *target_in;
    std::memset(out, 0, sizeof(*out));
    auto unit = [](double u) { return std::isfinite(u) && u >= 0.0 && u < 1.0; };
    if (!unit(u_accept) || !unit(u_residual)) return -20;
    const double normalization = validated_total(target);
    if (normalization < 0.0) return -21;
    uint64_t begin = 0;
    const uint64_t proposal_mass = law_mass(*law, proposal, &begin);
    if (proposal_mass == 0 || proposal_mass > kMassTotal || begin > kMassTotal - proposal_mass) return -22;
    // gather: q masses on p's support, in p's order; tokens outside q's support have q = 0
    uint64_t gathered = 0;
    bool proposal_in_target = false;
    std::array<uint64_t, kMaxTopK> q {};
    for (uint32_t i = 0; i < target.count; ++i) {
        q[i] = law_mass(*law, target.token[i], nullptr);
        if (q[i] > kMassTotal - gathered) return -23;
        gathered += q[i];
        if (target.token[i] == proposal) proposal_in_target = true;
    }
    if (!proposal_in_target && proposal_mass > kMassTotal - gathered) return -24;

    const double proposed_probability = static_cast<double>(proposal_mass) / static_cast<double>(kMassTotal);
    double acceptance = 0.0;
    gfo_prepared residual;
    std::memset(&residual, 0, sizeof(residual));
    for (uint32_t i = 0; i < target.count; ++i) {
        const double p = target.sampling_weight[i] / normalization;
        if (target.token[i] == proposal) acceptance = std::min(1.0, p / proposed_probability);
        const double qi = static_cast<double>(q[i]) / static_cast<double>(kMassTotal);
        const double diff = p - qi;
        if (diff <= 0.0) continue;
        residual.token[residual.count] = target.token[i];
        residual.sampling_weight[residual.count] = diff;
        ++residual.count;
        residual.total_sampling_weight += diff;
    }
    if (residual.count != 0) {
        for (uint32_t i = 0; i < residual.count; ++i)
            residual.probability[i] = residual.sampling_weight[i] / residual.total_sampling_weight;
    } else if (acceptance < 1.0) {
        return -25;
    }
    out->acceptance_probability = acceptance;
    out->residual_total = residual.total_sampling_weight;
    out->residual_count = residual.count;
    if (u_accept < acceptance) {
        out->accepted = 1;
        out->token = proposal;
        out->next_root = proposal;
        return 0;
    }
    if (validated_total(residual) < 0.0) return -26;
    out->accepted = 0;
    out->token = select_prepared(residual, u_residual * residual.total_sampling_weight);
    out->next_root = out->token;
    return 0;
}

// per-row sampler history (the reference's SamplerHistorySnapshot: the tokens a repetition
// penalty applies to, src/engine/sampling.cpp:430-446); null for none
struct RowHistory { const uint32_t* tokens[2]; uint32_t count[2]; };

int spec_accept(const gfo_token_logit* row0, uint32_t n0, const gfo_token_logit* row1, uint32_t n1,
                const LawView& law, uint32_t proposal, const gfo_sampler_options* opt, double u_accept,
                double u_residual, double u_next, gfo_spec_result* out, const RowHistory& hist = RowHistory{}) {
    std::memset(out, 0, sizeof(*out));
    if (!(std::isfinite(u_next) && u_next >= 0.0 && u_next < 1.0)) return -20;
    gfo_prepared target;
    int rc = gfo_prepare_token_distribution(row0, n0, opt, hist.tokens[0], hist.count[0], &target);
    if (rc) return rc;
    rc = spec_from_prepared(&target, law, proposal, u_accept, u_residual, out);
    if (rc || !out->accepted) return rc;
    // a fully accepted chain leaves row 1's candidates to seed the next root
    gfo_prepared next;
    rc = gfo_prepare_token_distribution(row1, n1, opt, hist.tokens[1], hist.count[1], &next);
    if (rc) return rc - 100;
    out->next_root = opt->temperature == 0.0f
        ? next.token[0] : select_prepared(next, u_next * next.total_sampling_weight);
    return 0;
}
}  // namespace

int gfo_spec_from_prepared(const gfo_prepared* target, const gfo_draft_law* law, uint32_t proposal,
                           double u_accept, double u_residual, gfo_spec_result* out) {
    return spec_from_prepared(target, LawView{law, nullptr, 0}, proposal, u_accept, u_residual, out);
}

int gfo_spec_accept(const gfo_token_logit* row0, uint32_t n0, const gfo_token_logit* row1,
                    uint32_t n1, const gfo_draft_law* law, uint32_t proposal,
                    const gfo_sampler_options* opt, double u_accept, double u_residual,
                    double u_next, gfo_spec_result* out) {
    return spec_accept(row0, n0, row1, n1, LawView{law, nullptr, 0}, proposal, opt, u_accept, u_residual, u_next, out);
}

int gfo_spec_accept_history(const gfo_token_logit* row0, uint32_t n0, const uint32_t* history0, uint32_t count0,
                            const gfo_token_logit* row1, uint32_t n1, const uint32_t* history1, uint32_t count1,
                            const gfo_draft_law* law, uint32_t proposal, const gfo_sampler_options* opt,
                            double u_accept, double u_residual, double u_next, gfo_spec_result* out) {
    const RowHistory h {{history0, history1}, {count0, count1}};
    return spec_accept(row0, n0, row1, n1, LawView{law, nullptr, 0}, proposal, opt, u_accept, u_residual, u_next, out, h);
}

// Gemma3DraftPlan::gather for one target token (src/engine/gemma3_draft.mm:1570-1578): its mass under a
// compact law in draft ids and the start of its interval; target_to_draft may be null (shared vocabulary)
uint64_t gfo_law_mass_mapped(const gfo_draft_law* law, const int32_t* target_to_draft, uint32_t token, uint64_t* begin) {
    return law_mass(LawView{law, nullptr, 0, target_to_draft}, token, begin);
}

int gfo_spec_accept_mapped(const gfo_token_logit* row0, uint32_t n0, const uint32_t* history0, uint32_t count0,
                           const gfo_token_logit* row1, uint32_t n1, const uint32_t* history1, uint32_t count1,
                           const gfo_draft_law* law, const int32_t* target_to_draft, uint32_t proposal,
                           const gfo_sampler_options* opt, double u_accept, double u_residual, double u_next,
                           gfo_spec_result* out) {
    const RowHistory h {{history0, history1}, {count0, count1}};
    return spec_accept(row0, n0, row1, n1, LawView{law, nullptr, 0, target_to_draft}, proposal, opt, u_accept, u_residual,
                       u_next, out, h);
}

int gfo_spec_accept_full_mapped(const gfo_token_logit* row0, uint32_t n0, const gfo_token_logit* row1,
                                uint32_t n1, const uint64_t* cdf, uint32_t vocab, const int32_t* target_to_draft,
                                uint32_t proposal, const gfo_sampler_options* opt, double u_accept,
                                double u_residual, double u_next, gfo_spec_result* out) {
    return spec_accept(row0, n0, row1, n1, LawView{nullptr, cdf, vocab, target_to_draft}, proposal, opt, u_accept, u_residual,
                       u_next, out);
}

int gfo_spec_accept_full(const gfo_token_logit* row0, uint32_t n0, const gfo_token_logit* row1,
                         uint32_t n1, const uint64_t* cdf, uint32_t vocab, uint32_t proposal,
                         const gfo_sampler_options* opt, double u_accept, double u_residual,
                         double u_next, gfo_spec_result* out) {
    return spec_accept(row0, n0, row1, n1, LawView{nullptr, cdf, vocab}, proposal, opt, u_accept, u_residual, u_next, out);
}

void gfo_philox4x32_10(const uint32_t counter[4], const uint32_t key[2], uint32_t out[4]) {
    uint32_t c0 = counter[0], c1 = counter[1], c2 = counter[2], c3 = counter[3];
    uint32_t k0 = key[0], k1 = key[1];
    for (int round = 0; round < 10; ++round) {
        const uint64_t p0 = uint64_t{0xD2511F53u} * c0;
        const uint64_t p1 = uint64_t{0xCD9E8D57u} * c2;
        const uint32_t n0 = static_cast<uint32_t>(p1 >> 32) ^ c1 ^ k0;
        const uint32_t n1 = static_cast<uint32_t>(p1);
        const uint32_t n2 = static_cast<uint32_t>(p0 >> 32) ^ c3 ^ k1;
        const uint32_t n3 = static_cast<uint32_t>(p0);
        c0 = n0; c1 = n1; c2 = n2; c3 = n3;
        k0 += 0x9E3779B9u;
        k1 += 0xBB67AE85u;
    }
    out[0] = c0; out[1] = c1; out[2] = c2; out[3] = c3;
}

static inline double unit_double(uint32_t hi, uint32_t lo) {
    const uint64_t bits = ((uint64_t{hi} << 32) | lo) >> 11;  // 53 bits
    return static_cast<double>(bits) * 0x1.0p-53;
}

void gfo_step_draws(uint64_t seed, uint64_t step, uint32_t* word, double* u_accept,
                    double* u_residual, double* u_next) {
    const uint32_t key[2] = {static_cast<uint32_t>(seed), static_cast<uint32_t>(seed >> 32)};
    uint32_t a[4], b[4];
    const uint32_t c0[4] = {static_cast<uint32_t>(step), static_cast<uint32_t>(step >> 32), 0, 0};
    const uint32_t c1[4] = {static_cast<uint32_t>(step), static_cast<uint32_t>(step >> 32), 1, 0};
    gfo_philox4x32_10(c0, key, a);
    gfo_philox4x32_10(c1, key, b);
    *word = a[0];
    *u_accept = unit_double(a[1], a[2]);
    *u_residual = unit_double(b[0], b[1]);
    *u_next = unit_double(b[2], b[3]);
}

uint32_t gfo_selection_request(const gfo_selection_row* raw, uint32_t vocab, uint32_t top_k,
                               int repetition_enabled, gfo_resolved_row* out) {
    std::memset(out, 0, sizeof *out);
    out->top_k = top_k;
    out->base_candidate_count = top_k;
    const uint32_t limit = raw->history_window_limit;
    if (limit > 64 || raw->history_length > limit || raw->suffix_count > 23
        || (raw->history_length == 0 && raw->history_head != 0)
        || (raw->history_length > 0 && raw->history_head >= limit))
        return 2u;
    uint32_t status = 0;
    // the ring as the sampler keeps it: appending to a full window overwrites the oldest slot
    uint32_t ring[64], head = raw->history_head, length = raw->history_length;
    for (uint32_t i = 0; i < 64; ++i) ring[i] = raw->history_token_ids[i];
    for (uint32_t i = 0; i < length; ++i)
        if (ring[(head + i) % limit] >= vocab) status |= 4u;
    for (uint32_t i = 0; i < raw->suffix_count; ++i) {
        const uint32_t token = raw->suffix_token_ids[i];
        if (token >= vocab) status |= 4u;
        if (limit == 0) continue;
        if (length < limit) {
            ring[(head + length) % limit] = token;
            ++length;
        } else {
            ring[head] = token;
            head = (head + 1) % limit;
        }
    }
    if (repetition_enabled) {
        for (uint32_t i = 0; i < length; ++i) {
            const uint32_t token = ring[(head + i) % limit];
            if (token >= vocab) continue;
            bool seen = false;
            for (uint32_t j = 0; j < out->history_count; ++j) seen = seen || out->history_token_ids[j] == token;
            if (!seen) out->history_token_ids[out->history_count++] = token;
        }
    }
    out->base_candidate_count = top_k + out->history_count;
    return status;
}

}  // extern "C"
