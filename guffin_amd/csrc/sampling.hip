// Proposal law of the drafter and lossless accept / residual sampling (gfx950).
//
// Reference behaviour:
//   compact proposal law (integer 2^32-mass CDF)   src/engine/gemma3_draft.mm:191-294, 995-1070
//   gather of q on p's support                     src/engine/gemma3_draft.mm:1528-1581
//   target law p (all double)                      src/engine/sampling.cpp:394-499
//   validation / Neumaier total                    src/engine/sampling.cpp:117-158
//   accept min(1,p/q), residual max(p-q,0)         src/engine/sampling.cpp:561-656
//   inverse-CDF selections                         src/engine/sampling.cpp:247-257, 501-514
//   draw consumption order                         src/engine/sampling.cpp:896-934
// The reference evaluates the target law and the accept test on the host from a compact
// read-back; here both run on the device in the same fp64 operation order (sequential sums
// are taken by one lane in the reference's order), so decisions depend only on the inputs and
// the draws.  Draws come from Philox4x32-10 keyed (seed, step) unless injected.
#include "common.hpp"

namespace guffin {
namespace {

constexpr uint32_t kMaxTopK = 256, kMaxCandidates = 384, kHistoryCap = 64;
constexpr uint64_t kMassTotal = uint64_t{1} << 32;
constexpr uint32_t kLawFull = 0xFFFFFFFFu;  // DraftLaw::count of a law held as a full-vocabulary table

struct Candidates { uint32_t count; uint32_t status; struct { uint32_t token; float logit; } values[384]; };
struct DraftLaw { uint32_t count; uint32_t pad; uint32_t ids[256]; uint64_t cdf[257]; };
struct SamplerOptions { float temperature; uint32_t top_k; float top_p; float min_p; float repetition_penalty; };
struct StepDraws { uint32_t word; uint32_t pad; double u_accept, u_residual, u_next; };
struct SpecResult {
    uint32_t accepted, token, next_root, status;
    double acceptance_probability, residual_total;
    uint32_t residual_count, proposal;
};

// ---- Philox4x32-10 ----------------------------------------------------------------------
__device__ __forceinline__ void philox(uint32_t c0, uint32_t c1, uint32_t c2, uint32_t c3, uint32_t k0, uint32_t k1,
                                       uint32_t (&out)[4]) {
#pragma unroll
    for (int round = 0; round < 10; ++round) {
        const uint64_t p0 = uint64_t{0xD2511F53u} * c0, p1 = uint64_t{0xCD9E8D57u} * c2;
        const uint32_t n0 = static_cast<uint32_t>(p1 >> 32) ^ c1 ^ k0, n1 = static_cast<uint32_t>(p1);
        const uint32_t n2 = static_cast<uint32_t>(p0 >> 32) ^ c3 ^ k1, n3 = static_cast<uint32_t>(p0);
        c0 = n0; c1 = n1; c2 = n2; c3 = n3;
        k0 += 0x9E3779B9u; k1 += 0xBB67AE85u;
    }
    out[0] = c0; out[1] = c1; out[2] = c2; out[3] = c3;
}
__device__ __forceinline__ double unit_double(uint32_t hi, uint32_t lo) {
    return static_cast<double>(((uint64_t{hi} << 32) | lo) >> 11) * 0x1.0p-53;
}
// word, u_accept from counter (step, 0); u_residual, u_next from counter (step, 1)
__device__ __forceinline__ StepDraws step_draws(uint64_t seed, uint64_t step) {
    uint32_t a[4], b[4];
    const uint32_t k0 = static_cast<uint32_t>(seed), k1 = static_cast<uint32_t>(seed >> 32);
    const uint32_t s0 = static_cast<uint32_t>(step), s1 = static_cast<uint32_t>(step >> 32);
    philox(s0, s1, 0, 0, k0, k1, a);
    philox(s0, s1, 1, 0, k0, k1, b);
    StepDraws d;
    d.word = a[0]; d.pad = 0;
    d.u_accept = unit_double(a[1], a[2]);
    d.u_residual = unit_double(b[0], b[1]);
    d.u_next = unit_double(b[2], b[3]);
    return d;
}

// exp for the law's f32 weights from IEEE-exact operations only (fma, floor, exponent
// scaling), so the integer CDF is reproducible bit for bit on any conforming machine.
__device__ __forceinline__ float law_exp(float x) {
    if (!(x > -86.0f)) return x != x ? x : 0.0f;
    if (x > 88.0f) return INFINITY;
    const float kf = floorf(fmaf(x, 1.44269502162933349609375f, 0.5f));
    float r = fmaf(kf, -0.693145751953125f, x);
    r = fmaf(kf, -1.428606765330187045037746429443359375e-06f, r);
    float p = 1.0f / 5040.0f;
    p = fmaf(p, r, 1.0f / 720.0f);
    p = fmaf(p, r, 1.0f / 120.0f);
    p = fmaf(p, r, 1.0f / 24.0f);
    p = fmaf(p, r, 1.0f / 6.0f);
    p = fmaf(p, r, 0.5f);
    p = fmaf(p, r, 1.0f);
    p = fmaf(p, r, 1.0f);
    const int k = static_cast<int>(kf);
    return __fmul_rn(p, __uint_as_float(static_cast<uint32_t>(k + 127) << 23));
}

__device__ __forceinline__ bool options_valid(const SamplerOptions& o) {
    return isfinite(o.temperature) && o.temperature >= 0.f && o.top_k >= 1 && o.top_k <= kMaxTopK
        && isfinite(o.top_p) && o.top_p > 0.f && o.top_p <= 1.f && isfinite(o.min_p) && o.min_p >= 0.f
        && o.min_p <= 1.f && isfinite(o.repetition_penalty) && o.repetition_penalty > 0.f;
}

// bitonic sort of n (power of two) 64-bit keys in LDS, ascending or descending
__device__ __forceinline__ void bitonic(uint64_t* keys, uint32_t n, bool desc) {
    for (uint32_t width = 2; width <= n; width <<= 1)
        for (uint32_t stride = width >> 1; stride > 0; stride >>= 1) {
            __syncthreads();
            for (uint32_t i = threadIdx.x; i < n / 2; i += blockDim.x) {
                const uint32_t lo = 2 * i - (i & (stride - 1)), hi = lo + stride;
                const bool first_dir = (lo & width) == 0;
                const uint64_t a = keys[lo], b = keys[hi];
                if (((a < b) == desc) == first_dir) { keys[lo] = b; keys[hi] = a; }
            }
        }
    __syncthreads();
}

// Sort of the first n keys in LDS by rank, n at most the workgroup's size: every thread counts the keys that go
// before its own (all lanes read the same word: a broadcast) and drops its key at that place.  Three barriers
// instead of the bitonic network's one per stage (28 for 128 keys, 45 for 512).
// Distinct keys, ascending: a permutation of the n places.
__device__ __forceinline__ void rank_sort_ascending(uint64_t* keys, uint32_t n) {
    __syncthreads();
    const uint32_t t = threadIdx.x;
    const uint64_t mine = t < n ? keys[t] : 0;
    uint32_t rank = 0;
    if (t < n)
        for (uint32_t j = 0; j < n; ++j) rank += keys[j] < mine;
    __syncthreads();
    if (t < n) keys[rank] = mine;
    __syncthreads();
}
// Descending, keys distinct except for zeros (padding and dropped duplicates), which end up behind the others in
// the first `span` places.
__device__ __forceinline__ void rank_sort_descending(uint64_t* keys, uint32_t n, uint32_t span) {
    __syncthreads();
    const uint32_t t = threadIdx.x;
    const uint64_t mine = t < n ? keys[t] : 0;
    uint32_t rank = 0;
    if (mine != 0)
        for (uint32_t j = 0; j < n; ++j) rank += keys[j] > mine;
    __syncthreads();
    if (t < span) keys[t] = 0;
    __syncthreads();
    if (mine != 0) keys[rank] = mine;
    __syncthreads();
}

__device__ __forceinline__ uint64_t score_key(float score, uint32_t token) {
    const uint32_t b = __float_as_uint(score + 0.0f);
    const uint32_t ordered = (b & 0x80000000u) ? ~b : (b | 0x80000000u);
    return (uint64_t(ordered) << 32) | (0xFFFFFFFFu - token);
}

// =========================================================================================
// Compact proposal law from the best 257 scores (sorted, score = logit / T)
// =========================================================================================
__global__ void __launch_bounds__(256)
draft_law_kernel(const Candidates* __restrict__ top, SamplerOptions opt, uint64_t seed, uint64_t step,
                 const StepDraws* __restrict__ injected, DraftLaw* __restrict__ law,
                 uint32_t* __restrict__ proposal, uint32_t* __restrict__ status, uint32_t* __restrict__ full_error) {
    // full_error != nullptr: the full-vocabulary kernels follow, guarded by law->count; a support of
    // more than 256 ties then hands over to them instead of failing
    __shared__ uint64_t keys[256];
    __shared__ float score[256], weight[256], running[256];
    __shared__ uint64_t edge[257];
    __shared__ uint32_t s_n, s_first, s_bad, s_chosen;
    const uint32_t t = threadIdx.x;
    const uint32_t avail = top->count;
    // every thread fetches its own entry once; the single-lane sections below work on LDS only
    const bool usable = options_valid(opt) && opt.temperature > 0.f && opt.top_k <= 64 && avail >= 1;
    const uint32_t k = usable ? (opt.top_k < avail ? opt.top_k : avail) : 1u;
    const float cutoff = usable ? top->values[k - 1].logit : 0.f;
    const float first_logit = usable ? top->values[0].logit : 0.f;
    const float my_logit = t < avail ? top->values[t].logit : -INFINITY;
    const uint32_t my_token = t < avail ? top->values[t].token : 0u;
    if (t == 0) { s_first = 256u; s_bad = 0; s_chosen = 0xFFFFFFFFu; }
    __syncthreads();
    // entries are sorted by (score desc, token asc): the support is a prefix, its length the first
    // entry that is below the cutoff or -inf
    if (!(t < avail && !(my_logit < cutoff) && my_logit != -INFINITY)) atomicMin(&s_first, t);
    __syncthreads();
    if (t == 0) {
        uint32_t st = 0, n = 0;
        if (!usable) st = GUFFIN_STATUS_LAW_INVALID;
        if (top->status & GUFFIN_STATUS_NONFINITE) st = GUFFIN_STATUS_LAW_INVALID | GUFFIN_STATUS_NONFINITE;
        if (!st) {
            n = s_first;
            if (n == 256u && avail > 256u) {   // all 256 are in: a 257th eligible entry overflows the compact law
                const float more = top->values[256].logit;
                if (!(more < cutoff) && more != -INFINITY) n = 257u;
            }
            if (n == 0) st = GUFFIN_STATUS_LAW_INVALID;  // nothing eligible
            if (n > 256) st = GUFFIN_STATUS_LAW_INVALID | 32u;  // support overflow: needs the full-vocabulary law
        }
        s_n = st ? 0 : n;
        if (full_error) *full_error = 0;
        if (st == (GUFFIN_STATUS_LAW_INVALID | 32u) && full_error) { law->count = kLawFull; *proposal = 0xFFFFFFFFu; }
        else if (st) { atomicOr(status, st); law->count = 0; *proposal = 0xFFFFFFFFu; }
    }
    __syncthreads();
    const uint32_t n = s_n;
    if (n == 0) return;
    score[t] = t < n ? my_logit : -INFINITY;
    weight[t] = t < n ? law_exp(my_logit - first_logit) : 0.f;
    __syncthreads();
    if (t == 0) {  // descending-tail top-p / min-p in the reference's sequential order
        // the tail sums from the last entry down; the last of them, in slot 0 (always kept), is the total: the
        // same adds in the same order
        float tail = 0.f;
        for (uint32_t j = n; j > 0; --j) {
            tail = __fadd_rn(tail, weight[j - 1]);
            running[j - 1] = tail;
        }
    }
    __syncthreads();
    if (t > 0 && t < n) {
        const bool keep = (opt.top_p >= 1.0f || __fdiv_rn(running[t], running[0]) > __fsub_rn(1.0f, opt.top_p))
                          && (opt.min_p <= 0.0f || weight[t] >= opt.min_p);
        if (!keep) score[t] = -INFINITY;
    }
    __syncthreads();
    // ascending token id; the score rides in the low half of the key
    keys[t] = t < n ? (uint64_t(my_token) << 32) | __float_as_uint(score[t]) : ~uint64_t{0};
    rank_sort_ascending(keys, n);   // entries beyond the support are all-ones keys already in their final place
    const float s = __uint_as_float(static_cast<uint32_t>(keys[t]));
    score[t] = t < n ? s : -INFINITY;
    __syncthreads();
    {   // the maximum of the support (a maximum does not depend on the order it is taken in)
        const float wave_best = wave_max(t < n ? score[t] : -INFINITY);
        if ((t & 63u) == 0) weight[t >> 6] = wave_best;
    }
    __syncthreads();
    const float maximum = fmaxf(fmaxf(weight[0], weight[1]), fmaxf(weight[2], weight[3]));
    __syncthreads();
    weight[t] = t < n ? law_exp(__fsub_rn(score[t], maximum)) : 0.f;
    __syncthreads();
    if (t == 0) {   // the f32 running sums in token order; the quotients and edges are per-lane work
        float prefix = 0.f;
        for (uint32_t i = 0; i < n; ++i) { prefix = __fadd_rn(prefix, weight[i]); running[i] = prefix; }
        edge[0] = 0;
    }
    __syncthreads();
    const float total = running[n - 1];
    const bool total_ok = total > 0.f && isfinite(total);
    uint64_t next = 0;
    if (t < n) {
        float scaled = __fmul_rn(__fdiv_rn(running[t], total), 4294967296.0f);
        scaled = fminf(fmaxf(scaled, 0.0f), 4294967296.0f);
        next = static_cast<uint64_t>(scaled);
        edge[t + 1] = next;
    }
    __syncthreads();
    const StepDraws d = injected ? *injected : step_draws(seed, step);
    if (t < n) {
        const uint64_t last = edge[t];
        if (next < last || next > kMassTotal || (t == n - 1 && next != kMassTotal)) s_bad = 1;
        if (uint64_t(d.word) >= last && uint64_t(d.word) < next) s_chosen = static_cast<uint32_t>(keys[t] >> 32);
        law->ids[t] = static_cast<uint32_t>(keys[t] >> 32);
        law->cdf[t + 1] = next;
    }
    __syncthreads();
    if (t == 0) {
        law->count = n; law->pad = 0; law->cdf[0] = 0;
        const bool bad = !total_ok || s_bad;
        if (bad) atomicOr(status, GUFFIN_STATUS_LAW_INVALID);
        *proposal = bad ? 0xFFFFFFFFu : s_chosen;
    }
}

// =========================================================================================
// Full-vocabulary proposal law: the drafter's law when the compact support does not apply
// (top_k > 64, greedy drafting, or more than 256 tokens tied into the support).
// src/engine/gemma3_draft.mm:295-395 (kernels), :1040-1166 (dispatch order).  Every f32 sum is
// taken in the reference's order: sequentially inside a 256-token tile, then sequentially over
// the tile totals.  A guard pointer makes every kernel a no-op unless the compact kernel handed
// over (law->count == kLawFull), like the reference's compact-count guards.
// =========================================================================================
constexpr uint32_t kSortTile = 2048, kLawTile = 256;

struct FullLawWs {
    uint64_t* keys_a; uint64_t* keys_b;  // sort ping-pong, padded to a power of two
    float* scores;                       // processed score by token id; -inf once filtered out
    float* prefix;                       // running f32 sums inside each 256-tile
    float* offsets;                      // [tiles + 1] running sums of the tile totals
    float* best;                         // [0] maximum of the surviving scores, [1] argmax as bits
    uint32_t* error;                     // law-local error word (also mirrored into status)
};

__device__ __forceinline__ bool guarded_off(const uint32_t* guard) { return guard && *guard != kLawFull; }
__device__ __forceinline__ float key_score(uint64_t key) {
    const uint32_t o = static_cast<uint32_t>(key >> 32);
    return __uint_as_float((o & 0x80000000u) ? (o & 0x7FFFFFFFu) : ~o);
}
__device__ __forceinline__ uint32_t key_token(uint64_t key) { return 0xFFFFFFFFu - static_cast<uint32_t>(key); }
__device__ __forceinline__ void law_fail(uint32_t* status, uint32_t* error, uint32_t bits) {
    atomicOr(status, bits);
    atomicOr(error, bits);
}

// unguarded entry: claims the law slot for the full table
__global__ void law_begin_kernel(DraftLaw* law, uint32_t* proposal, uint32_t* error) {
    law->count = kLawFull; law->pad = 0; *proposal = 0xFFFFFFFFu; *error = 0;
}

// score = logit / T (gd_process), then 2048-token tiles sorted by (score desc, token asc)
__global__ void __launch_bounds__(1024)
law_sort_tile_kernel(const float* __restrict__ logits, uint32_t vocab, float temperature, bool sort, bool suppressed_ok,
                     const uint32_t* __restrict__ guard, FullLawWs ws, uint32_t* __restrict__ status) {
    if (guarded_off(guard)) return;
    __shared__ uint64_t keys[kSortTile];
    for (uint32_t e = threadIdx.x; e < kSortTile; e += blockDim.x) {
        const uint32_t token = blockIdx.x * kSortTile + e;
        uint64_t key = 0;  // padding sorts behind every real entry
        if (token < vocab) {
            float score = logits[token];
            // a score of -inf marks a draft token the vocabulary map gives no target token (its raw logit was
            // validated where the scores were made): it stays out of every sum and sorts last
            const bool suppressed = suppressed_ok && score == -INFINITY;
            if (!suppressed) {
                if (!isfinite(score)) { law_fail(status, ws.error, GUFFIN_STATUS_LAW_INVALID | GUFFIN_STATUS_NONFINITE); score = 0.f; }
                if (temperature > 0.f) score = __fdiv_rn(score, temperature);
                if (!isfinite(score)) { law_fail(status, ws.error, GUFFIN_STATUS_LAW_INVALID | GUFFIN_STATUS_NONFINITE); score = 0.f; }
            }
            ws.scores[token] = score;
            key = score_key(score, token);
        }
        keys[e] = key;
    }
    if (!sort) return;
    bitonic(keys, kSortTile, true);
    for (uint32_t e = threadIdx.x; e < kSortTile; e += blockDim.x) ws.keys_a[size_t(blockIdx.x) * kSortTile + e] = keys[e];
}

// one merge level of sorted runs of `width` keys (descending; keys are distinct except padding)
__global__ void __launch_bounds__(256)
law_merge_kernel(const uint64_t* __restrict__ in, uint64_t* __restrict__ out, uint32_t width, uint32_t padded,
                 const uint32_t* __restrict__ guard) {
    if (guarded_off(guard)) return;
    const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= padded) return;
    const uint32_t rank = i % (2 * width);
    const uint64_t* a = in + (i - rank);
    const uint64_t* b = a + width;
    uint32_t lo = rank > width ? rank - width : 0, hi = rank < width ? rank : width;
    while (lo < hi) {  // how many of the first `rank` outputs come from run a
        const uint32_t mid = (lo + hi) >> 1;
        if (a[mid] >= b[rank - mid - 1]) lo = mid + 1; else hi = mid;
    }
    const uint32_t ai = lo, bi = rank - lo;
    out[i] = (ai < width && (bi >= width || a[ai] >= b[bi])) ? a[ai] : b[bi];
}

// sequential offsets over the tile totals left in offsets[1..tiles] (gd_offsets); one thread
__device__ void finish_offsets(float* offsets, uint32_t tiles) {
    float s = 0.f;
    offsets[0] = 0.f;
    for (uint32_t g = 0; g < tiles; ++g) { s = __fadd_rn(s, offsets[g + 1]); offsets[g + 1] = s; }
}

// gd_filter_prefix + gd_offsets: weights of the sorted entries walked from the tail
__global__ void __launch_bounds__(1024)
law_filter_prefix_kernel(const uint64_t* __restrict__ sorted, uint32_t vocab, uint32_t top_k,
                         const uint32_t* __restrict__ guard, FullLawWs ws) {
    if (guarded_off(guard)) return;
    const uint32_t tiles = vocab / kLawTile;
    const float best = key_score(sorted[0]);
    const float cutoff = key_score(sorted[(top_k < vocab ? top_k : vocab) - 1]);
    for (uint32_t g = threadIdx.x; g < tiles; g += blockDim.x) {
        float run = 0.f;
        for (uint32_t j = 0; j < kLawTile; ++j) {
            const float score = key_score(sorted[vocab - 1 - (g * kLawTile + j)]);
            run = __fadd_rn(run, score >= cutoff ? law_exp(__fsub_rn(score, best)) : 0.f);
            ws.prefix[g * kLawTile + j] = run;
        }
        ws.offsets[g + 1] = run;
    }
    __threadfence();
    __syncthreads();
    if (threadIdx.x == 0) finish_offsets(ws.offsets, tiles);
}

// gd_filter_apply: top-k cutoff (ties kept), ascending-tail top-p, min-p; the best entry always stays
__global__ void __launch_bounds__(256)
law_filter_apply_kernel(const uint64_t* __restrict__ sorted, uint32_t vocab, SamplerOptions opt,
                        const uint32_t* __restrict__ guard, FullLawWs ws) {
    if (guarded_off(guard)) return;
    const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= vocab) return;
    const uint32_t tiles = vocab / kLawTile;
    const uint64_t item = sorted[vocab - 1 - i];
    const float score = key_score(item), best = key_score(sorted[0]);
    const float cutoff = key_score(sorted[(opt.top_k < vocab ? opt.top_k : vocab) - 1]);
    bool keep = score >= cutoff;
    const float tail = __fdiv_rn(__fadd_rn(ws.offsets[i / kLawTile], ws.prefix[i]), ws.offsets[tiles]);
    if (opt.top_p < 1.0f && tail <= __fsub_rn(1.0f, opt.top_p) && i != vocab - 1) keep = false;
    if (opt.min_p > 0.0f && law_exp(__fsub_rn(score, best)) < opt.min_p && i != vocab - 1) keep = false;
    if (!keep) ws.scores[key_token(item)] = -INFINITY;
}

// gd_max + gd_max_finish + gd_prefix + gd_offsets: maximum (lowest id on ties) of the surviving
// scores, then the weights exp(score - max) summed in token order
__global__ void __launch_bounds__(1024)
law_weights_kernel(uint32_t vocab, bool greedy, const uint32_t* __restrict__ guard, FullLawWs ws,
                   uint32_t* __restrict__ status) {
    if (guarded_off(guard)) return;
    __shared__ float s_max[1024];
    __shared__ uint32_t s_arg[1024];
    const uint32_t t = threadIdx.x, tiles = vocab / kLawTile;
    float m = -INFINITY;
    uint32_t arg = 0xFFFFFFFFu;
    for (uint32_t i = t; i < vocab; i += blockDim.x) {
        const float v = ws.scores[i];
        if (v > m) { m = v; arg = i; }  // ids ascend within a thread: the first maximum is the lowest id
    }
    s_max[t] = m; s_arg[t] = arg;
    __syncthreads();
    for (uint32_t half = blockDim.x >> 1; half > 0; half >>= 1) {
        if (t < half && (s_max[t + half] > s_max[t] || (s_max[t + half] == s_max[t] && s_arg[t + half] < s_arg[t]))) {
            s_max[t] = s_max[t + half]; s_arg[t] = s_arg[t + half];
        }
        __syncthreads();
    }
    const float maximum = s_max[0];
    if (t == 0) {
        ws.best[0] = maximum;
        ws.best[1] = __uint_as_float(s_arg[0]);
        if (!isfinite(maximum)) law_fail(status, ws.error, GUFFIN_STATUS_LAW_INVALID);
    }
    if (greedy) return;
    for (uint32_t g = t; g < tiles; g += blockDim.x) {
        float run = 0.f;
        for (uint32_t j = 0; j < kLawTile; ++j) {
            const float score = ws.scores[g * kLawTile + j];
            // the reference divides by a temperature of exactly 1 here: scores were tempered up front
            run = __fadd_rn(run, score > -INFINITY ? law_exp(__fdiv_rn(__fsub_rn(score, maximum), 1.0f)) : 0.f);
            ws.prefix[g * kLawTile + j] = run;
        }
        ws.offsets[g + 1] = run;
    }
    __threadfence();
    __syncthreads();
    if (t == 0) {
        finish_offsets(ws.offsets, tiles);
        const float total = ws.offsets[tiles];
        if (!(total > 0.f) || !isfinite(total)) law_fail(status, ws.error, GUFFIN_STATUS_LAW_INVALID);
    }
}

__device__ __forceinline__ uint64_t full_cdf_at(uint32_t i, uint32_t vocab, bool greedy, const FullLawWs& ws) {
    if (greedy) return i <= __float_as_uint(ws.best[1]) ? 0 : kMassTotal;
    if (i == 0) return 0;
    if (i == vocab) return kMassTotal;
    const uint32_t b = i / kLawTile;
    const float sum = (i % kLawTile == 0) ? ws.offsets[b] : __fadd_rn(ws.offsets[b], ws.prefix[i - 1]);
    float scaled = __fmul_rn(__fdiv_rn(sum, ws.offsets[vocab / kLawTile]), 4294967296.0f);
    scaled = fminf(fmaxf(scaled, 0.0f), 4294967296.0f);
    return static_cast<uint64_t>(scaled);
}

// gd_cdf + gd_select: the u64 table, its validation, and the token whose bin holds the step's word
__global__ void __launch_bounds__(256)
law_cdf_select_kernel(uint32_t vocab, bool greedy, uint64_t seed, uint64_t step, const StepDraws* __restrict__ injected,
                      const uint32_t* __restrict__ guard, FullLawWs ws, uint64_t* __restrict__ cdf,
                      uint32_t* __restrict__ proposal, uint32_t* __restrict__ status) {
    if (guarded_off(guard)) return;
    const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i > vocab) return;
    if (*ws.error != 0) { cdf[i] = 0; return; }  // raised by an earlier kernel: no law, no proposal
    const uint64_t begin = full_cdf_at(i, vocab, greedy, ws);
    cdf[i] = begin;
    if (i == vocab) return;
    const uint64_t end = full_cdf_at(i + 1, vocab, greedy, ws);
    if (begin > end || end > kMassTotal) { atomicOr(status, GUFFIN_STATUS_LAW_INVALID); return; }
    if (begin < end && !(ws.scores[i] > -INFINITY)) { atomicOr(status, GUFFIN_STATUS_LAW_INVALID); return; }
    const uint64_t word = injected ? injected->word : step_draws(seed, step).word;
    if (word >= begin && word < end) *proposal = i;
}

// =========================================================================================
// Target law (prepare_token_distribution) — whole workgroup, 512 threads
// =========================================================================================
struct Prepared {
    uint32_t count;
    double total;
    uint32_t token[kMaxTopK];
    double weight[kMaxTopK];
};

struct Scratch {
    uint64_t keys[512];
    float logit[512];
    double w[kMaxTopK];
    double run[kMaxTopK];            // running sums of w, taken by one lane in index order
    uint32_t tok[kMaxCandidates];    // the candidate record, staged once
    float raw[kMaxCandidates];
    uint32_t hist[kHistoryCap];
    uint32_t kept, cut;              // ends of the top-p and min-p prefixes
    uint32_t flag;
    double value;
    int err;
};

// returns 0 or a negative error; result in `out` (shared); uses all threads.  Sums whose order matters are
// taken by one lane over LDS; divisions, comparisons and exponentials are spread over the lanes.
__device__ int prepare_distribution(const Candidates* cand, const SamplerOptions& opt, const uint32_t* history,
                                    uint32_t history_count, Scratch& sc, Prepared& out) {
    const uint32_t t = threadIdx.x, n = cand->count;
    if (t == 0) sc.err = (!options_valid(opt) ? -1 : (n == 0 || n > kMaxCandidates) ? -2 : history_count > 64 ? -3 : 0);
    __syncthreads();
    if (sc.err) return sc.err;
    const uint32_t request_top_k = opt.temperature == 0.f ? 1u : opt.top_k;
    if (t < n) { sc.tok[t] = cand->values[t].token; sc.raw[t] = cand->values[t].logit; }
    if (t < history_count) sc.hist[t] = history[t];
    __syncthreads();
    // dedup (a later duplicate must carry the same logit), repetition penalty, sort key
    uint64_t key = 0;
    if (t < n) {
        const uint32_t token = sc.tok[t];
        float logit = sc.raw[t];
        bool dup = false;
        if (!isfinite(logit)) atomicMin(&sc.err, -4);
        for (uint32_t j = 0; j < t; ++j)
            if (sc.tok[j] == token) {
                dup = true;
                if (sc.raw[j] != logit) atomicMin(&sc.err, -5);
            }
        if (!dup) {
            for (uint32_t h = 0; h < history_count; ++h)
                if (sc.hist[h] == token) {
                    logit = logit < 0.f ? __fmul_rn(logit, opt.repetition_penalty) : __fdiv_rn(logit, opt.repetition_penalty);
                    break;
                }
            key = score_key(logit, token);
        }
    }
    if (t < 512) sc.keys[t] = key;
    __syncthreads();
    if (sc.err) return sc.err;
    uint32_t span = 64;   // the sort covers the record only (a real key is never 0, the padding is)
    while (span < n) span <<= 1;
    rank_sort_descending(sc.keys, n, span);
    // unique count = number of non-zero keys (a real key is never 0: ordered(logit) has a set bit)
    uint32_t mine = (t < span && sc.keys[t] != 0) ? 1u : 0u;
    const uint32_t unique = __syncthreads_count(mine);
    if (unique < request_top_k) return -6;
    uint32_t count = unique < request_top_k ? unique : request_top_k;
    // logits back from the sorted keys
    if (t < count) {
        const uint32_t o = static_cast<uint32_t>(sc.keys[t] >> 32);
        sc.logit[t] = __uint_as_float((o & 0x80000000u) ? (o & 0x7FFFFFFFu) : ~o);
        out.token[t] = 0xFFFFFFFFu - static_cast<uint32_t>(sc.keys[t]);
    }
    __syncthreads();
    if (opt.temperature == 0.f) {
        if (t == 0) { out.count = 1; out.total = 1.0; out.weight[0] = 1.0; }
        __syncthreads();
        return 0;
    }
    const float max_logit = sc.logit[0];
    if (t < count) sc.w[t] = exp(static_cast<double>(__fsub_rn(sc.logit[t], max_logit)));
    __syncthreads();
    if (t == 0) {
        double running = 0.0;
        for (uint32_t i = 0; i < count; ++i) { running += sc.w[i]; sc.run[i] = running; }
        sc.kept = count; sc.cut = count;
    }
    __syncthreads();
    {
        // top-p keeps entries up to and including the first whose running share reaches top_p; min-p then
        // keeps the leading entries (the first always) whose weight is at least min_p
        const double total = sc.run[count - 1];
        if (t + 1 < count && !(sc.run[t] / total < static_cast<double>(opt.top_p))) atomicMin(&sc.kept, t + 1);
        if (opt.min_p > 0.f && t >= 1 && t < count && !(sc.w[t] >= static_cast<double>(opt.min_p))) atomicMin(&sc.cut, t);
    }
    __syncthreads();
    count = sc.kept < sc.cut ? sc.kept : sc.cut;
    if (t < count)
        out.weight[t] = exp(static_cast<double>(__fsub_rn(sc.logit[t], max_logit)) / static_cast<double>(opt.temperature));
    __syncthreads();
    if (t == 0) {
        double norm = 0.0;
        for (uint32_t i = 0; i < count; ++i) norm += out.weight[i];
        out.count = count;
        out.total = norm;
        sc.err = (!isfinite(norm) || norm <= 0.0) ? -7 : 0;
    }
    __syncthreads();
    return sc.err;
}

// Neumaier-compensated total with the reference's consistency checks; all threads call it (the quotients
// are checked per lane, the compensated sum is one lane's), every thread gets the result: -1 when invalid.
__device__ double validated_total(const Prepared& p, Scratch& sc) {
    const uint32_t t = threadIdx.x;
    __syncthreads();
    const uint32_t count = p.count;
    const double stored = p.total;
    const bool shape_ok = !(count == 0 || count > kMaxTopK || !isfinite(stored) || stored <= 0.0);
    if (t == 0) sc.flag = 0;
    __syncthreads();
    if (shape_ok && t < count) {
        const double w = p.weight[t];
        const double prob = w / stored;  // the stored probability is exactly this quotient
        if (!isfinite(prob) || prob < 0.0 || prob > 1.0 || !isfinite(w) || w < 0.0) sc.flag = 1;
    }
    __syncthreads();
    if (t == 0) {
        double result = -1.0;
        if (shape_ok && !sc.flag) {
            double total = 0.0, correction = 0.0;
            for (uint32_t i = 0; i < count; ++i) {
                const double w = p.weight[i];
                const double sum = total + w;
                correction += total >= w ? (total - sum) + w : (w - sum) + total;
                total = sum;
            }
            total += correction;
            const double tol = static_cast<double>(count) * 2.220446049250313e-16 * total;
            if (isfinite(total) && total > 0.0 && !(fabs(total - stored) > tol)) result = total;
        }
        sc.value = result;
    }
    __syncthreads();
    return sc.value;
}

__device__ uint32_t select_prepared(const Prepared& p, double draw) {
    double cumulative = 0.0;
    for (uint32_t i = 0; i < p.count; ++i) {
        cumulative += p.weight[i];
        if (draw < cumulative) return p.token[i];
    }
    return p.token[p.count - 1];
}

// target_to_draft: null when both sides share one vocabulary; else the law lives in draft ids and a
// target token's mass is that of the draft token mapped to it, if any (Gemma3DraftPlan::gather,
// src/engine/gemma3_draft.mm:1570-1578)
// The compact law as the acceptance kernel keeps it in LDS (ids ascending, cdf[i] .. cdf[i + 1] the mass of ids[i]).
struct LawCopy { uint32_t count; uint32_t ids[256]; uint64_t cdf[257]; };

__device__ uint64_t law_mass(const LawCopy& law, const uint64_t* full_cdf, uint32_t vocab, uint32_t token,
                             uint64_t* begin, const int32_t* target_to_draft = nullptr) {
    if (target_to_draft) {
        const int32_t draft = target_to_draft[token];
        if (draft < 0) { if (begin) *begin = 0; return 0; }
        token = static_cast<uint32_t>(draft);
    }
    if (law.count == kLawFull) {  // gather from the full table (src/engine/gemma3_draft.mm:1544-1545)
        if (!full_cdf || token >= vocab) { if (begin) *begin = 0; return 0; }
        if (begin) *begin = full_cdf[token];
        return full_cdf[token + 1] - full_cdf[token];
    }
    const uint32_t count = law.count < 256u ? law.count : 256u;
    uint32_t lo = 0, hi = count;
    while (lo < hi) {
        const uint32_t mid = (lo + hi) >> 1;
        if (law.ids[mid] < token) lo = mid + 1; else hi = mid;
    }
    if (lo == count || law.ids[lo] != token) { if (begin) *begin = 0; return 0; }
    if (begin) *begin = law.cdf[lo];
    return law.cdf[lo + 1] - law.cdf[lo];
}

__global__ void __launch_bounds__(512)
spec_accept_kernel(const Candidates* __restrict__ rows, const DraftLaw* __restrict__ law,
                   const uint64_t* __restrict__ full_cdf, uint32_t vocab, const uint32_t* __restrict__ history,
                   const uint32_t* __restrict__ history_count, const uint32_t* __restrict__ proposal_ptr, SamplerOptions opt, uint64_t seed, uint64_t step,
                   const StepDraws* __restrict__ injected, SpecResult* __restrict__ result,
                   uint32_t* __restrict__ status, const int32_t* __restrict__ target_to_draft) {
    __shared__ Scratch sc;
    __shared__ Prepared target, residual;
    __shared__ uint64_t q[kMaxTopK];
    __shared__ double diff[kMaxTopK];
    __shared__ double s_proposed, s_acceptance;
    __shared__ int s_code;
    __shared__ uint32_t s_accepted, s_draw_residual;
    __shared__ LawCopy q_law;
    const uint32_t t = threadIdx.x;
    const uint32_t proposal = *proposal_ptr;
    const StepDraws d = injected ? *injected : step_draws(seed, step);
    // the compact law comes in once, every word by its own lane (the record is always whole in memory):
    // the gathers below search it in LDS instead of through a chain of dependent trips to memory
    if (t < 256) { q_law.ids[t] = law->ids[t]; q_law.cdf[t] = law->cdf[t]; }
    if (t == 256) { q_law.cdf[256] = law->cdf[256]; q_law.count = law->count; }
    if (t == 0) {
        result->accepted = 0; result->token = 0xFFFFFFFFu; result->next_root = 0xFFFFFFFFu; result->status = 0;
        result->acceptance_probability = 0.0; result->residual_total = 0.0; result->residual_count = 0;
        result->proposal = proposal;
    }
    // history: [2][64] token ids and their counts per row (null: no repetition history)
    int rc = prepare_distribution(&rows[0], opt, history, history ? history_count[0] : 0u, sc, target);
    if (!rc && t < target.count) q[t] = law_mass(q_law, full_cdf, vocab, target.token[t], nullptr, target_to_draft);
    const double normalization = rc ? -1.0 : validated_total(target, sc);
    __syncthreads();
    if (t == 0) {
        int code = rc;
        auto unit = [](double u) { return isfinite(u) && u >= 0.0 && u < 1.0; };
        if (!code && (!unit(d.u_accept) || !unit(d.u_residual) || !unit(d.u_next))) code = -20;
        if (!code && normalization < 0.0) code = -21;
        uint64_t begin = 0, proposal_mass = 0;
        if (!code) {
            proposal_mass = law_mass(q_law, full_cdf, vocab, proposal, &begin, target_to_draft);
            if (proposal_mass == 0 || proposal_mass > kMassTotal || begin > kMassTotal - proposal_mass) code = -22;
        }
        bool in_target = false;
        if (!code) {
            uint64_t gathered = 0;
            for (uint32_t i = 0; i < target.count && !code; ++i) {
                if (q[i] > kMassTotal - gathered) code = -23;
                gathered += q[i];
                if (target.token[i] == proposal) in_target = true;
            }
            if (!code && !in_target && proposal_mass > kMassTotal - gathered) code = -24;
        }
        s_code = code;
        s_accepted = 0;
        s_draw_residual = 0;
        s_acceptance = 0.0;
        s_proposed = static_cast<double>(proposal_mass) / static_cast<double>(kMassTotal);
    }
    __syncthreads();
    if (s_code == 0) {
        // p, p / q of the proposal and p - q per lane; the residual's order and sum stay one lane's
        if (t < target.count) {
            const double p = target.weight[t] / normalization;
            if (target.token[t] == proposal) s_acceptance = fmin(1.0, p / s_proposed);   // tokens are distinct
            diff[t] = p - static_cast<double>(q[t]) / static_cast<double>(kMassTotal);
        }
        __syncthreads();
        if (t == 0) {
            int code = 0;
            const double acceptance = s_acceptance;
            residual.count = 0; residual.total = 0.0;
            for (uint32_t i = 0; i < target.count; ++i) {
                const double excess = diff[i];
                if (excess <= 0.0) continue;
                residual.token[residual.count] = target.token[i];
                residual.weight[residual.count] = excess;
                ++residual.count;
                residual.total += excess;
            }
            if (residual.count == 0 && acceptance < 1.0) code = -25;
            result->acceptance_probability = acceptance;
            result->residual_total = residual.total;
            result->residual_count = residual.count;
            if (!code) {
                if (d.u_accept < acceptance) {
                    s_accepted = 1;
                    result->accepted = 1; result->token = proposal; result->next_root = proposal;
                } else {
                    s_draw_residual = 1;
                }
            }
            s_code = code;
        }
        __syncthreads();
        if (s_draw_residual) {
            const double residual_total = validated_total(residual, sc);
            if (t == 0) {
                if (residual_total < 0.0) {
                    s_code = -26;
                } else {
                    const uint32_t tok = select_prepared(residual, d.u_residual * residual.total);
                    result->token = tok; result->next_root = tok;
                }
            }
            __syncthreads();
        }
    }
    if (s_code == 0 && s_accepted) {
        // a fully accepted chain leaves row 1's candidates to seed the next root
        rc = prepare_distribution(&rows[1], opt, history ? history + 64 : nullptr, history ? history_count[1] : 0u, sc, target);
        if (t == 0) {
            if (rc) s_code = rc - 100;
            else result->next_root = opt.temperature == 0.f ? target.token[0]
                                                             : select_prepared(target, d.u_next * target.total);
        }
    }
    __syncthreads();
    if (t == 0 && s_code != 0) {
        result->status = static_cast<uint32_t>(-s_code);
        result->token = 0xFFFFFFFFu; result->next_root = 0xFFFFFFFFu; result->accepted = 0;
        if (status) atomicOr(status, GUFFIN_STATUS_LAW_INVALID);
    }
}

}  // namespace

int select_candidates_scaled(hipStream_t s, const float* logits, uint32_t rows, uint32_t vocab, uint32_t retain,
                             float divisor, const uint32_t* history, const uint32_t* history_count,
                             void* workspace, void* result, uint32_t* status, bool suppressed_ok = false,
                             const uint32_t* row_retain = nullptr, uint32_t row_stride = 1);

}  // namespace guffin

using namespace guffin;

extern "C" uint64_t guffin_hip_draft_law_workspace_bytes(uint32_t vocab) {
    // workspace of the 257-best selection plus the sorted candidate row
    return ((guffin_hip_select_workspace_bytes(1, vocab, 257) + 15) & ~uint64_t{15}) + sizeof(Candidates) + 16;
}

namespace {

uint32_t padded_vocab(uint32_t vocab) {
    uint32_t p = kSortTile;
    while (p < vocab) p <<= 1;
    return p;
}
uint64_t align16(uint64_t v) { return (v + 15) & ~uint64_t{15}; }
uint64_t compact_ws_bytes(uint32_t vocab) { return align16(guffin_hip_draft_law_workspace_bytes(vocab)); }

FullLawWs carve_full_ws(uint8_t* base, uint32_t vocab) {
    const uint64_t padded = padded_vocab(vocab), tiles = vocab / kLawTile;
    FullLawWs ws;
    uint64_t at = 0;
    auto take = [&](uint64_t bytes) { uint8_t* p = base ? base + at : nullptr; at += align16(bytes); return p; };
    ws.keys_a = reinterpret_cast<uint64_t*>(take(padded * 8));
    ws.keys_b = reinterpret_cast<uint64_t*>(take(padded * 8));
    ws.scores = reinterpret_cast<float*>(take(uint64_t(vocab) * 4));
    ws.prefix = reinterpret_cast<float*>(take(uint64_t(vocab) * 4));
    ws.offsets = reinterpret_cast<float*>(take((tiles + 1) * 4));
    ws.best = reinterpret_cast<float*>(take(8));
    ws.error = reinterpret_cast<uint32_t*>(take(4));
    return ws;
}
uint64_t full_ws_bytes(uint32_t vocab) {
    const uint64_t padded = padded_vocab(vocab), tiles = vocab / kLawTile;
    return align16(padded * 8) * 2 + align16(uint64_t(vocab) * 4) * 2 + align16((tiles + 1) * 4) + 16 + 16;
}
bool compact_options(const SamplerOptions& o) { return o.temperature > 0.f && o.top_k >= 1 && o.top_k <= 64; }

int launch_compact_law(hipStream_t s, const float* logits, uint32_t vocab, const SamplerOptions& opt, uint64_t seed,
                       uint64_t step, const void* injected_draws, void* workspace, void* law, uint32_t* proposal,
                       uint32_t* status, uint32_t* full_error, bool suppressed_ok = false) {
    uint8_t* ws = static_cast<uint8_t*>(workspace);
    Candidates* top = reinterpret_cast<Candidates*>(ws + ((guffin_hip_select_workspace_bytes(1, vocab, 257) + 15) & ~uint64_t{15}));
    // the k-th best score and every tie with it: the best 257 scores decide both
    if (int rc = select_candidates_scaled(s, logits, 1, vocab, vocab < 257 ? vocab : 257, opt.temperature, nullptr,
                                          nullptr, ws, top, status, suppressed_ok))
        return rc;
    launch(draft_law_kernel, dim3(1), dim3(256), 0, s, top, opt, seed, step,
                       static_cast<const StepDraws*>(injected_draws), static_cast<DraftLaw*>(law), proposal, status,
                       full_error);
    return check_launch("draft_law");
}

// the full-vocabulary kernels in the reference's dispatch order (src/engine/gemma3_draft.mm:1040-1166)
int launch_full_law(hipStream_t s, const float* logits, uint32_t vocab, const SamplerOptions& opt, uint64_t seed,
                    uint64_t step, const void* injected_draws, const uint32_t* guard, const FullLawWs& ws,
                    uint64_t* cdf, uint32_t* proposal, uint32_t* status, bool suppressed_ok = false) {
    const bool greedy = opt.temperature == 0.f;
    const uint32_t padded = padded_vocab(vocab);
    launch(law_sort_tile_kernel, dim3(padded / kSortTile), dim3(1024), 0, s, logits, vocab, opt.temperature,
                       !greedy, suppressed_ok, guard, ws, status);
    if (!greedy) {
        const uint64_t* sorted = ws.keys_a;
        uint64_t* other = ws.keys_b;
        for (uint32_t width = kSortTile; width < padded; width <<= 1) {
            launch(law_merge_kernel, dim3(padded / 256), dim3(256), 0, s, sorted, other, width, padded, guard);
            const uint64_t* done = other;
            other = const_cast<uint64_t*>(sorted);
            sorted = done;
        }
        launch(law_filter_prefix_kernel, dim3(1), dim3(1024), 0, s, sorted, vocab, opt.top_k, guard, ws);
        launch(law_filter_apply_kernel, dim3((vocab + 255) / 256), dim3(256), 0, s, sorted, vocab, opt, guard, ws);
    }
    launch(law_weights_kernel, dim3(1), dim3(1024), 0, s, vocab, greedy, guard, ws, status);
    launch(law_cdf_select_kernel, dim3(vocab / 256 + 1), dim3(256), 0, s, vocab, greedy, seed, step,
                       static_cast<const StepDraws*>(injected_draws), guard, ws, cdf, proposal, status);
    return check_launch("draft_law_full");
}

}  // namespace

extern "C" int guffin_hip_draft_law(void* stream, const float* logits, uint32_t vocab, const void* options,
                                    uint64_t seed, uint64_t step, const void* injected_draws, void* workspace,
                                    void* law, uint32_t* proposal, uint32_t* status) {
    if (!logits || !options || !workspace || !law || !proposal || !status) return fail(GUFFIN_E_ARG, "draft_law: null pointer");
    if (vocab < 1) return fail(GUFFIN_E_SHAPE, "draft_law: empty vocabulary");
    if (reinterpret_cast<uintptr_t>(workspace) & 7u) return fail(GUFFIN_E_ALIGN, "draft_law: workspace must be 8-byte aligned");
    const SamplerOptions opt = *static_cast<const SamplerOptions*>(options);
    if (!compact_options(opt))
        return fail(GUFFIN_E_ARG, "draft_law: the compact law needs temperature > 0 and top_k in [1, 64]");
    return launch_compact_law(as_stream(stream), logits, vocab, opt, seed, step, injected_draws, workspace, law,
                              proposal, status, nullptr);
}

namespace guffin {
namespace {
// scores[i] = logits[i], divided by the penalty (multiplied when negative) for the tokens of the
// sampler history, and -inf for a draft token that the vocabulary map gives no target token: the
// drafter's gd_process without its division by the temperature, which follows in the selection
// (src/engine/gemma3_draft.mm:191-204).  With a map the raw logits are validated here, the
// suppressed ones included.
__global__ void __launch_bounds__(256)
draft_process_kernel(const float* __restrict__ logits, uint32_t vocab, const uint32_t* __restrict__ history,
                     uint32_t count, float penalty, const int32_t* __restrict__ draft_to_target,
                     float* __restrict__ scores, uint32_t* __restrict__ status) {
    __shared__ uint32_t seen[kHistoryCap];
    if (threadIdx.x < count) seen[threadIdx.x] = history[threadIdx.x];
    __syncthreads();
    bool bad = false;
    for (uint32_t i = blockIdx.x * blockDim.x + threadIdx.x; i < vocab; i += gridDim.x * blockDim.x) {
        float v = logits[i];
        bad |= !isfinite(v);
        bool hit = false;
        for (uint32_t j = 0; j < count; ++j) hit |= seen[j] == i;
        if (hit && penalty != 1.0f) v = v < 0.f ? v * penalty : v / penalty;
        if (draft_to_target && draft_to_target[i] < 0) v = -INFINITY;
        scores[i] = v;
    }
    if (bad && draft_to_target && status) atomicOr(status, GUFFIN_STATUS_NONFINITE);
}

// proposal in draft ids -> the target's id for it
__global__ void map_proposal_kernel(const int32_t* __restrict__ draft_to_target, uint32_t vocab,
                                    const uint32_t* __restrict__ draft_proposal, uint32_t* __restrict__ target_proposal) {
    const uint32_t d = *draft_proposal;
    *target_proposal = d < vocab && draft_to_target[d] >= 0 ? static_cast<uint32_t>(draft_to_target[d]) : 0xFFFFFFFFu;
}
}  // namespace
}  // namespace guffin

extern "C" int guffin_hip_draft_process(void* stream, const float* logits, uint32_t vocab, const uint32_t* history,
                                        uint32_t history_count, float repetition_penalty, float* scores) {
    if (!logits || !scores || (history_count && !history)) return fail(GUFFIN_E_ARG, "draft_process: null pointer");
    if (vocab == 0) return fail(GUFFIN_E_SHAPE, "draft_process: empty vocabulary");
    if (history_count > kHistoryCap) return fail(GUFFIN_E_CAPACITY, "draft_process: at most 64 history tokens");
    if (!std::isfinite(repetition_penalty) || !(repetition_penalty > 0.f)) return fail(GUFFIN_E_ARG, "draft_process: the penalty must be positive");
    const uint32_t blocks = std::min<uint32_t>((vocab + 255) / 256, 1024);
    launch(draft_process_kernel, dim3(blocks), dim3(256), 0, as_stream(stream), logits, vocab, history,
                       history_count, repetition_penalty, static_cast<const int32_t*>(nullptr), scores,
                       static_cast<uint32_t*>(nullptr));
    return check_launch("draft_process");
}

extern "C" int guffin_hip_draft_law_mapped(void* stream, const float* logits, uint32_t vocab, const int32_t* draft_to_target,
                                           const uint32_t* history, uint32_t history_count, const void* options,
                                           uint64_t seed, uint64_t step, const void* injected_draws, void* workspace,
                                           float* scores, void* law, uint32_t* draft_proposal, uint32_t* target_proposal,
                                           uint32_t* status) {
    if (!logits || !draft_to_target || !options || !workspace || !scores || !law || !draft_proposal || !target_proposal || !status
        || (history_count && !history))
        return fail(GUFFIN_E_ARG, "draft_law_mapped: null pointer");
    if (vocab == 0) return fail(GUFFIN_E_SHAPE, "draft_law_mapped: empty vocabulary");
    if (history_count > kHistoryCap) return fail(GUFFIN_E_CAPACITY, "draft_law_mapped: at most 64 history tokens");
    if (reinterpret_cast<uintptr_t>(workspace) & 15u) return fail(GUFFIN_E_ALIGN, "draft_law_mapped: workspace must be 16-byte aligned");
    const SamplerOptions opt = *static_cast<const SamplerOptions*>(options);
    if (!compact_options(opt))
        return fail(GUFFIN_E_ARG, "draft_law_mapped: the compact law needs temperature > 0 and top_k in [1, 64]");
    if (!std::isfinite(opt.repetition_penalty) || !(opt.repetition_penalty > 0.f)) return fail(GUFFIN_E_ARG, "draft_law_mapped: the penalty must be positive");
    hipStream_t s = as_stream(stream);
    const uint32_t blocks = std::min<uint32_t>((vocab + 255) / 256, 1024);
    launch(draft_process_kernel, dim3(blocks), dim3(256), 0, s, logits, vocab, history, history_count,
                       opt.repetition_penalty, draft_to_target, scores, status);
    if (int rc = check_launch("draft_process")) return rc;
    if (int rc = launch_compact_law(s, scores, vocab, opt, seed, step, injected_draws, workspace, law, draft_proposal, status,
                                    nullptr, true))
        return rc;
    launch(map_proposal_kernel, dim3(1), dim3(1), 0, s, draft_to_target, vocab, draft_proposal, target_proposal);
    return check_launch("map_proposal");
}

extern "C" uint64_t guffin_hip_draft_law_any_workspace_bytes(uint32_t vocab) {
    return compact_ws_bytes(vocab) + full_ws_bytes(vocab);
}

namespace {
int draft_law_any(void* stream, const float* logits, uint32_t vocab, const void* options, uint64_t seed, uint64_t step,
                  const void* injected_draws, void* workspace, void* law, uint64_t* full_cdf, uint32_t* proposal,
                  uint32_t* status, bool suppressed_ok) {
    if (!logits || !options || !workspace || !law || !full_cdf || !proposal || !status)
        return fail(GUFFIN_E_ARG, "draft_law_any: null pointer");
    if (vocab < kLawTile || vocab % kLawTile != 0)
        return fail(GUFFIN_E_SHAPE, "draft_law_any: the vocabulary must be a positive multiple of 256");
    if (reinterpret_cast<uintptr_t>(workspace) & 15u) return fail(GUFFIN_E_ALIGN, "draft_law_any: workspace must be 16-byte aligned");
    if (reinterpret_cast<uintptr_t>(full_cdf) & 7u) return fail(GUFFIN_E_ALIGN, "draft_law_any: the table must be 8-byte aligned");
    const SamplerOptions opt = *static_cast<const SamplerOptions*>(options);
    if (!std::isfinite(opt.temperature) || opt.temperature < 0.f || opt.top_k < 1 || opt.top_k > kMaxTopK
        || !(opt.top_p > 0.f) || opt.top_p > 1.f || !(opt.min_p >= 0.f) || opt.min_p > 1.f)
        return fail(GUFFIN_E_ARG, "draft_law_any: sampler options out of range");
    hipStream_t s = as_stream(stream);
    uint8_t* base = static_cast<uint8_t*>(workspace);
    const FullLawWs ws = carve_full_ws(base + compact_ws_bytes(vocab), vocab);
    DraftLaw* slot = static_cast<DraftLaw*>(law);
    if (compact_options(opt)) {
        // the compact law; its kernel hands over to the guarded full-vocabulary kernels when more
        // than 256 tokens tie into the support
        if (int rc = launch_compact_law(s, logits, vocab, opt, seed, step, injected_draws, base, law, proposal, status, ws.error, suppressed_ok))
            return rc;
        return launch_full_law(s, logits, vocab, opt, seed, step, injected_draws, &slot->count, ws, full_cdf, proposal, status, suppressed_ok);
    }
    launch(law_begin_kernel, dim3(1), dim3(1), 0, s, slot, proposal, ws.error);
    return launch_full_law(s, logits, vocab, opt, seed, step, injected_draws, nullptr, ws, full_cdf, proposal, status, suppressed_ok);
}
}  // namespace


extern "C" int guffin_hip_draft_law_any(void* stream, const float* logits, uint32_t vocab, const void* options,
                                        uint64_t seed, uint64_t step, const void* injected_draws, void* workspace,
                                        void* law, uint64_t* full_cdf, uint32_t* proposal, uint32_t* status) {
    return draft_law_any(stream, logits, vocab, options, seed, step, injected_draws, workspace, law, full_cdf, proposal, status, false);
}

extern "C" int guffin_hip_draft_law_any_mapped(void* stream, const float* logits, uint32_t vocab, const int32_t* draft_to_target,
                                               const uint32_t* history, uint32_t history_count, const void* options,
                                               uint64_t seed, uint64_t step, const void* injected_draws, void* workspace,
                                               float* scores, void* law, uint64_t* full_cdf, uint32_t* draft_proposal,
                                               uint32_t* target_proposal, uint32_t* status) {
    if (!logits || !draft_to_target || !options || !scores || !draft_proposal || !target_proposal || !status || (history_count && !history))
        return fail(GUFFIN_E_ARG, "draft_law_any_mapped: null pointer");
    if (vocab == 0) return fail(GUFFIN_E_SHAPE, "draft_law_any_mapped: empty vocabulary");
    if (history_count > kHistoryCap) return fail(GUFFIN_E_CAPACITY, "draft_law_any_mapped: at most 64 history tokens");
    const SamplerOptions opt = *static_cast<const SamplerOptions*>(options);
    if (!std::isfinite(opt.repetition_penalty) || !(opt.repetition_penalty > 0.f)) return fail(GUFFIN_E_ARG, "draft_law_any_mapped: the penalty must be positive");
    hipStream_t s = as_stream(stream);
    const uint32_t blocks = std::min<uint32_t>((vocab + 255) / 256, 1024);
    launch(draft_process_kernel, dim3(blocks), dim3(256), 0, s, logits, vocab, history, history_count,
                       opt.repetition_penalty, draft_to_target, scores, status);
    if (int rc = check_launch("draft_process")) return rc;
    if (int rc = draft_law_any(stream, scores, vocab, options, seed, step, injected_draws, workspace, law, full_cdf, draft_proposal,
                               status, true))
        return rc;
    launch(map_proposal_kernel, dim3(1), dim3(1), 0, s, draft_to_target, vocab, draft_proposal, target_proposal);
    return check_launch("map_proposal");
}

extern "C" int guffin_hip_spec_accept_mapped(void* stream, const void* target_candidates, const void* law,
                                             const uint64_t* full_cdf, uint32_t vocab, const int32_t* target_to_draft,
                                             const uint32_t* history, const uint32_t* history_count,
                                             const uint32_t* proposal, const void* options, uint64_t seed, uint64_t step,
                                             const void* injected_draws, void* result, uint32_t* status) {
    if (!target_candidates || !law || !proposal || !options || !result) return fail(GUFFIN_E_ARG, "spec_accept: null pointer");
    if ((history == nullptr) != (history_count == nullptr)) return fail(GUFFIN_E_ARG, "spec_accept: history needs its counts");
    const SamplerOptions opt = *static_cast<const SamplerOptions*>(options);
    launch(spec_accept_kernel, dim3(1), dim3(512), 0, as_stream(stream),
                       static_cast<const Candidates*>(target_candidates), static_cast<const DraftLaw*>(law), full_cdf,
                       vocab, history, history_count, proposal, opt, seed, step,
                       static_cast<const StepDraws*>(injected_draws), static_cast<SpecResult*>(result), status,
                       target_to_draft);
    return check_launch("spec_accept");
}

extern "C" int guffin_hip_spec_accept_history(void* stream, const void* target_candidates, const void* law,
                                              const uint64_t* full_cdf, uint32_t vocab, const uint32_t* history,
                                              const uint32_t* history_count, const uint32_t* proposal,
                                              const void* options, uint64_t seed, uint64_t step,
                                              const void* injected_draws, void* result, uint32_t* status) {
    return guffin_hip_spec_accept_mapped(stream, target_candidates, law, full_cdf, vocab, nullptr, history, history_count,
                                         proposal, options, seed, step, injected_draws, result, status);
}

extern "C" int guffin_hip_spec_accept_law(void* stream, const void* target_candidates, const void* law,
                                          const uint64_t* full_cdf, uint32_t vocab, const uint32_t* proposal,
                                          const void* options, uint64_t seed, uint64_t step,
                                          const void* injected_draws, void* result, uint32_t* status) {
    return guffin_hip_spec_accept_history(stream, target_candidates, law, full_cdf, vocab, nullptr, nullptr, proposal,
                                          options, seed, step, injected_draws, result, status);
}

extern "C" int guffin_hip_spec_accept(void* stream, const void* target_candidates, const void* law,
                                      const uint32_t* proposal, const void* options, uint64_t seed, uint64_t step,
                                      const void* injected_draws, void* result, uint32_t* status) {
    return guffin_hip_spec_accept_law(stream, target_candidates, law, nullptr, 0, proposal, options, seed, step,
                                      injected_draws, result, status);
}

extern "C" int guffin_hip_step_draws(uint64_t seed, uint64_t step, void* out_draws_host) {
    // host restatement of the device draw schedule, for callers that log or inject draws
    if (!out_draws_host) return fail(GUFFIN_E_ARG, "step_draws: null pointer");
    auto round = [](uint32_t (&c)[4], uint32_t (&k)[2]) {
        const uint64_t p0 = uint64_t{0xD2511F53u} * c[0], p1 = uint64_t{0xCD9E8D57u} * c[2];
        const uint32_t n0 = static_cast<uint32_t>(p1 >> 32) ^ c[1] ^ k[0], n1 = static_cast<uint32_t>(p1);
        const uint32_t n2 = static_cast<uint32_t>(p0 >> 32) ^ c[3] ^ k[1], n3 = static_cast<uint32_t>(p0);
        c[0] = n0; c[1] = n1; c[2] = n2; c[3] = n3;
        k[0] += 0x9E3779B9u; k[1] += 0xBB67AE85u;
    };
    StepDraws d {};
    uint32_t out[2][4];
    for (uint32_t block = 0; block < 2; ++block) {
        uint32_t c[4] = {static_cast<uint32_t>(step), static_cast<uint32_t>(step >> 32), block, 0};
        uint32_t k[2] = {static_cast<uint32_t>(seed), static_cast<uint32_t>(seed >> 32)};
        for (int r = 0; r < 10; ++r) round(c, k);
        for (int i = 0; i < 4; ++i) out[block][i] = c[i];
    }
    auto unit = [](uint32_t hi, uint32_t lo) { return static_cast<double>(((uint64_t{hi} << 32) | lo) >> 11) * 0x1.0p-53; };
    d.word = out[0][0];
    d.u_accept = unit(out[0][1], out[0][2]);
    d.u_residual = unit(out[1][0], out[1][1]);
    d.u_next = unit(out[1][2], out[1][3]);
    *static_cast<StepDraws*>(out_draws_host) = d;
    return GUFFIN_OK;
}
