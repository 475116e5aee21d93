// Resolving one verify row's raw sampler history on the device, one wave per row.
//
// The row names a ring of `limit` slots with the oldest token at `head`, and a suffix of tokens that
// would have been observed before this row is sampled.  What the selection needs is the window after
// appending the suffix (a full window drops its oldest token per append), without later duplicates,
// and its length: top_k + length logits are retained so that a penalised token that falls out of the
// top_k still leaves top_k candidates.  Same outputs as verifier_selection_request_resolve_kernel
// (src/tensor/backends/metal/metal_kernels.mm:2336-2404) and, on the host,
// make_token_selection_request (src/engine/sampling.cpp:352-392).
#pragma once
#include <hip/hip_runtime.h>

#include <cstdint>

namespace guffin {

constexpr uint32_t kRequestHistory = 64;   // token_sampler_max_repetition_window
constexpr uint32_t kRequestSuffix = 23;    // external_speculation_max_horizon
constexpr uint32_t kRequestMalformed = 2u, kRequestBadToken = 4u;  // the reference's status bits

struct SelectionRow {   // VerifierDeviceSelectionRow, 364 bytes
    uint32_t history_token_ids[kRequestHistory];
    uint32_t suffix_token_ids[kRequestSuffix];
    uint32_t history_head, history_length, history_window_limit, suffix_count;
};
struct ResolvedRow {    // VerifierResolvedSelectionRow, 272 bytes
    uint32_t top_k, base_candidate_count, history_count, reserved;
    uint32_t history_token_ids[kRequestHistory];
};
static_assert(sizeof(SelectionRow) == 364 && sizeof(ResolvedRow) == 272, "the reference's layouts");

// Every wave of the workgroup calls this (it meets a workgroup barrier), each with its own row, and all
// 64 lanes of a wave with the same arguments.  Lane l gets the l-th token of the
// deduplicated window in `token` (0 past the end); returns the window's length and ORs the status bits
// of the row into `status` (the same value on every lane).
__device__ inline uint32_t resolve_history(const uint32_t* ring, uint32_t head, uint32_t length, uint32_t limit,
                                           const uint32_t* suffix, uint32_t suffix_count, uint32_t vocab,
                                           bool repetition, uint32_t lane, uint32_t& token, uint32_t& status) {
    token = 0;
    if (limit > kRequestHistory || length > limit || suffix_count > kRequestSuffix || (length == 0 && head != 0)
        || (length > 0 && head >= limit)) {
        status |= kRequestMalformed;
        return 0;
    }
    // every token the row names is checked, also those the appends push out of the window
    bool bad = lane < length && ring[(head + lane) % limit] >= vocab;
    bad |= lane < suffix_count && suffix[lane] >= vocab;
    if (__ballot(bad)) status |= kRequestBadToken;
    // the window after the appends = the last min(total, limit) tokens of history followed by suffix
    const uint32_t total = length + (limit ? suffix_count : 0u);
    const uint32_t n = total < limit ? total : limit;
    uint32_t mine = 0;
    if (lane < n) {
        const uint32_t at = total - n + lane;
        mine = at < length ? ring[(head + at) % limit] : suffix[at - length];
    }
    const bool live = repetition && lane < n && mine < vocab;
    bool later = false;   // an earlier lane holds the same token
    for (uint32_t other = 0; other < n; ++other) {
        const uint32_t theirs = __shfl(mine, other, 64);
        const bool theirs_live = __shfl(live ? 1 : 0, other, 64) != 0;
        later |= other < lane && theirs_live && theirs == mine;
    }
    const uint64_t keep = __ballot(live && !later);
    const uint32_t count = __popcll(keep);
    // compact: lane l takes the token of the l-th kept lane
    const uint32_t slot = __popcll(keep & ((uint64_t(1) << lane) - 1));
    __shared__ uint32_t compact[16][kRequestHistory];   // one line per wave of the workgroup
    uint32_t* line = compact[(threadIdx.x >> 6) & 15];
    if (live && !later) line[slot] = mine;
    __syncthreads();
    token = lane < count ? line[lane] : 0u;
    return count;
}

}  // namespace guffin
