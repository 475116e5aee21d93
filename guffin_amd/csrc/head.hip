// Output-head selection over the 262144-entry logits rows (gfx950).
//
// Replaces encode_token_candidates / encode_target_token_candidates and their tile-sort,
// merge-tree and finalize kernels (src/tensor/backends/metal/metal_command_context.hpp:326-345,
// src/tensor/backends/metal/metal_kernels.mm:3444-3884), and the CPU argmax
// (src/tensor/ops/reduction.cpp:93-117).  Order everywhere: higher logit first, then lower
// token id (src/engine/sampling.cpp:25-30, metal_kernels.mm:171-173).
//
// An entry is one 64-bit key {ordered(logit) : 32 | ~token : 32}; descending key order is the
// candidate order and keys are unique, so selection is a pure comparison network and the
// result is exact including ties.
//   stage 1  every workgroup sorts a 2048-logit tile in LDS (bitonic) and keeps its best R
//   stage 2  one workgroup per row picks the best `retain` of the G*R survivors (a threshold from
//            the sorted tile lists' heads plus a rank sort; a radix select where that does not
//            apply), then appends the logits of the history tokens
// A global top-R entry is necessarily a top-R entry of its own tile, so the two stages lose
// nothing.
#include "common.hpp"
#include "selection_request.hpp"

#include <cstddef>

namespace guffin {
namespace {

constexpr uint32_t kTile = 2048;          // logits per stage-1 workgroup

__device__ __forceinline__ uint64_t make_key(float logit, uint32_t token) {
    const uint32_t b = __float_as_uint(logit + 0.0f);  // -0 orders as +0, as a float comparison does
    const uint32_t ordered = (b & 0x80000000u) ? ~b : (b | 0x80000000u);
    return (uint64_t(ordered) << 32) | (0xFFFFFFFFu - token);
}
[[maybe_unused]] __device__ __forceinline__ float key_logit(uint64_t key) {
    const uint32_t o = static_cast<uint32_t>(key >> 32);
    return __uint_as_float((o & 0x80000000u) ? (o & 0x7FFFFFFFu) : ~o);
}
__device__ __forceinline__ uint32_t key_token(uint64_t key) { return 0xFFFFFFFFu - static_cast<uint32_t>(key); }

// descending bitonic sort of n (power of two) keys in LDS by all threads of the workgroup
__device__ __forceinline__ void bitonic_desc(uint64_t* keys, uint32_t n) {
    for (uint32_t width = 2; width <= n; width <<= 1) {
        for (uint32_t stride = width >> 1; stride > 0; stride >>= 1) {
            __syncthreads();
            for (uint32_t i = threadIdx.x; i < n / 2; i += blockDim.x) {
                const uint32_t lo = 2 * i - (i & (stride - 1));   // index with the `stride` bit clear
                const uint32_t hi = lo + stride;
                const bool descending = (lo & width) == 0;
                const uint64_t a = keys[lo], b = keys[hi];
                if ((a < b) == descending) { keys[lo] = b; keys[hi] = a; }
            }
        }
    }
    __syncthreads();
}

__global__ void __launch_bounds__(1024)
topk_tile_kernel(const float* __restrict__ logits, uint64_t* __restrict__ survivors, uint32_t vocab,
                 uint32_t keep, float divisor, uint32_t* __restrict__ status, bool suppressed_ok) {
    __shared__ uint64_t keys[kTile];
    const uint32_t tile = blockIdx.x, row = blockIdx.y;
    const float* lr = logits + size_t(row) * vocab;
    bool bad = false;
    for (uint32_t i = threadIdx.x; i < kTile; i += blockDim.x) {
        const uint32_t t = tile * kTile + i;
        uint64_t k = 0;  // below every real key
        if (t < vocab) {
            const float v = lr[t] / divisor;  // IEEE division: the drafter's score = logit / T
            // -inf marks a score that its producer suppressed (a draft token without a target token)
            bad |= (!isfinite(v) || !isfinite(lr[t])) && !(suppressed_ok && lr[t] == -INFINITY);
            k = make_key(v, t);
        }
        keys[i] = k;
    }
    if (bad && status) atomicOr(status + row, GUFFIN_STATUS_NONFINITE);
    bitonic_desc(keys, kTile);
    uint64_t* out = survivors + (size_t(row) * gridDim.x + tile) * keep;
    for (uint32_t i = threadIdx.x; i < keep; i += blockDim.x) out[i] = keys[i];
}

struct Candidates {  // layout of one row of the result (sampling.hpp:57-61 plus a status word)
    uint32_t count;
    uint32_t status;
    struct { uint32_t token; float logit; } values[384];
};

// Adds one to hist[bin] for every lane with `valid`; lanes of a wave that hit the same bin are
// counted with one atomic (keys cluster in a few bins, and same-address LDS atomics serialise).
__device__ __forceinline__ void hist_add(uint32_t* hist, bool valid, uint32_t bin, uint32_t lane) {
    uint64_t todo = __ballot(valid);
    for (int it = 0; it < 8 && todo; ++it) {
        const int leader = __ffsll(static_cast<long long>(todo)) - 1;
        const uint32_t b0 = __shfl(bin, leader, kWave);
        const uint64_t same = __ballot(valid && bin == b0) & todo;
        if (lane == uint32_t(leader)) atomicAdd(&hist[b0], static_cast<uint32_t>(__popcll(same)));
        todo &= ~same;
    }
    if ((todo >> lane) & 1u) atomicAdd(&hist[bin], 1u);
}

// Writes one row of the result from its `retain` selected keys (candidate order) and appends the logits of
// the row's history tokens; all threads of the workgroup call it after the keys are complete.
__device__ void emit_candidates(const uint64_t* keys, uint32_t retain, uint32_t row, const float* __restrict__ logits,
                                uint32_t vocab, float divisor, const uint32_t* __restrict__ history,
                                const uint32_t* __restrict__ history_count, uint32_t row_stride, uint32_t history_stride,
                                Candidates* __restrict__ result, uint32_t* __restrict__ status) {
    __syncthreads();
    Candidates& out = result[row];
    const uint32_t hc = history_count ? history_count[size_t(row) * row_stride] : 0;
    for (uint32_t i = threadIdx.x; i < retain; i += blockDim.x) {
        const uint32_t token = key_token(keys[i]);
        out.values[i].token = token;
        out.values[i].logit = logits[size_t(row) * vocab + token] / divisor;  // the native value, not the key's
    }
    uint32_t st = 0;
    for (uint32_t i = threadIdx.x; i < hc; i += blockDim.x) {
        const uint32_t token = history[size_t(row) * history_stride + i];
        if (token >= vocab) {
            st |= GUFFIN_STATUS_BAD_TOKEN;
            out.values[retain + i].token = 0xFFFFFFFFu;
            out.values[retain + i].logit = -INFINITY;
        } else {
            const float v = logits[size_t(row) * vocab + token] / divisor;
            if (!isfinite(v)) st |= GUFFIN_STATUS_NONFINITE;
            out.values[retain + i].token = token;
            out.values[retain + i].logit = v;
        }
    }
    if (st && status) atomicOr(status + row, st);
    __syncthreads();
    if (threadIdx.x == 0) {
        out.count = retain + hc;
        out.status = status ? status[row] : 0;
    }
}

// Stage 2: exact selection of the best `retain` of n unique keys.  Sorted tile lists take the
// threshold shortcut below; otherwise an 8-pass radix select (one byte per pass, most significant
// first: a 256-bin histogram in LDS, then the bin that holds the retain-th largest key).  Either
// way a rank sort of the selected keys follows.
template <int kMine>
__global__ void __launch_bounds__(1024)
topk_merge_kernel(const float* __restrict__ logits, const uint64_t* __restrict__ survivors, uint32_t n_survivors,
                  uint32_t tile_keep, uint32_t vocab, uint32_t retain_cap, float divisor, const uint32_t* __restrict__ history,
                  const uint32_t* __restrict__ history_count, const uint32_t* __restrict__ row_retain, uint32_t row_stride,
                  uint32_t history_stride, Candidates* __restrict__ result, uint32_t* __restrict__ status) {
    __shared__ uint32_t hist[256];
    __shared__ uint64_t sel[512];
    __shared__ uint64_t keys[512];  // selected keys in candidate order
    __shared__ uint32_t s_bin, s_above, s_count, s_in_bin;
    __shared__ uint64_t floor_key;
    const uint32_t row = blockIdx.x, lane = threadIdx.x & 63;
    // a row may ask for fewer than the launch's capacity (top_k plus ITS history count); history_count
    // and row_retain are read `row_stride` words apart (1, or the stride of a resolved-request record)
    uint32_t retain = retain_cap;
    if (row_retain) {
        const uint32_t want = row_retain[size_t(row) * row_stride];
        retain = want < 1 ? 1 : (want < retain_cap ? want : retain_cap);
    }
    const uint64_t* src = survivors + size_t(row) * n_survivors;
    // up to kMine keys per thread stay in registers (8 for the verify pass's lists, 34 for the 257 per
    // tile that the proposal law asks for); longer survivor lists are re-read from memory in every pass
    const bool cached = n_survivors <= kMine * blockDim.x;
    uint64_t mine[kMine];
#pragma unroll
    for (int u = 0; u < kMine; ++u) {
        const uint32_t i = threadIdx.x + u * blockDim.x;
        mine[u] = cached && i < n_survivors ? src[i] : 0;
    }
    // Shortcut for sorted tile lists (tile_keep > 0: the survivors are `tiles` descending lists of tile_keep
    // keys): the retain-th largest of the tiles' first r keys (tiles * r >= retain of them) is a lower bound
    // of the retain-th largest key overall, so only keys at or above it can be selected.  They are few (a
    // little over `retain` unless the logits tie massively); a rank sort of them is the exact answer.
    bool done = false;
    if (cached && tile_keep > 0) {
        const uint32_t tiles = n_survivors / tile_keep;
        const uint32_t r = (retain + tiles - 1) / tiles;
        const uint32_t heads = tiles * r;
        if (r <= tile_keep && heads <= 512) {
            for (uint32_t i = threadIdx.x; i < heads; i += blockDim.x) sel[i] = src[(i / r) * tile_keep + i % r];
            if (threadIdx.x == 0) { s_count = 0; floor_key = 0; }   // a floor of zero lets every key through
            __syncthreads();
            for (uint32_t i = threadIdx.x; i < heads; i += blockDim.x) {
                const uint64_t k = sel[i];
                uint32_t rank = 0;
                for (uint32_t j = 0; j < heads; ++j) rank += sel[j] > k;
                if (rank == retain - 1) floor_key = k;   // real keys are unique; only the zero padding repeats
            }
            __syncthreads();
            const uint64_t bound = floor_key;
            __syncthreads();
#pragma unroll
            for (int u = 0; u < kMine; ++u) {
                if (threadIdx.x + u * blockDim.x < n_survivors && mine[u] >= bound) {
                    const uint32_t at = atomicAdd(&s_count, 1u);
                    if (at < 512) sel[at] = mine[u];
                }
            }
            __syncthreads();
            const uint32_t n = s_count;
            if (n <= 512) {   // else: too many ties at the bound, the general path below decides
                for (uint32_t i = threadIdx.x; i < n; i += blockDim.x) {
                    const uint64_t k = sel[i];
                    uint32_t rank = 0;
                    for (uint32_t j = 0; j < n; ++j) rank += sel[j] > k;
                    if (rank < retain) keys[rank] = k;
                }
                done = true;
            }
            __syncthreads();
        }
    }
    if (!done) {
        uint64_t prefix = 0;
        uint32_t remaining = retain;  // rank of the wanted key among the keys that match `prefix`
        for (int pass = 0; pass < 8; ++pass) {
            const int shift = 56 - 8 * pass;
            for (uint32_t i = threadIdx.x; i < 256; i += blockDim.x) hist[i] = 0;
            __syncthreads();
            if (cached) {
    #pragma unroll
                for (int u = 0; u < kMine; ++u) {
                    const uint64_t k = mine[u];
                    hist_add(hist, threadIdx.x + u * blockDim.x < n_survivors && (pass == 0 || (k >> (shift + 8)) == prefix),
                             static_cast<uint32_t>(k >> shift) & 255u, lane);
                }
            } else {
                for (uint32_t i0 = 0; i0 < n_survivors; i0 += blockDim.x) {  // whole waves stay converged
                    const uint32_t i = i0 + threadIdx.x;
                    const uint64_t k = i < n_survivors ? src[i] : 0;
                    hist_add(hist, i < n_survivors && (pass == 0 || (k >> (shift + 8)) == prefix),
                             static_cast<uint32_t>(k >> shift) & 255u, lane);
                }
            }
            __syncthreads();
            if (threadIdx.x < 64) {  // lane l owns bins 255-4l .. 252-4l, highest first
                uint32_t c[4];
    #pragma unroll
                for (int j = 0; j < 4; ++j) c[j] = hist[255 - 4 * lane - j];
                const uint32_t own = c[0] + c[1] + c[2] + c[3];
                const uint32_t incl = wave_inclusive_scan(own);
                uint32_t above = incl - own;
                if (above < remaining && remaining <= incl) {
    #pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        if (remaining <= above + c[j]) { s_bin = 255 - 4 * lane - j; s_above = above; s_in_bin = c[j]; break; }
                        above += c[j];
                    }
                }
            }
            __syncthreads();
            prefix = (prefix << 8) | s_bin;
            remaining -= s_above;
            // the upper 32 bits are the logit: if every key that shares the threshold logit is wanted
            // (no tie across the cut), the token bits need no passes
            if (pass == 3 && s_in_bin == remaining) { prefix <<= 32; remaining = 0; break; }
        }
        // `prefix` is the retain-th largest key; keys above it are taken, then `remaining` copies of it
        // (more than one only for the zero padding of a short last tile)
        if (threadIdx.x == 0) s_count = 0;
        __syncthreads();
        if (cached) {
    #pragma unroll
            for (int u = 0; u < kMine; ++u)
                if (threadIdx.x + u * blockDim.x < n_survivors && mine[u] > prefix) sel[atomicAdd(&s_count, 1u)] = mine[u];
        } else {
            for (uint32_t i = threadIdx.x; i < n_survivors; i += blockDim.x) {
                const uint64_t k = src[i];
                if (k > prefix) sel[atomicAdd(&s_count, 1u)] = k;
            }
        }
        __syncthreads();
        const uint32_t above_total = s_count;
        for (uint32_t i = threadIdx.x; i < remaining; i += blockDim.x) sel[above_total + i] = prefix;
        __syncthreads();
        for (uint32_t i = threadIdx.x; i < retain; i += blockDim.x) {
            const uint64_t k = sel[i];
            uint32_t rank = 0;
            for (uint32_t j = 0; j < retain; ++j) {
                const uint64_t o = sel[j];
                rank += (o > k) || (o == k && j < i);
            }
            keys[rank] = k;
        }
    }
    emit_candidates(keys, retain, row, logits, vocab, divisor, history, history_count, row_stride, history_stride, result, status);
}

// ---- selection by threshold ------------------------------------------------------------------
// For large vocabularies the sort of every tile is more work than the answer needs.  The maxima of the
// 256-logit segments give a bound first: with at least `retain` segments, the retain-th largest segment
// maximum is at or below the retain-th largest logit of the row, so only logits at or above it can be
// selected, and on anything but massively tied rows they are few more than `retain`.  Two launches:
//   segment_max_kernel       the ordered score bits of every segment's maximum; clears the row's counters
//   threshold_select_kernel  every workgroup finds the bound for itself (a 4-pass radix select over at most
//                            1024 words), collects the keys of its 4096 logits that reach it into the row's
//                            list, and the workgroup that finishes last sorts the list and writes the row
// The list and the counters move with device-scope accesses (the workgroups sit on different L2s), every
// workgroup waits for its own stores before it counts itself done, and nobody waits for anybody: the last
// arrival is whoever draws the last ticket.  A row whose list overflows (more than kCollectCap logits tie
// into the bound) is selected exactly, and slowly, by a radix select over the whole row in that workgroup.
constexpr uint32_t kSeg = 256, kMaxSegs = 1024, kCollectTile = 4096, kCollectCap = 2048;
constexpr uint32_t kThresholdRowWords = kMaxSegs + 4 + 2 * kCollectCap;   // segment maxima, counter, done, pad, list

__device__ __forceinline__ uint32_t ordered_bits(float v) {
    const uint32_t b = __float_as_uint(v + 0.0f);
    return (b & 0x80000000u) ? ~b : (b | 0x80000000u);
}

__global__ void __launch_bounds__(256)
segment_max_kernel(const float* __restrict__ logits, uint32_t vocab, uint32_t segs, float divisor, uint32_t* __restrict__ ws) {
    const uint32_t row = blockIdx.y, lane = threadIdx.x & 63;
    const uint32_t seg = blockIdx.x * 4 + (threadIdx.x >> 6);
    uint32_t* row_ws = ws + size_t(row) * kThresholdRowWords;
    if (blockIdx.x == 0 && threadIdx.x < 4) row_ws[kMaxSegs + threadIdx.x] = 0;
    if (seg >= segs) return;
    const float* lr = logits + size_t(row) * vocab;
    uint32_t best = 0;
#pragma unroll
    for (uint32_t u = 0; u < kSeg / 64; ++u) {
        const uint32_t t = seg * kSeg + u * 64 + lane;
        if (t < vocab) {
            const uint32_t o = ordered_bits(lr[t] / divisor);
            best = o > best ? o : best;
        }
    }
    best = wave_max_u32(best);
    if (lane == 0) row_ws[seg] = best;
}

// the bin (highest first) that holds the `remaining`-th largest entry of a 256-bin histogram; first wave only
__device__ __forceinline__ void find_bin(const uint32_t* hist, uint32_t remaining, uint32_t lane, uint32_t& s_bin,
                                         uint32_t& s_above) {
    uint32_t c[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) c[j] = hist[255 - 4 * lane - j];
    const uint32_t own = c[0] + c[1] + c[2] + c[3];
    const uint32_t incl = wave_inclusive_scan(own);
    uint32_t above = incl - own;
    if (above < remaining && remaining <= incl) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            if (remaining <= above + c[j]) { s_bin = 255 - 4 * lane - j; s_above = above; break; }
            above += c[j];
        }
    }
}

__global__ void __launch_bounds__(1024)
threshold_select_kernel(const float* __restrict__ logits, uint32_t vocab, uint32_t segs, uint32_t retain_cap, float divisor,
                        const uint32_t* __restrict__ history, const uint32_t* __restrict__ history_count,
                        const uint32_t* __restrict__ row_retain, uint32_t row_stride, uint32_t history_stride,
                        uint32_t* __restrict__ ws, Candidates* __restrict__ result, uint32_t* __restrict__ status,
                        bool suppressed_ok) {
    __shared__ uint32_t hist[256];
    __shared__ uint64_t sel[kCollectCap];
    __shared__ uint64_t keys[512];
    __shared__ uint32_t s_bin, s_above, s_last, s_count;
    const uint32_t row = blockIdx.y, tid = threadIdx.x, lane = tid & 63;
    uint32_t retain = retain_cap;
    if (row_retain) {
        const uint32_t want = row_retain[size_t(row) * row_stride];
        retain = want < 1 ? 1 : (want < retain_cap ? want : retain_cap);
    }
    uint32_t* row_ws = ws + size_t(row) * kThresholdRowWords;
    uint32_t* counter = row_ws + kMaxSegs;
    uint32_t* done = counter + 1;
    uint64_t* list = reinterpret_cast<uint64_t*>(row_ws + kMaxSegs + 4);
    const float* lr = logits + size_t(row) * vocab;
    // this workgroup's logits are requested before the bound is worked out
    float mine[kCollectTile / 1024];
#pragma unroll
    for (uint32_t u = 0; u < kCollectTile / 1024; ++u) {
        const uint32_t t = blockIdx.x * kCollectTile + u * 1024 + tid;
        mine[u] = t < vocab ? lr[t] : 0.f;
    }
    // ---- the bound: the retain-th largest segment maximum (segs >= retain by the launch's condition) ----
    const uint32_t word = tid < segs ? row_ws[tid] : 0u;
    uint32_t prefix = 0, remaining = retain;
    for (int pass = 0; pass < 4; ++pass) {
        const int shift = 24 - 8 * pass;
        if (tid < 256) hist[tid] = 0;
        __syncthreads();
        hist_add(hist, tid < segs && (pass == 0 || (word >> (shift + 8)) == prefix), (word >> shift) & 255u, lane);
        __syncthreads();
        if (tid < 64) find_bin(hist, remaining, lane, s_bin, s_above);
        __syncthreads();
        prefix = (prefix << 8) | s_bin;
        remaining -= s_above;
    }
    const uint32_t bound = prefix;
    // ---- collect ----------------------------------------------------------------------------------
    bool bad = false;
#pragma unroll
    for (uint32_t u = 0; u < kCollectTile / 1024; ++u) {
        const uint32_t t = blockIdx.x * kCollectTile + u * 1024 + tid;
        bool hit = false;
        uint64_t key = 0;
        if (t < vocab) {
            const float v = mine[u] / divisor;
            bad |= (!isfinite(v) || !isfinite(mine[u])) && !(suppressed_ok && mine[u] == -INFINITY);
            key = make_key(v, t);
            hit = static_cast<uint32_t>(key >> 32) >= bound;
        }
        const uint64_t mask = __ballot(hit);
        if (mask) {
            const int leader = __ffsll(static_cast<long long>(mask)) - 1;
            uint32_t base = 0;
            if (lane == uint32_t(leader))
                base = __hip_atomic_fetch_add(counter, static_cast<uint32_t>(__popcll(mask)), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            base = __shfl(base, leader, kWave);
            const uint32_t at = base + static_cast<uint32_t>(__popcll(mask & ((uint64_t{1} << lane) - 1)));
            if (hit && at < kCollectCap) __hip_atomic_store(list + at, key, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    }
    if (bad && status) atomicOr(status + row, GUFFIN_STATUS_NONFINITE);
    // ---- the last workgroup of the row to get here finishes it -----------------------------------------
    __builtin_amdgcn_s_waitcnt(0);
    __syncthreads();
    if (tid == 0) {
        const uint32_t before = __hip_atomic_fetch_add(done, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        s_last = before + 1 == gridDim.x;
        s_count = 0;
    }
    __syncthreads();
    if (!s_last) return;
    const uint32_t n = __hip_atomic_load(counter, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (n <= kCollectCap) {
        for (uint32_t i = tid; i < n; i += blockDim.x) sel[i] = __hip_atomic_load(list + i, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (n <= 512) {
            __syncthreads();
            for (uint32_t i = tid; i < n; i += blockDim.x) {
                const uint64_t k = sel[i];
                uint32_t rank = 0;
                for (uint32_t j = 0; j < n; ++j) rank += sel[j] > k;
                if (rank < retain) keys[rank] = k;
            }
        } else {
            for (uint32_t i = n + tid; i < kCollectCap; i += blockDim.x) sel[i] = 0;
            bitonic_desc(sel, kCollectCap);
            for (uint32_t i = tid; i < retain; i += blockDim.x) keys[i] = sel[i];
        }
    } else {
        // more ties than the list holds: an 8-pass radix select over the whole row's keys, exact and slow
        uint64_t kprefix = 0;
        uint32_t left = retain;
        for (int pass = 0; pass < 8; ++pass) {
            const int shift = 56 - 8 * pass;
            if (tid < 256) hist[tid] = 0;
            __syncthreads();
            for (uint32_t i0 = 0; i0 < vocab; i0 += blockDim.x) {   // whole waves stay converged
                const uint32_t i = i0 + tid;
                const uint64_t k = i < vocab ? make_key(lr[i] / divisor, i) : 0;
                hist_add(hist, i < vocab && (pass == 0 || (k >> (shift + 8)) == kprefix), static_cast<uint32_t>(k >> shift) & 255u, lane);
            }
            __syncthreads();
            if (tid < 64) find_bin(hist, left, lane, s_bin, s_above);
            __syncthreads();
            kprefix = (kprefix << 8) | s_bin;
            left -= s_above;
        }
        // kprefix is the retain-th largest key (keys are unique): everything above it, then it
        for (uint32_t i = tid; i < vocab; i += blockDim.x) {
            const uint64_t k = make_key(lr[i] / divisor, i);
            if (k >= kprefix) sel[atomicAdd(&s_count, 1u)] = k;
        }
        __syncthreads();
        for (uint32_t i = tid; i < retain; i += blockDim.x) {
            const uint64_t k = sel[i];
            uint32_t rank = 0;
            for (uint32_t j = 0; j < retain; ++j) rank += sel[j] > k;
            keys[rank] = k;
        }
    }
    emit_candidates(keys, retain, row, logits, vocab, divisor, history, history_count, row_stride, history_stride, result, status);
}

// ---- verify-row input validation --------------------------------------------------------------
__global__ void input_validation_kernel(const uint32_t* __restrict__ actual, const uint32_t* __restrict__ expected,
                                        uint32_t rows, uint32_t vocab, uint32_t* __restrict__ status) {
    const uint32_t row = blockIdx.x * blockDim.x + threadIdx.x;
    if (row < rows && (actual[row] >= vocab || actual[row] != expected[row])) atomicOr(status, GUFFIN_STATUS_BAD_TOKEN);
}

// ---- selection requests --------------------------------------------------------------------
// One wave per row: the raw ring and suffix become the resolved record and the row's history list.
__global__ void __launch_bounds__(64)
selection_requests_kernel(const SelectionRow* __restrict__ raw, uint32_t vocab, uint32_t top_k, uint32_t repetition,
                          ResolvedRow* __restrict__ resolved, uint32_t* __restrict__ histories,
                          uint32_t* __restrict__ status) {
    const uint32_t row = blockIdx.x, lane = threadIdx.x;
    const SelectionRow& r = raw[row];
    uint32_t token = 0, st = 0;
    const uint32_t count = resolve_history(r.history_token_ids, r.history_head, r.history_length, r.history_window_limit,
                                           r.suffix_token_ids, r.suffix_count, vocab, repetition != 0, lane, token, st);
    ResolvedRow& out = resolved[row];
    out.history_token_ids[lane] = token;
    if (histories) histories[size_t(row) * kRequestHistory + lane] = token;
    if (lane == 0) {
        out.top_k = top_k;
        out.base_candidate_count = top_k + count;
        out.history_count = count;
        out.reserved = 0;
        if (st && status) atomicOr(status, st);
    }
}

// ---- greedy argmax ---------------------------------------------------------------------
__global__ void __launch_bounds__(256)
argmax_tile_kernel(const float* __restrict__ logits, uint64_t* __restrict__ partial, uint32_t vocab,
                   uint32_t* __restrict__ status) {
    __shared__ uint64_t best[4];
    const uint32_t row = blockIdx.y;
    const float* lr = logits + size_t(row) * vocab;
    uint64_t k = 0;
    bool bad = false;
    for (uint32_t t = blockIdx.x * blockDim.x + threadIdx.x; t < vocab; t += gridDim.x * blockDim.x) {
        const float v = lr[t];
        bad |= !isfinite(v);
        const uint64_t c = make_key(v, t);
        k = c > k ? c : k;
    }
    if (bad && status) atomicOr(status + row, GUFFIN_STATUS_NONFINITE);
#pragma unroll
    for (int s = 32; s > 0; s >>= 1) {
        const uint64_t o = __shfl_xor(k, s, kWave);
        k = o > k ? o : k;
    }
    if ((threadIdx.x & 63) == 0) best[threadIdx.x >> 6] = k;
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int i = 1; i < 4; ++i) k = best[i] > k ? best[i] : k;
        partial[size_t(row) * gridDim.x + blockIdx.x] = k;
    }
}

__global__ void __launch_bounds__(256)
argmax_final_kernel(const uint64_t* __restrict__ partial, uint32_t n, uint32_t* __restrict__ token,
                    float* __restrict__ logit) {
    __shared__ uint64_t best[4];
    const uint32_t row = blockIdx.x;
    uint64_t k = 0;
    for (uint32_t i = threadIdx.x; i < n; i += blockDim.x) {
        const uint64_t c = partial[size_t(row) * n + i];
        k = c > k ? c : k;
    }
#pragma unroll
    for (int s = 32; s > 0; s >>= 1) {
        const uint64_t o = __shfl_xor(k, s, kWave);
        k = o > k ? o : k;
    }
    if ((threadIdx.x & 63) == 0) best[threadIdx.x >> 6] = k;
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int i = 1; i < 4; ++i) k = best[i] > k ? best[i] : k;
        token[row] = key_token(k);
        if (logit) logit[row] = key_logit(k);
    }
}

}  // namespace

int head_init() { return 0; }

}  // namespace guffin

using namespace guffin;

extern "C" uint64_t guffin_hip_select_workspace_bytes(uint32_t rows, uint32_t vocab, uint32_t retain) {
    const uint64_t tiles = (uint64_t(vocab) + kTile - 1) / kTile;
    const uint64_t keep = retain < kTile ? retain : kTile;
    const uint64_t sorted_tiles = rows * tiles * keep * 8, by_threshold = uint64_t(rows) * kThresholdRowWords * 4;
    return sorted_tiles > by_threshold ? sorted_tiles : by_threshold;   // either path may serve the call
}

namespace guffin {
int select_candidates_scaled(hipStream_t s, const float* logits, uint32_t rows, uint32_t vocab, uint32_t retain,
                             float divisor, const uint32_t* history, const uint32_t* history_count,
                             void* workspace, void* result, uint32_t* status, bool suppressed_ok = false,
                             const uint32_t* row_retain = nullptr, uint32_t row_stride = 1);
}

extern "C" int guffin_hip_select_candidates(void* stream, const float* logits, uint32_t rows, uint32_t vocab,
                                            uint32_t retain, const uint32_t* history, const uint32_t* history_count,
                                            void* workspace, void* result, uint32_t* status) {
    return select_candidates_scaled(as_stream(stream), logits, rows, vocab, retain, 1.0f, history, history_count,
                                    workspace, result, status);
}

int guffin::select_candidates_scaled(hipStream_t s, const float* logits, uint32_t rows, uint32_t vocab,
                                     uint32_t retain, float divisor, const uint32_t* history,
                                     const uint32_t* history_count, void* workspace, void* result, uint32_t* status,
                                     bool suppressed_ok, const uint32_t* row_retain, uint32_t row_stride) {
    if (!logits || !workspace || !result) return fail(GUFFIN_E_ARG, "select_candidates: null pointer");
    if (rows == 0 || vocab == 0) return fail(GUFFIN_E_SHAPE, "select_candidates: empty shape");
    if (retain == 0 || retain > 320) return fail(GUFFIN_E_CAPACITY, "select_candidates: retain must be in [1, 320] (top_k <= 256 plus 64 history tokens)");
    if ((history == nullptr) != (history_count == nullptr)) return fail(GUFFIN_E_ARG, "select_candidates: history and its counts come together");
    if (reinterpret_cast<uintptr_t>(workspace) & 7u) return fail(GUFFIN_E_ALIGN, "select_candidates: workspace must be 8-byte aligned");
    const uint32_t keep = retain < vocab ? retain : vocab;
    const uint32_t tiles = (vocab + kTile - 1) / kTile;
    const uint32_t segs = (vocab + kSeg - 1) / kSeg;
    if (segs <= kMaxSegs && segs >= 2 * keep) {   // large vocabulary: a bound from the segment maxima, then one pass
        uint32_t* words = static_cast<uint32_t*>(workspace);
        launch(segment_max_kernel, dim3((segs + 3) / 4, rows), dim3(256), 0, s, logits, vocab, segs, divisor, words);
        if (int rc = check_launch("select_candidates(segment maxima)")) return rc;
        launch(threshold_select_kernel, dim3((vocab + kCollectTile - 1) / kCollectTile, rows), dim3(1024), 0, s,
                           logits, vocab, segs, keep, divisor, history, history_count, row_retain, row_stride,
                           row_stride == 1 ? 64u : row_stride, words, static_cast<Candidates*>(result), status, suppressed_ok);
        return check_launch("select_candidates(threshold)");
    }
    uint64_t* surv = static_cast<uint64_t*>(workspace);
    launch(topk_tile_kernel, dim3(tiles, rows), dim3(1024), 0, s, logits, surv, vocab, keep, divisor, status, suppressed_ok);
    if (int rc = check_launch("select_candidates(tile)")) return rc;
    if (tiles * keep <= 8 * 1024)
        launch(topk_merge_kernel<8>, dim3(rows), dim3(1024), 0, s, logits, surv, tiles * keep, keep, vocab,
                           keep, divisor, history, history_count, row_retain, row_stride, row_stride == 1 ? 64u : row_stride,
                           static_cast<Candidates*>(result), status);
    else
        launch(topk_merge_kernel<34>, dim3(rows), dim3(1024), 0, s, logits, surv, tiles * keep, keep, vocab,
                           keep, divisor, history, history_count, row_retain, row_stride, row_stride == 1 ? 64u : row_stride,
                           static_cast<Candidates*>(result), status);
    return check_launch("select_candidates(merge)");
}

extern "C" int guffin_hip_input_validation(void* stream, const uint32_t* actual, const uint32_t* expected, uint32_t rows,
                                           uint32_t vocab, uint32_t* status) {
    if (!actual || !expected || !status) return fail(GUFFIN_E_ARG, "input_validation: null pointer");
    if (rows == 0 || vocab == 0) return fail(GUFFIN_E_SHAPE, "input_validation: empty shape");
    launch(input_validation_kernel, dim3((rows + 63) / 64), dim3(64), 0, as_stream(stream), actual, expected,
                       rows, vocab, status);
    return check_launch("input_validation");
}

extern "C" int guffin_hip_selection_requests(void* stream, const void* raw, uint32_t rows, uint32_t vocab, uint32_t top_k,
                                             uint32_t repetition_enabled, void* resolved, uint32_t* histories,
                                             uint32_t* status) {
    if (!raw || !resolved) return fail(GUFFIN_E_ARG, "selection_requests: null pointer");
    if (rows == 0 || vocab == 0) return fail(GUFFIN_E_SHAPE, "selection_requests: empty shape");
    if (top_k == 0 || top_k > 256) return fail(GUFFIN_E_CAPACITY, "selection_requests: top_k must be in [1, 256]");
    if ((reinterpret_cast<uintptr_t>(raw) | reinterpret_cast<uintptr_t>(resolved)) & 3u)
        return fail(GUFFIN_E_ALIGN, "selection_requests: rows must be 4-byte aligned");
    launch(selection_requests_kernel, dim3(rows), dim3(64), 0, as_stream(stream),
                       static_cast<const SelectionRow*>(raw), vocab, top_k, repetition_enabled,
                       static_cast<ResolvedRow*>(resolved), histories, status);
    return check_launch("selection_requests");
}

extern "C" int guffin_hip_select_candidates_resolved(void* stream, const float* logits, uint32_t rows, uint32_t vocab,
                                                     uint32_t retain_capacity, const void* resolved, void* workspace,
                                                     void* result, uint32_t* status) {
    if (!resolved) return fail(GUFFIN_E_ARG, "select_candidates_resolved: null pointer");
    const uint32_t* words = static_cast<const uint32_t*>(resolved);
    constexpr uint32_t stride = sizeof(ResolvedRow) / 4;
    // history ids, their count and the row's retain all sit in the record; the ids are 68 words apart too
    return select_candidates_scaled(as_stream(stream), logits, rows, vocab, retain_capacity, 1.0f,
                                    words + offsetof(ResolvedRow, history_token_ids) / 4,
                                    words + offsetof(ResolvedRow, history_count) / 4, workspace, result, status, false,
                                    words + offsetof(ResolvedRow, base_candidate_count) / 4, stride);
}

extern "C" int guffin_hip_argmax(void* stream, const float* logits, uint32_t rows, uint32_t vocab, void* workspace,
                                 uint32_t* token, float* logit, uint32_t* status) {
    if (!logits || !workspace || !token) return fail(GUFFIN_E_ARG, "argmax: null pointer");
    if (rows == 0 || vocab == 0) return fail(GUFFIN_E_SHAPE, "argmax: empty shape");
    if (reinterpret_cast<uintptr_t>(workspace) & 7u) return fail(GUFFIN_E_ALIGN, "argmax: workspace must be 8-byte aligned");
    const uint32_t blocks = vocab / 1024 < 1 ? 1 : (vocab / 1024 > 256 ? 256 : vocab / 1024);
    hipStream_t s = as_stream(stream);
    uint64_t* part = static_cast<uint64_t*>(workspace);  // rows * 256 keys at most
    launch(argmax_tile_kernel, dim3(blocks, rows), dim3(256), 0, s, logits, part, vocab, status);
    if (int rc = check_launch("argmax(tile)")) return rc;
    launch(argmax_final_kernel, dim3(rows), dim3(256), 0, s, part, blocks, token, logit);
    return check_launch("argmax(final)");
}
