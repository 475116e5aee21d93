// GQA decode / verify attention over an fp16 KV cache (gfx950).
//
// Replaces MetalCommandContext::encode_verifier_attention and its partition reducer
// (src/tensor/backends/metal/metal_command_context.hpp:267,
//  src/tensor/backends/metal/metal_kernels.mm:3061-3382); CPU definition
// src/tensor/ops/attention.cpp:482-618 with softmax.cpp:42-71.
//
// Token list of a query row, in order: `base_count` committed tokens read from the ring
// at slot (base_first + t) & ring_mask, then the row's ancestors among the private rows
// of this verify pass.  All rows of a pass (<= 2) and the `group` query heads that share a
// KV head are served by one workgroup, so each K/V row is read once per KV head and
// partition: the rows' lists are merged into one virtual list (union of the ring ranges,
// then every private row) with a per-row validity mask.
//
// Workgroup = (partition of TP consecutive virtual tokens, KV head), 256 threads.
//   pass 1  scores: 16 lanes split the head dimension of one token (512-byte K rows, each of a
//           lane's two requests part of 256 contiguous bytes), four tokens per wave at a time;
//           fp16 keys enter v_fma_mix_f32 directly;
//           a 4-step exchange inside each 16-lane group finishes the dot product.
//   softmax per query over the partition in LDS (max, exp, sum).
//   pass 2  values: a half wave owns one token (a lane eight output dims, 16-byte loads);
//           halves are combined by one lane exchange, the four waves through LDS.
// Partitions emit (max, denominator, unnormalised output); a second kernel merges them in
// partition order.  fp32 throughout, keys/values stay fp16 in memory.
#include <algorithm>

#include "common.hpp"
#include "receipt.hpp"

namespace guffin {
namespace {

typedef _Float16 half2_t __attribute__((ext_vector_type(2)));

constexpr int kMaxRows = 2;

struct AttnArgs {
    const float* q;              // [rows][q_heads][hd]
    const uint16_t* ring_k; const uint16_t* ring_v;   // [cap][kv_heads][hd]
    const uint16_t* priv_k; const uint16_t* priv_v;   // [private rows][kv_heads][hd]
    const uint32_t* schedule;    // [rows][4]
    const uint32_t* ancestors;
    float* part_out;             // [rows][q_heads][partitions][hd]
    float* part_ml;              // [rows][q_heads][partitions][2]
    uint32_t rows, q_heads, kv_heads, hd, ring_mask, tp, span, partitions, private_rows;   // span: tokens the last partition may hold (>= tp)
    float scale;
    // fused mode: q, k, v arrive as the projections' partial planes; every workgroup prepares
    // the query heads it serves (head norm, rotation) and the partition that holds a private
    // row prepares that row's key and value and publishes them as fp16
    const float* q_raw; const float* k_raw; const float* v_raw;
    uint32_t planes; size_t q_stride, k_stride, v_stride;
    const float* q_norm; const float* k_norm; const float2* rope;   // rope: [rows][hd/2] (cos, sin)
    uint16_t* priv_k_out; uint16_t* priv_v_out;
    float eps; uint32_t* status;
    // the rows' schedule words and ancestor masks when the host knows them (contiguous rows at a host-known
    // position): they arrive with the launch arguments instead of through two dependent trips to memory
    uint32_t inline_schedule, sched[kMaxRows][4], amask[kMaxRows];
};

// One head row (hd = 256) by one wave, in registers: lane l holds columns l, l+64, l+128, l+192.
// load: sum of the partial planes plus gamma and the rotation pairs, all requested together;
// finish: optional RMS norm with gamma and rotation of the pairs (i, i + 128) — the arithmetic of
// qkv_post_kernel.  Several rows may be loaded before any is finished (one memory round trip).
struct HeadRow { float v[4]; float gm[4]; float2 rp[2]; };

__device__ __forceinline__ void load_head_row(HeadRow& h, const float* src, uint32_t planes, size_t stride,
                                              const float* gamma, const float2* rope_row, uint32_t lane) {
#pragma unroll
    for (int i = 0; i < 4; ++i) h.gm[i] = gamma ? gamma[lane + 64 * i] : 1.f;
    h.rp[0] = rope_row ? rope_row[lane] : make_float2(1.f, 0.f);
    h.rp[1] = rope_row ? rope_row[lane + 64] : make_float2(1.f, 0.f);
    // up to four planes: every plane of every column is requested before the first add (a loop over a
    // run-time plane count waits for each plane of each column in turn: eight dependent trips for two planes)
    if (planes <= 4) {
        float t[4][4];
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int s = 0; s < 4; ++s) t[i][s] = uint32_t(s) < planes ? src[lane + 64 * i + s * stride] : 0.f;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            float v = t[i][0];
#pragma unroll
            for (int s = 1; s < 4; ++s) v = uint32_t(s) < planes ? v + t[i][s] : v;   // plane order, as load_planes
            h.v[i] = v;
        }
        return;
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) h.v[i] = load_planes(src + lane + 64 * i, planes, stride);
}

__device__ __forceinline__ void finish_head_row(HeadRow& h, bool norm, bool rotate, float eps) {
    if (norm) {
        float ss = 0.f;
#pragma unroll
        for (int i = 0; i < 4; ++i) ss = fmaf(h.v[i], h.v[i], ss);
        ss = wave_sum(ss);
        const float inv = 1.0f / sqrtf(ss / 256.0f + eps);
#pragma unroll
        for (int i = 0; i < 4; ++i) h.v[i] = h.v[i] * inv * h.gm[i];
    }
    if (rotate) {
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const float first = h.v[i], second = h.v[i + 2];
            h.v[i] = __fsub_rn(__fmul_rn(first, h.rp[i].x), __fmul_rn(second, h.rp[i].y));
            h.v[i + 2] = __fadd_rn(__fmul_rn(first, h.rp[i].y), __fmul_rn(second, h.rp[i].x));
        }
    }
}

// A workgroup barrier for data that moves through LDS: it waits for this wave's LDS operations only.
// (__syncthreads() also waits for every vector load in flight -- here the key rows requested before the
// queries are prepared and the value rows requested before the softmax, which are meant to stay in flight
// across it.)  Nothing a wave stores to global memory in this kernel is read by another wave of the launch.
__device__ __forceinline__ void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

__device__ __forceinline__ float dot2(float acc, uint32_t packed_half2, float a, float b) {
    const half2_t h = __builtin_bit_cast(half2_t, packed_half2);
    acc = fmaf(static_cast<float>(h.x), a, acc);
    return fmaf(static_cast<float>(h.y), b, acc);
}

// waves of a partition's workgroup: two per SIMD.  With eight the queries and the private rows' key / value are
// prepared by different waves, and a 32-token partition is one round of keys and two of values per wave.
// (Eight query rows keep four waves: their per-wave output slots would not fit 64 KB of LDS otherwise.)
constexpr int attention_waves(int queries) { return queries <= 4 ? 8 : 4; }

template <int ROWS, int GROUP, int HD, bool FUSED>
__global__ void __launch_bounds__(64 * attention_waves(ROWS * GROUP)) attn_partial_kernel(AttnArgs a) {
    static_assert(HD == 256, "head dimension 256 (16 lanes x 16 dims)");
    constexpr int NQ = ROWS * GROUP;
    constexpr int kAW = attention_waves(NQ);
    extern __shared__ float lds[];
    float* sc = lds;                          // [NQ][tp] scores, then probabilities
    float* merge = lds + NQ * a.span;         // [kAW][NQ][HD]
    float* q_s = merge + kAW * NQ * HD;       // fused: [NQ][HD] prepared queries
    __shared__ float s_max[NQ], s_sum[NQ];
    __shared__ __attribute__((aligned(16))) uint16_t k_s[FUSED ? ROWS : 1][HD], v_s[FUSED ? ROWS : 1][HD];

    const uint32_t part = blockIdx.x, kvh = blockIdx.y;
    const uint32_t lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
    constexpr uint32_t group = GROUP;
    // Every launch argument is asked for here, in one go: left to their first uses, the scalar loads of a
    // 300-byte argument block are spread over the blocks of the prologue, one dependent trip each.
    asm volatile("" :: "s"(a.q), "s"(a.ring_k), "s"(a.ring_v), "s"(a.priv_k), "s"(a.priv_v), "s"(a.schedule), "s"(a.ancestors),
                 "s"(a.part_out), "s"(a.part_ml), "s"(a.rows), "s"(a.q_heads), "s"(a.kv_heads), "s"(a.ring_mask), "s"(a.tp),
                 "s"(a.span), "s"(a.partitions), "s"(a.private_rows), "s"(a.scale), "s"(a.q_raw), "s"(a.k_raw), "s"(a.v_raw),
                 "s"(a.planes), "s"(a.q_stride), "s"(a.k_stride), "s"(a.v_stride), "s"(a.q_norm), "s"(a.k_norm), "s"(a.rope),
                 "s"(a.priv_k_out), "s"(a.priv_v_out));
    asm volatile("" :: "s"(a.eps), "s"(a.status), "s"(a.inline_schedule), "s"(a.sched[0][0]), "s"(a.sched[0][1]),
                 "s"(a.sched[0][2]), "s"(a.sched[0][3]), "s"(a.sched[kMaxRows - 1][0]), "s"(a.sched[kMaxRows - 1][1]),
                 "s"(a.sched[kMaxRows - 1][2]), "s"(a.sched[kMaxRows - 1][3]), "s"(a.amask[0]), "s"(a.amask[kMaxRows - 1]));
    const uint32_t row_stride = a.kv_heads * HD;  // in halves

    // fused: the query rows of this wave (w, w+kAW, ..) are requested first; their addresses need
    // nothing but the launch arguments, so they travel together with the schedule below
    constexpr int QI = (NQ + kAW - 1) / kAW;
    HeadRow qr[FUSED ? QI : 1];
    if constexpr (FUSED) {
#pragma unroll
        for (int i = 0; i < QI; ++i) {
            const uint32_t item = wv + kAW * i;
            if (item < NQ) {
                const uint32_t r = item / group, head = kvh * group + item % group;
                load_head_row(qr[i], a.q_raw + (size_t(r) * a.q_heads + head) * HD, a.planes, a.q_stride, a.q_norm,
                              a.rope + size_t(r) * (HD / 2), lane);
            }
        }
    }

    // merged virtual token list
    uint32_t u_first = 0xFFFFFFFFu, u_end = 0;
    uint32_t bfirst[ROWS], bend[ROWS], amask[ROWS];
#pragma unroll
    for (int r = 0; r < ROWS; ++r) {
        bfirst[r] = 0; bend[r] = 0; amask[r] = 0;
        if (a.inline_schedule) {
            bfirst[r] = a.sched[r][0]; bend[r] = a.sched[r][0] + a.sched[r][1];
            if (a.sched[r][1]) { u_first = min(u_first, bfirst[r]); u_end = max(u_end, bend[r]); }
            amask[r] = a.amask[r];
        } else {
            const uint32_t* s = a.schedule + 4 * r;
            bfirst[r] = s[0]; bend[r] = s[0] + s[1];
            if (s[1]) { u_first = min(u_first, s[0]); u_end = max(u_end, s[0] + s[1]); }
            for (uint32_t i = 0; i < s[3]; ++i) amask[r] |= 1u << a.ancestors[s[2] + i];
        }
    }
    if (u_end == 0) { u_first = 0; }
    const uint32_t n_ring = u_end - u_first, n_total = n_ring + a.private_rows;
    // the last partition takes what is left (at most `span` tokens: the launch has one partition fewer when a
    // handful of tokens -- the private rows -- would otherwise need a workgroup of their own on a full chip)
    const uint32_t t0 = part * a.tp, t1 = part + 1 == a.partitions ? min(t0 + a.span, n_total) : min(t0 + a.tp, n_total);

    // ---- keys: four rounds of loads are issued before their dot products so that a wave keeps
    // 16 key rows (8 KB) in flight (a round is 4 tokens per wave, 4 kAW per workgroup); in fused mode the first
    // batch travels during the preparation
    constexpr int U = 4;
    // (a lane's 16 dimensions are 8 seg .. 8 seg + 7 of each half of the row: either request of a row's 16 lanes
    // then covers 256 contiguous bytes -- with 32 contiguous bytes per lane both requests touch every line of the row)
    const uint32_t slot = lane >> 4, seg = lane & 15;  // token slot in the wave, segment of the head dimension
    const uint32_t tb_first = t0 + wv * 4 + slot;
    uint4 k0[U], k1[U];
    // one round's key row of this lane group: token tb + 4 kAW u, into slot u
    auto load_key_round = [&](int u, uint32_t tb) {
        const uint32_t t = tb + 4 * kAW * u;
        k0[u] = make_uint4(0, 0, 0, 0); k1[u] = k0[u];
        if (t < t1) {
            const bool is_priv = t >= n_ring;
            if (FUSED && is_priv) return;  // taken from LDS once prepared
            const uint16_t* kp = is_priv ? a.priv_k + size_t(t - n_ring) * row_stride
                                         : a.ring_k + size_t((u_first + t) & a.ring_mask) * row_stride;
            kp += kvh * HD + seg * 8;
            // (4-byte aligned requests: a caller's K/V view may start at any word of its parent allocation)
            k0[u] = ld16_a4(reinterpret_cast<const uint8_t*>(kp)); k1[u] = ld16_a4(reinterpret_cast<const uint8_t*>(kp + HD / 2));
        }
    };
    auto load_keys = [&](uint32_t tb) {
#pragma unroll
        for (int u = 0; u < U; ++u) load_key_round(u, tb);
    };
    if constexpr (FUSED) load_keys(tb_first);
    // ---- values: a half wave covers one value row (32 lanes x 8 dims, 16-byte loads), a wave two
    // tokens per round, four rounds in flight; in fused mode the first batch is requested while
    // the softmax runs
    const uint32_t hsel = lane >> 5, dl = (lane & 31) * 8;
    const uint32_t vb_first = t0 + wv * 2 + hsel;
    constexpr int UV = 8;   // value rounds in flight: a round is half a key round's bytes (16 per lane)
    uint4 vv[UV];
    auto load_value_round = [&](int u, uint32_t tb) {
        const uint32_t t = tb + 2 * kAW * u;
        vv[u] = make_uint4(0, 0, 0, 0);
        if (t < t1) {
            const bool is_priv = t >= n_ring;
            if (FUSED && is_priv) return;  // taken from LDS once prepared
            const uint16_t* vp = is_priv ? a.priv_v + size_t(t - n_ring) * row_stride
                                         : a.ring_v + size_t((u_first + t) & a.ring_mask) * row_stride;
            vv[u] = ld16_a4(reinterpret_cast<const uint8_t*>(vp + kvh * HD + dl));
        }
    };
    auto load_values = [&](uint32_t tb) {
#pragma unroll
        for (int u = 0; u < UV; ++u) load_value_round(u, tb);
    };

    if constexpr (FUSED) {
        // wave w prepares query rows w, w+kAW, ..; the last 2 ROWS waves prepare the private rows' key / value
        // (row i/2, key for even i) when this partition holds it; every load is issued before any arithmetic
        HeadRow kvr;
        const uint32_t ki = wv - (kAW - 2 * ROWS);   // wraps for the waves below: pr >= ROWS then
        const uint32_t pr = ki >> 1, pt = n_ring + pr;
        const bool is_key = (ki & 1u) == 0;
        const bool mine = wv >= uint32_t(kAW - 2 * ROWS) && pr < ROWS && pr < a.private_rows && pt >= t0 && pt < t1;
        const size_t kv_off = (size_t(pr) * a.kv_heads + kvh) * HD;
        if (mine)
            load_head_row(kvr, (is_key ? a.k_raw : a.v_raw) + kv_off, a.planes, is_key ? a.k_stride : a.v_stride,
                          is_key ? a.k_norm : nullptr, is_key ? a.rope + size_t(pr) * (HD / 2) : nullptr, lane);
#pragma unroll
        for (int i = 0; i < QI; ++i) {
            const uint32_t item = wv + kAW * i;
            if (item < NQ) {
                finish_head_row(qr[i], a.q_norm != nullptr, true, a.eps);
#pragma unroll
                for (int c = 0; c < 4; ++c) q_s[item * HD + lane + 64 * c] = qr[i].v[c];
            }
        }
        if (mine) {
            finish_head_row(kvr, is_key && a.k_norm != nullptr, is_key, a.eps);
            bool bad = false;
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                const _Float16 hv = static_cast<_Float16>(kvr.v[c]);  // round-to-nearest-even, after rotation
                bad |= !isfinite(static_cast<float>(hv));
                const uint16_t bits = __builtin_bit_cast(uint16_t, hv);
                (is_key ? k_s : v_s)[pr][lane + 64 * c] = bits;
                (is_key ? a.priv_k_out : a.priv_v_out)[kv_off + lane + 64 * c] = bits;
            }
            if (bad && a.status) atomicOr(a.status, GUFFIN_STATUS_KV_NONFINITE);
        }
        lds_barrier();
    }
    // ---- pass 1: scores ------------------------------------------------------------
    {
        float qv[NQ][16];
#pragma unroll
        for (int n = 0; n < NQ; ++n) {
            const uint32_t r = n / group, g = n % group;
            const float* qp = FUSED ? q_s + n * HD + seg * 8
                                    : a.q + (size_t(r) * a.q_heads + kvh * group + g) * HD + seg * 8;
#pragma unroll
            for (int i = 0; i < 8; ++i) { qv[n][i] = qp[i] * a.scale; qv[n][8 + i] = qp[HD / 2 + i] * a.scale; }
        }
        // U rounds stay in flight for the whole walk: a slot is asked for its next row (U rounds on) as soon as its
        // row has been read, so a long partition streams instead of filling and draining once per batch
        if constexpr (!FUSED) load_keys(tb_first);
        for (uint32_t tb = tb_first; tb < t0 + a.span; tb += 4 * kAW * U) {
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const uint32_t t = tb + 4 * kAW * u;
                if (t >= t0 + a.span) break;
                const bool in_range = t < t1, is_priv = t >= n_ring;
                const uint32_t pos = u_first + t, prow = t - n_ring;
                if (FUSED && in_range && is_priv) {
                    const uint16_t* kp = &k_s[prow][seg * 8];
                    k0[u] = *reinterpret_cast<const uint4*>(kp); k1[u] = *reinterpret_cast<const uint4*>(kp + HD / 2);
                }
                const uint32_t kw[8] = {k0[u].x, k0[u].y, k0[u].z, k0[u].w, k1[u].x, k1[u].y, k1[u].z, k1[u].w};
                if (tb + 4 * kAW * U < t0 + a.span) load_key_round(u, tb + 4 * kAW * U);
                float s[NQ];
#pragma unroll
                for (int n = 0; n < NQ; ++n) {
                    s[n] = 0.f;
#pragma unroll
                    for (int i = 0; i < 8; ++i) s[n] = dot2(s[n], kw[i], qv[n][2 * i], qv[n][2 * i + 1]);
                    s[n] = row16_sum(s[n]);
                }
                if (seg == 0) {
#pragma unroll
                    for (int n = 0; n < NQ; ++n) {
                        const uint32_t r = n / group;
                        const bool valid = in_range && (is_priv ? ((amask[r] >> prow) & 1u) != 0
                                                                : (pos >= bfirst[r] && pos < bend[r]));
                        sc[n * a.span + (t - t0)] = valid ? s[n] : -INFINITY;
                    }
                }
            }
        }
    }
    if constexpr (FUSED) load_values(vb_first);  // in flight during the softmax
    lds_barrier();

    // ---- softmax over the partition, one wave per query ----------------------------------
    for (uint32_t n = wv; n < NQ; n += kAW) {
        float m = -INFINITY;
        for (uint32_t i = lane; i < a.span; i += 64) m = fmaxf(m, sc[n * a.span + i]);
        m = wave_max(m);
        float l = 0.f;
        for (uint32_t i = lane; i < a.span; i += 64) {
            const float v = sc[n * a.span + i];
            const float p = v == -INFINITY ? 0.f : expf(v - m);
            sc[n * a.span + i] = p;
            l += p;
        }
        l = wave_sum(l);
        if (lane == 0) { s_max[n] = m; s_sum[n] = l; }
    }
    lds_barrier();
    // ---- pass 2: values; halves are combined by a lane exchange, waves via LDS ------------
    {
        float acc[NQ][8];
#pragma unroll
        for (int n = 0; n < NQ; ++n)
#pragma unroll
            for (int i = 0; i < 8; ++i) acc[n][i] = 0.f;
        if constexpr (!FUSED) load_values(vb_first);
        for (uint32_t tb = vb_first; tb < t1; tb += 2 * kAW * UV) {
#pragma unroll
            for (int u = 0; u < UV; ++u) {
                const uint32_t t = tb + 2 * kAW * u;
                if (t >= t1) break;
                if (FUSED && t >= n_ring) vv[u] = *reinterpret_cast<const uint4*>(&v_s[t - n_ring][dl]);
                const uint32_t w4[4] = {vv[u].x, vv[u].y, vv[u].z, vv[u].w};
                if (tb + 2 * kAW * UV < t1) load_value_round(u, tb + 2 * kAW * UV);
#pragma unroll
                for (int n = 0; n < NQ; ++n) {
                    const float p = sc[n * a.span + (t - t0)];
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        const half2_t h = __builtin_bit_cast(half2_t, w4[i]);
                        acc[n][2 * i] = fmaf(static_cast<float>(h.x), p, acc[n][2 * i]);
                        acc[n][2 * i + 1] = fmaf(static_cast<float>(h.y), p, acc[n][2 * i + 1]);
                    }
                }
            }
        }
#pragma unroll
        for (int n = 0; n < NQ; ++n) {
#pragma unroll
            for (int i = 0; i < 8; ++i) acc[n][i] += __shfl_xor(acc[n][i], 32, kWave);
            if (hsel == 0) {
                float* mp = merge + (wv * NQ + n) * HD + dl;
                *reinterpret_cast<float4*>(mp) = make_float4(acc[n][0], acc[n][1], acc[n][2], acc[n][3]);
                *reinterpret_cast<float4*>(mp + 4) = make_float4(acc[n][4], acc[n][5], acc[n][6], acc[n][7]);
            }
        }
    }
    lds_barrier();
    for (uint32_t i = threadIdx.x; i < NQ * HD; i += 64 * kAW) {
        const uint32_t n = i / HD, d = i % HD;
        float pair[kAW / 2];   // waves in pairs, the pairs in order
#pragma unroll
        for (int w = 0; w < kAW; w += 2) pair[w / 2] = merge[(w * NQ + n) * HD + d] + merge[((w + 1) * NQ + n) * HD + d];
        float v = pair[0] + pair[1];
#pragma unroll
        for (int w = 2; w < kAW / 2; w += 2) v += pair[w] + pair[w + 1];
        const uint32_t r = n / group, g = n % group, head = kvh * group + g;
        const size_t slot = (size_t(r) * a.q_heads + head) * a.partitions + part;
        a.part_out[slot * HD + d] = v;
        if (d == 0) { a.part_ml[slot * 2] = s_max[n]; a.part_ml[slot * 2 + 1] = s_sum[n]; }
    }
}

// out[row][head][:] = sum_p e^(m_p - M) acc_p / sum_p e^(m_p - M) l_p, partitions in order.
// Each thread owns one output dimension.  The outputs of the first 64 partitions are requested at
// once, before the weights exist (indices beyond the last partition read the last one again and
// meet a zero weight), so up to 64 partitions cost one trip to memory; weights and denominators
// terms are formed once, in parallel, in LDS.
constexpr int kMergeAhead = 64;
template <int AHEAD>
__global__ void __launch_bounds__(256)
attn_merge_kernel(const float* __restrict__ part_out, const float* __restrict__ part_ml, float* __restrict__ out,
                  float* __restrict__ out_sums, uint32_t partitions, uint32_t hd, uint32_t q_heads,
                  uint32_t* __restrict__ status) {
    extern __shared__ float wgt[];  // [max(partitions, 64)] weights, then as many partition sums l_p
    __shared__ float red[4];
    __shared__ float rowbuf[1024];
    const uint32_t rh = blockIdx.x;  // row * q_heads + head
    const uint32_t lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
    const uint32_t slots = partitions > uint32_t(AHEAD) ? partitions : uint32_t(AHEAD);
    float* lsum = wgt + slots;
    const float* ml = part_ml + size_t(rh) * partitions * 2;
    const float* po = part_out + size_t(rh) * partitions * hd;
    const uint32_t d0 = threadIdx.x;
    // this thread's (maximum, denominator) pair, requested first and once: the maximum and the weights below
    // would otherwise each fetch the two words one after the other
    const float2 own = threadIdx.x < partitions ? reinterpret_cast<const float2*>(ml)[threadIdx.x] : make_float2(0.f, 0.f);
    float pre[AHEAD];
#pragma unroll
    for (int p = 0; p < AHEAD; ++p) {
        const uint32_t q = uint32_t(p) < partitions ? uint32_t(p) : partitions - 1;
        pre[p] = d0 < hd ? po[size_t(q) * hd + d0] : 0.f;
    }
    float m = own.y > 0.f ? own.x : -INFINITY;
    for (uint32_t p = threadIdx.x + 256; p < partitions; p += 256) if (ml[2 * p + 1] > 0.f) m = fmaxf(m, ml[2 * p]);
    m = wave_max(m);
    if (lane == 0) red[wv] = m;
    __syncthreads();
    const float M = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
    for (uint32_t p = threadIdx.x; p < slots; p += 256) {
        const bool first = p == threadIdx.x;
        const float l = first ? own.y : p < partitions ? ml[2 * p + 1] : 0.f;
        wgt[p] = l > 0.f ? expf((first ? own.x : ml[2 * p]) - M) : 0.f;
        lsum[p] = l;
    }
    __syncthreads();
    float denom = 0.f, acc0 = 0.f;
#pragma unroll
    for (int q = 0; q < AHEAD; ++q) {
        denom = fmaf(wgt[q], lsum[q], denom);
        acc0 = fmaf(wgt[q], pre[q], acc0);
    }
    for (uint32_t p = AHEAD; p < partitions; ++p) denom = fmaf(wgt[p], lsum[p], denom);
    bool bad = false;
    for (uint32_t d = threadIdx.x; d < hd; d += blockDim.x) {
        float acc = 0.f;
        uint32_t p = 0;
        if (d == d0) { acc = acc0; p = partitions < uint32_t(AHEAD) ? partitions : uint32_t(AHEAD); }
        for (; p + 4 <= partitions; p += 4) {
            const float v0 = po[size_t(p) * hd + d], v1 = po[size_t(p + 1) * hd + d], v2 = po[size_t(p + 2) * hd + d],
                        v3 = po[size_t(p + 3) * hd + d];
            acc = fmaf(wgt[p], v0, acc); acc = fmaf(wgt[p + 1], v1, acc);
            acc = fmaf(wgt[p + 2], v2, acc); acc = fmaf(wgt[p + 3], v3, acc);
        }
        for (; p < partitions; ++p) acc = fmaf(wgt[p], po[size_t(p) * hd + d], acc);
        const float v = acc / denom;
        bad |= !isfinite(v);
        out[size_t(rh) * hd + d] = v;
        rowbuf[d] = v;
    }
    if (bad && status) atomicOr(status, GUFFIN_STATUS_NONFINITE);
    if (out_sums) {
        __syncthreads();
        // receipt of the attention output row [q_heads*hd], the o-projection's input
        emit_receipt(rowbuf, (rh % q_heads) * hd, hd, rh / q_heads, gridDim.x / q_heads, q_heads * hd, out_sums);
    }
}

template <int ROWS, int GROUP>
int launch_partial(hipStream_t s, const AttnArgs& a) {
    constexpr int NQ = ROWS * GROUP;
    constexpr int kAW = attention_waves(NQ);
    const bool fused = a.q_raw != nullptr;
    const size_t lds = (size_t(NQ) * a.span + size_t(kAW) * NQ * 256 + (fused ? size_t(NQ) * 256 : 0)) * sizeof(float);
    if (fused)
        launch((attn_partial_kernel<ROWS, GROUP, 256, true>), dim3(a.partitions, a.kv_heads), dim3(64 * kAW), lds, s, a);
    else
        launch((attn_partial_kernel<ROWS, GROUP, 256, false>), dim3(a.partitions, a.kv_heads), dim3(64 * kAW), lds, s, a);
    return check_launch("attention_partial");
}

}  // namespace
}  // namespace guffin

using namespace guffin;

namespace {
struct AttentionSplit { uint32_t partitions, tp, span; };
AttentionSplit attention_split(uint32_t max_tokens, uint32_t kv_heads) {
    uint32_t tp = 256;
    const uint32_t floor_tp = ((max_tokens + 31) / 32) * kv_heads < 64 ? 16u : 32u;
    while (tp > floor_tp && ((max_tokens + tp - 1) / tp) * kv_heads < 256) tp >>= 1;
    uint32_t partitions = (max_tokens + tp - 1) / tp;
    tp = (((max_tokens + partitions - 1) / partitions) + 15u) & ~15u;   // whole rounds of 16 tokens per workgroup
    partitions = (max_tokens + tp - 1) / tp;
    uint32_t span = tp;
    // A last partition of at most 16 tokens that alone pushes the launch past one workgroup per CU (1025 tokens
    // on 8 KV heads: 33 x 8 = 264) is folded into the one before it: the eight workgroups that would share a
    // CU with another finish 2 us after everybody else.
    if (partitions > 1) {
        const uint32_t rem = max_tokens - (partitions - 1) * tp;
        if (rem <= 16 && partitions * kv_heads > 256 && (partitions - 1) * kv_heads <= 256) { partitions -= 1; span = tp + 16; }
    }
    return {partitions, tp, span};
}
}  // namespace

extern "C" uint32_t guffin_hip_attention_partitions(uint32_t max_tokens, uint32_t kv_heads) {
    // tokens per partition: aim at >= 256 workgroups, between 32 and 256 tokens each; a context so
    // small that 32-token partitions give fewer than 64 workgroups (the drafter's window) is cut into
    // 16-token partitions, which shortens every workgroup's chain of dependent steps
    if (max_tokens == 0 || kv_heads == 0) return 0;
    return attention_split(max_tokens, kv_heads).partitions;
}

namespace {
struct FusedInputs {
    const float* q_raw; const float* k_raw; const float* v_raw;
    uint32_t planes; uint64_t q_stride, k_stride, v_stride;
    const float* q_norm; const float* k_norm; const float* rope; float eps;
};

int attention_decode(void* stream, const float* q, const FusedInputs* fused, const void* ring_k, const void* ring_v,
                     void* priv_k, void* priv_v, const uint32_t* schedule, const uint32_t* ancestors, float* out,
                     float* out_sums, float* partial_out, float* partial_ml, uint32_t rows, uint32_t private_rows,
                     uint32_t max_tokens, uint32_t ring_mask, uint32_t q_heads, uint32_t kv_heads, uint32_t head_dim,
                     float scale, uint32_t* status, const uint32_t* host_schedule = nullptr, const uint32_t* host_amask = nullptr) {
    if ((!q && !fused) || !ring_k || !ring_v || !priv_k || !priv_v || !schedule || !ancestors || !out || !partial_out || !partial_ml)
        return fail(GUFFIN_E_ARG, "attention_decode: null pointer");
    if (rows == 0 || rows > kMaxRows || private_rows > 32) return fail(GUFFIN_E_SHAPE, "attention_decode: rows must be 1 or 2, private rows <= 32");
    if (head_dim != 256) return fail(GUFFIN_E_SHAPE, "attention_decode: head_dim must be 256");
    if (reinterpret_cast<uintptr_t>(out_sums) & 255u) return fail(GUFFIN_E_ALIGN, "attention_decode: the receipt must be 256-byte aligned");
    if (kv_heads == 0 || q_heads % kv_heads != 0) return fail(GUFFIN_E_SHAPE, "attention_decode: q_heads must be a multiple of kv_heads");
    if ((ring_mask & (ring_mask + 1)) != 0) return fail(GUFFIN_E_ARG, "attention_decode: ring capacity must be a power of two");
    if (max_tokens == 0) return fail(GUFFIN_E_SHAPE, "attention_decode: max_tokens must cover every row's token list");
    if (!(scale > 0.f)) return fail(GUFFIN_E_ARG, "attention_decode: scale must be positive");
    // K/V views may start at any 4-byte offset of their allocation (the reference's tests use a 12-byte one,
    // tests/tensor/gemma3_metal_tests.cpp:765-774): the kernels ask for their rows as 4-byte aligned 16-byte pieces
    if ((reinterpret_cast<uintptr_t>(ring_k) & 3u) || (reinterpret_cast<uintptr_t>(ring_v) & 3u)
        || (reinterpret_cast<uintptr_t>(priv_k) & 3u) || (reinterpret_cast<uintptr_t>(priv_v) & 3u))
        return fail(GUFFIN_E_ALIGN, "attention_decode: KV rows must be 4-byte aligned");
    const uint32_t group = q_heads / kv_heads;
    AttnArgs a {};
    a.q = q;
    a.ring_k = static_cast<const uint16_t*>(ring_k); a.ring_v = static_cast<const uint16_t*>(ring_v);
    a.priv_k = static_cast<const uint16_t*>(priv_k); a.priv_v = static_cast<const uint16_t*>(priv_v);
    a.schedule = schedule; a.ancestors = ancestors; a.part_out = partial_out; a.part_ml = partial_ml;
    a.rows = rows; a.q_heads = q_heads; a.kv_heads = kv_heads; a.hd = head_dim; a.ring_mask = ring_mask;
    const AttentionSplit split = attention_split(max_tokens, kv_heads);
    a.partitions = split.partitions; a.tp = split.tp; a.span = split.span;
    a.private_rows = private_rows; a.scale = scale;
    if (host_schedule && host_amask) {
        a.inline_schedule = 1;
        for (uint32_t r = 0; r < rows; ++r) {
            for (int k = 0; k < 4; ++k) a.sched[r][k] = host_schedule[4 * r + k];
            a.amask[r] = host_amask[r];
        }
    }
    if (fused) {
        if (!fused->q_raw || !fused->k_raw || !fused->v_raw || !fused->rope)
            return fail(GUFFIN_E_ARG, "qkv_attention: null pointer");
        if (fused->planes == 0 || private_rows != rows)
            return fail(GUFFIN_E_SHAPE, "qkv_attention: planes >= 1 and one private row per query row");
        if (!(fused->eps > 0.f)) return fail(GUFFIN_E_ARG, "qkv_attention: epsilon must be positive");
        if (reinterpret_cast<uintptr_t>(fused->rope) & 7u) return fail(GUFFIN_E_ALIGN, "qkv_attention: rope table must be 8-byte aligned");
        a.q_raw = fused->q_raw; a.k_raw = fused->k_raw; a.v_raw = fused->v_raw; a.planes = fused->planes;
        a.q_stride = fused->q_stride; a.k_stride = fused->k_stride; a.v_stride = fused->v_stride;
        a.q_norm = fused->q_norm; a.k_norm = fused->k_norm; a.rope = reinterpret_cast<const float2*>(fused->rope);
        a.priv_k_out = static_cast<uint16_t*>(priv_k); a.priv_v_out = static_cast<uint16_t*>(priv_v);
        a.eps = fused->eps; a.status = status;
    }
    hipStream_t s = as_stream(stream);
    int rc;
    switch (group * 10 + rows) {
        case 11: rc = launch_partial<1, 1>(s, a); break;
        case 12: rc = launch_partial<2, 1>(s, a); break;
        case 21: rc = launch_partial<1, 2>(s, a); break;
        case 22: rc = launch_partial<2, 2>(s, a); break;
        case 41: rc = launch_partial<1, 4>(s, a); break;
        case 42: rc = launch_partial<2, 4>(s, a); break;
        default: return fail(GUFFIN_E_SHAPE, "attention_decode: q_heads / kv_heads must be 1, 2 or 4");
    }
    if (rc) return rc;
    // the outputs requested ahead: 32 when the partitions are that few (a local layer), else 64
    if (a.partitions <= 32)
        launch(attn_merge_kernel<32>, dim3(rows * q_heads), dim3(256), 2 * 32 * sizeof(float), s, partial_out, partial_ml, out,
                           out_sums, a.partitions, head_dim, q_heads, status);
    else
        launch(attn_merge_kernel<kMergeAhead>, dim3(rows * q_heads), dim3(256), 2 * std::max<uint32_t>(a.partitions, kMergeAhead) * sizeof(float), s, partial_out, partial_ml, out,
                           out_sums, a.partitions, head_dim, q_heads, status);
    return check_launch("attention_merge");
}
}  // namespace

extern "C" int guffin_hip_attention_decode(void* stream, const float* q, const void* ring_k, const void* ring_v,
                                           const void* priv_k, const void* priv_v, const uint32_t* schedule,
                                           const uint32_t* ancestors, float* out, float* out_sums,
                                           float* partial_out, float* partial_ml, uint32_t rows,
                                           uint32_t private_rows, uint32_t max_tokens, uint32_t ring_mask,
                                           uint32_t q_heads, uint32_t kv_heads, uint32_t head_dim, float scale,
                                           uint32_t* status) {
    if (!q) return fail(GUFFIN_E_ARG, "attention_decode: null pointer");
    return attention_decode(stream, q, nullptr, ring_k, ring_v, const_cast<void*>(priv_k), const_cast<void*>(priv_v),
                            schedule, ancestors, out, out_sums, partial_out, partial_ml, rows, private_rows, max_tokens,
                            ring_mask, q_heads, kv_heads, head_dim, scale, status);
}

// guffin_hip_qkv_attention for contiguous rows whose schedule the host knows: the same words the device copy
// holds (`schedule`, still passed) travel as launch arguments.
namespace guffin {
int qkv_attention_scheduled(void* stream, const float* q_raw, const float* k_raw, const float* v_raw, uint32_t planes,
                            uint64_t q_plane_stride, uint64_t k_plane_stride, uint64_t v_plane_stride, const float* q_norm,
                            const float* k_norm, const float* rope_table, float eps, const void* ring_k, const void* ring_v,
                            void* priv_k, void* priv_v, const uint32_t* schedule, const uint32_t* ancestors,
                            const uint32_t* host_schedule, const uint32_t* host_amask, float* out, float* out_sums,
                            float* partial_out, float* partial_ml, uint32_t rows, uint32_t max_tokens, uint32_t ring_mask,
                            uint32_t q_heads, uint32_t kv_heads, uint32_t head_dim, float scale, uint32_t* status) {
    const FusedInputs f {q_raw, k_raw, v_raw, planes, q_plane_stride, k_plane_stride, v_plane_stride, q_norm, k_norm,
                         rope_table, eps};
    return attention_decode(stream, nullptr, &f, ring_k, ring_v, priv_k, priv_v, schedule, ancestors, out, out_sums,
                            partial_out, partial_ml, rows, rows, max_tokens, ring_mask, q_heads, kv_heads, head_dim,
                            scale, status, host_schedule, host_amask);
}
}  // namespace guffin

extern "C" int guffin_hip_qkv_attention(void* stream, const float* q_raw, const float* k_raw, const float* v_raw,
                                        uint32_t planes, uint64_t q_plane_stride, uint64_t k_plane_stride,
                                        uint64_t v_plane_stride, const float* q_norm, const float* k_norm,
                                        const float* rope_table, float eps, const void* ring_k, const void* ring_v,
                                        void* priv_k, void* priv_v, const uint32_t* schedule,
                                        const uint32_t* ancestors, float* out, float* out_sums, float* partial_out,
                                        float* partial_ml, uint32_t rows, uint32_t max_tokens, uint32_t ring_mask,
                                        uint32_t q_heads, uint32_t kv_heads, uint32_t head_dim, float scale,
                                        uint32_t* status) {
    const FusedInputs f {q_raw, k_raw, v_raw, planes, q_plane_stride, k_plane_stride, v_plane_stride, q_norm, k_norm,
                         rope_table, eps};
    return attention_decode(stream, nullptr, &f, ring_k, ring_v, priv_k, priv_v, schedule, ancestors, out, out_sums,
                            partial_out, partial_ml, rows, rows, max_tokens, ring_mask, q_heads, kv_heads, head_dim,
                            scale, status);
}
