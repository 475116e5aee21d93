// Dequant-GEMV kernels for GGUF block streams on gfx950 (wavefront 64).
//
// y[r, n] = sum_k x[r, k] * W[k, n] for 1 or 2 activation rows; column n of W owns the
// K/block consecutive blocks starting at block n*(K/block).
// Reference operator: src/tensor/backends/cpu_backend.cpp:301-323 (definition),
// src/tensor/backends/metal/metal_kernels.mm:551-750, 788-922, 267-436 (GPU work split
// this design replaces).
//
// Design (one scheme for Q4_K and Q6_K):
//  * A workgroup is S k-slices x T column tiles of waves.  Each wave owns C output
//    columns and, per pass, one "chunk" of consecutive blocks of each of them; a lane
//    owns a fixed 16-byte quant run of one block, so that every global load of the
//    wave is a set of contiguous 64/128-byte runs of the block stream and each lane
//    needs only a handful of scale fields.
//  * The activation rows are staged once per workgroup in LDS, permuted into the
//    order the lanes consume them (float4 j of lane l lives at [j][l]: conflict free),
//    together with the per-run sums the "-dmin*m" (Q4_K) and "-32" (Q6_K) terms need.
//  * Quants are unpacked four at a time (mask + v_cvt_f32_ubyteN) and accumulated with
//    fp32 FMAs against the fp32 activations; scales are applied once per 16/32-run.
//  * The first pass's weight loads are issued before the activations are staged;
//    later passes rely on the other resident waves to cover the load latency.
//  * C*R partial sums are reduced across the wave with a halving exchange (fixed
//    order), k-slices are combined through LDS in slice order: results are
//    deterministic, and each row's arithmetic does not depend on R.
// Q8_0 (34-byte blocks) maps one lane to one block and sums a column's block partials
// from LDS in block order.
#include "common.hpp"

namespace guffin {
namespace {

// ---------------------------------------------------------------------------------
// Bit-exact block decode (one thread per element)
// ---------------------------------------------------------------------------------
__device__ __forceinline__ float q8_0_element(const uint8_t* b, uint32_t i) {
    const float d = h2f(ld_u16(b));
    return __fmul_rn(d, static_cast<float>(static_cast<int8_t>(b[2 + i])));
}

__device__ __forceinline__ float q4_k_element(const uint8_t* b, uint32_t i) {
    const float d = h2f(ld_u16(b)), dmin = h2f(ld_u16(b + 2));
    const uint8_t* s = b + 4;
    const uint32_t g = i >> 5;
    uint32_t sc, mn;
    if (g < 4) {
        sc = s[g] & 63u;
        mn = s[g + 4] & 63u;
    } else {
        sc = (s[g + 4] & 0x0Fu) | ((s[g - 4] >> 6) << 4);
        mn = (s[g + 4] >> 4) | ((s[g] >> 6) << 4);
    }
    const uint32_t byte = b[16 + (i >> 6) * 32 + (i & 31)];
    const uint32_t q = (i & 63) < 32 ? (byte & 0x0Fu) : (byte >> 4);
    const float a = __fmul_rn(__fmul_rn(d, static_cast<float>(sc)), static_cast<float>(q));
    return __fsub_rn(a, __fmul_rn(dmin, static_cast<float>(mn)));
}

__device__ __forceinline__ float q6_k_element(const uint8_t* b, uint32_t i) {
    const uint32_t half = i >> 7, r = i & 127, l = r & 31;
    const uint32_t lo_byte = b[half * 64 + ((r >> 5) & 1) * 32 + l];
    const uint32_t lo = r < 64 ? (lo_byte & 0x0Fu) : (lo_byte >> 4);
    const uint32_t hi = (b[128 + half * 32 + l] >> ((r >> 5) * 2)) & 3u;
    const int q = static_cast<int>(lo | (hi << 4)) - 32;
    const float scale = static_cast<float>(static_cast<int8_t>(b[192 + (i >> 4)]));
    const float d = h2f(ld_u16(b + 208));
    return __fmul_rn(__fmul_rn(d, scale), static_cast<float>(q));
}

template <int DTYPE>
__global__ void dequant_kernel(const uint8_t* __restrict__ blocks, uint64_t n_elems, float* __restrict__ out) {
    constexpr uint32_t be = DTYPE == GUFFIN_Q8_0 ? 32 : 256;
    constexpr uint32_t bb = DTYPE == GUFFIN_Q8_0 ? 34 : DTYPE == GUFFIN_Q4_K ? 144 : 210;
    const uint64_t stride = uint64_t(gridDim.x) * blockDim.x;
    for (uint64_t e = uint64_t(blockIdx.x) * blockDim.x + threadIdx.x; e < n_elems; e += stride) {
        const uint8_t* b = blocks + (e / be) * bb;
        const uint32_t i = static_cast<uint32_t>(e % be);
        float v;
        if constexpr (DTYPE == GUFFIN_Q8_0) v = q8_0_element(b, i);
        else if constexpr (DTYPE == GUFFIN_Q4_K) v = q4_k_element(b, i);
        else v = q6_k_element(b, i);
        out[e] = v;
    }
}

// ---------------------------------------------------------------------------------
// Shared pieces of the K-quant GEMV
// ---------------------------------------------------------------------------------
struct GemvDims {
    uint32_t K, N, nblk;      // inputs, output columns, blocks per column
    uint32_t nchunks;         // chunks (16 Q4_K / 8 Q6_K blocks) per column
    uint32_t S, T;            // k-slices and column tiles per workgroup
    uint32_t ntilegroups;     // ceil(N / (T*C))
};

// LDS image of the activations for the Q4_K lane mapping.
//   lane = (block_in_chunk << 2) | (hh << 1) | t0i   handles, for hh = sub-block pair and
//   t0i = 16-byte half, the quant bytes [16j,16j+16) and [64+16j, 64+16j+16) of its block.
//   which = 0..3 : low / high nibbles of the first run, low / high nibbles of the second.
// Element e (0..255) of a block: e = 128*(which>>1) + 64*hh + 32*(which&1) + 16*t0i + 4*q4 + i.
__device__ __forceinline__ void stage_q4k(const float* __restrict__ x, float4* lds4, float* sums,
                                          int R, uint32_t K, uint32_t nchunks) {
    const uint32_t f4_per_row = nchunks * 1024u;
    const uint32_t total = R * f4_per_row;
    for (uint32_t f = threadIdx.x; f < total; f += blockDim.x) {
        const uint32_t r = f / f4_per_row, cf = f - r * f4_per_row;
        const uint32_t chunk = cf >> 10, fl = cf & 1023u;
        const uint32_t k = chunk * 4096u + fl * 4u;
        float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
        if (k < K) v = ldf4_a4(x + size_t(r) * K + k);
        const uint32_t bl = fl >> 6, e = (fl & 63u) * 4u;
        const uint32_t which = ((e >> 7) << 1) | ((e >> 5) & 1u);
        const uint32_t lane = (bl << 2) | (((e >> 6) & 1u) << 1) | ((e >> 4) & 1u);
        const uint32_t q4 = (e >> 2) & 3u;
        lds4[r * f4_per_row + chunk * 1024u + (which * 4u + q4) * 64u + lane] = v;
        float s = (v.x + v.y) + (v.z + v.w);
        s += __shfl_xor(s, 1, kWave);
        s += __shfl_xor(s, 2, kWave);
        if (q4 == 0) sums[(r * nchunks + chunk) * 256u + which * 64u + lane] = s;
    }
}

// Q6_K lane mapping: lane = (block_in_chunk << 3) | (h << 2) | t, 8 blocks per chunk.
//   lane owns ql bytes [h*64 + 16t, +16): low nibbles are elements h*128 + 32*(t>>1) + 16*(t&1) + i,
//   high nibbles the same + 64.  which = 0 (low run) / 1 (high run).
__device__ __forceinline__ void stage_q6k(const float* __restrict__ x, float4* lds4, float* sums,
                                          int R, uint32_t K, uint32_t nchunks) {
    const uint32_t f4_per_row = nchunks * 512u;
    const uint32_t total = R * f4_per_row;
    for (uint32_t f = threadIdx.x; f < total; f += blockDim.x) {
        const uint32_t r = f / f4_per_row, cf = f - r * f4_per_row;
        const uint32_t chunk = cf >> 9, fl = cf & 511u;
        const uint32_t k = chunk * 2048u + fl * 4u;
        float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
        if (k < K) v = ldf4_a4(x + size_t(r) * K + k);
        const uint32_t bl = fl >> 6, e = (fl & 63u) * 4u;  // e = element in block
        const uint32_t h = e >> 7, rr = e & 127u;
        const uint32_t which = rr >> 6;
        const uint32_t t = (((rr >> 5) & 1u) << 1) | ((rr >> 4) & 1u);
        const uint32_t lane = (bl << 3) | (h << 2) | t;
        const uint32_t q4 = (rr >> 2) & 3u;
        lds4[r * f4_per_row + chunk * 512u + (which * 4u + q4) * 64u + lane] = v;
        float s = (v.x + v.y) + (v.z + v.w);
        s += __shfl_xor(s, 1, kWave);
        s += __shfl_xor(s, 2, kWave);
        if (q4 == 0) sums[(r * nchunks + chunk) * 128u + which * 64u + lane] = s;
    }
}

struct Q4Regs { uint4 hdr, qa, qb; };
struct Q6Regs { uint4 ql, qh; uint2 sc; uint32_t d; };

__device__ __forceinline__ void zero(Q4Regs& r) {
    r.hdr = make_uint4(0, 0, 0, 0); r.qa = r.hdr; r.qb = r.hdr;
}
__device__ __forceinline__ void zero(Q6Regs& r) {
    r.ql = make_uint4(0, 0, 0, 0); r.qh = r.ql; r.sc = make_uint2(0, 0); r.d = 0;
}

// 16 quants of one run (4 dwords of masked bytes) against 16 activations, R rows
template <int R>
__device__ __forceinline__ void dot16(const uint32_t (&q)[4], const float4 (&xv)[R][4], float (&p)[R]) {
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        const uint32_t v = opaque(q[k]);
        const float f0 = ub0(v), f1 = ub1(v), f2 = ub2(v), f3 = ub3(v);
#pragma unroll
        for (int r = 0; r < R; ++r) {
            p[r] = fmaf(f0, xv[r][k].x, p[r]);
            p[r] = fmaf(f1, xv[r][k].y, p[r]);
            p[r] = fmaf(f2, xv[r][k].z, p[r]);
            p[r] = fmaf(f3, xv[r][k].w, p[r]);
        }
    }
}

// ---------------------------------------------------------------------------------
// Q4_K
// ---------------------------------------------------------------------------------
template <int R, int C>
__global__ void __launch_bounds__(1024)
gemv_q4k_kernel(const uint8_t* __restrict__ w, const float* __restrict__ x, float* __restrict__ y,
                GemvDims dm) {
    extern __shared__ float4 lds4[];
    const uint32_t f4_per_row = dm.nchunks * 1024u;
    float* sums = reinterpret_cast<float*>(lds4 + R * f4_per_row);
    float* red = sums + R * dm.nchunks * 256u;  // [2][S][T][C*R]

    const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
    const uint32_t slice = wv % dm.S, tile = wv / dm.S;
    const uint32_t bl = lane >> 2, j = lane & 3, hh = j >> 1;
    const uint32_t passes = (dm.nchunks + dm.S - 1) / dm.S;
    const size_t col_bytes = size_t(dm.nblk) * 144u;

    auto load = [&](Q4Regs (&regs)[C], uint32_t tg, uint32_t pass) {
        const uint32_t chunk = pass * dm.S + slice;
        const uint32_t b = chunk * 16u + bl;
        const uint32_t col0 = (tg * dm.T + tile) * C;
#pragma unroll
        for (int c = 0; c < C; ++c) {
            const uint32_t col = col0 + c;
            if (chunk < dm.nchunks && b < dm.nblk && col < dm.N) {
                const uint8_t* blk = w + col * col_bytes + size_t(b) * 144u;
                regs[c].hdr = ld16_a4(blk);
                regs[c].qa = ld16_a4(blk + 16 + 16 * j);
                regs[c].qb = ld16_a4(blk + 80 + 16 * j);
            } else {
                zero(regs[c]);
            }
        }
    };

    const uint32_t n_items = dm.ntilegroups > blockIdx.x
        ? ((dm.ntilegroups - blockIdx.x + gridDim.x - 1) / gridDim.x) * passes : 0;
    Q4Regs cur[C];
    if (n_items) load(cur, blockIdx.x, 0);  // in flight while the activations are staged
    stage_q4k(x, lds4, sums, R, dm.K, dm.nchunks);
    __syncthreads();

    float acc[C * R];
#pragma unroll
    for (int i = 0; i < C * R; ++i) acc[i] = 0.f;

    for (uint32_t it = 0; it < n_items; ++it) {
        const uint32_t tg = blockIdx.x + (it / passes) * gridDim.x, pass = it % passes;
        if (it) load(cur, tg, pass);

        const uint32_t chunk = pass * dm.S + slice;
        if (chunk < dm.nchunks) {
            const float4* xl = lds4 + chunk * 1024u + lane;
            const float* sm = sums + chunk * 256u + lane;
            uint32_t scp[C], mp[C];
#pragma unroll
            for (int c = 0; c < C; ++c) {
                const uint32_t s0 = cur[c].hdr.y >> (16 * hh), s1 = cur[c].hdr.z >> (16 * hh),
                               s2 = cur[c].hdr.w >> (16 * hh);
                const uint32_t sc_lo = s0 & 0x3F3Fu, m_lo = s1 & 0x3F3Fu;
                const uint32_t sc_hi = (s2 & 0x0F0Fu) | ((s0 & 0xC0C0u) >> 2);
                const uint32_t m_hi = ((s2 >> 4) & 0x0F0Fu) | ((s1 & 0xC0C0u) >> 2);
                scp[c] = opaque(sc_lo | (sc_hi << 16));  // bytes: run0 low, run0 high, run1 low, run1 high
                mp[c] = opaque(m_lo | (m_hi << 16));
            }
            // which = 2*run + nibble: one 16-activation run per row is live at a time
#pragma unroll
            for (int which = 0; which < 4; ++which) {
                float4 xv[R][4];
                float sx[R];
#pragma unroll
                for (int r = 0; r < R; ++r) {
#pragma unroll
                    for (int q4 = 0; q4 < 4; ++q4) xv[r][q4] = xl[r * f4_per_row + (which * 4 + q4) * 64];
                    sx[r] = sm[r * dm.nchunks * 256u + which * 64];
                }
#pragma unroll
                for (int c = 0; c < C; ++c) {
                    const uint4 q = (which & 2) ? cur[c].qb : cur[c].qa;
                    const uint32_t mask = (which & 1) ? 0xF0F0F0F0u : 0x0F0F0F0Fu;  // high nibbles stay 16x too large
                    const uint32_t nib[4] = {q.x & mask, q.y & mask, q.z & mask, q.w & mask};
                    float p[R];
#pragma unroll
                    for (int r = 0; r < R; ++r) p[r] = 0.f;
                    dot16<R>(nib, xv, p);
                    const float scb = which == 0 ? ub0(scp[c]) : which == 1 ? ub1(scp[c]) : which == 2 ? ub2(scp[c]) : ub3(scp[c]);
                    const float mb = which == 0 ? ub0(mp[c]) : which == 1 ? ub1(mp[c]) : which == 2 ? ub2(mp[c]) : ub3(mp[c]);
                    const float d = h2f(cur[c].hdr.x & 0xFFFFu), dmin = h2f(cur[c].hdr.x >> 16);
                    const float sf = (which & 1) ? (d * 0.0625f) * scb : d * scb;
                    const float mf = dmin * mb;
#pragma unroll
                    for (int r = 0; r < R; ++r) {
                        acc[c * R + r] = fmaf(sf, p[r], acc[c * R + r]);
                        acc[c * R + r] = fmaf(-mf, sx[r], acc[c * R + r]);
                    }
                }
            }
        }

        if (pass + 1 == passes) {  // tile group finished: reduce and store
            wave_reduce_multi<C * R>(acc, lane);
            constexpr int shift = reduce_multi_shift<C * R>();
            const uint32_t idx = lane >> shift;
            const bool owner = (lane & ((1 << shift) - 1)) == 0;
            if (dm.S == 1) {
                const uint32_t col = (tg * dm.T + tile) * C + idx / R;
                if (owner && col < dm.N) y[size_t(idx % R) * dm.N + col] = acc[0];
            } else {
                float* buf = red + ((it / passes) & 1u) * (dm.S * dm.T * C * R);
                if (owner) buf[(slice * dm.T + tile) * (C * R) + idx] = acc[0];
                __syncthreads();
                if (threadIdx.x < dm.T * C * R) {
                    const uint32_t tl = threadIdx.x / (C * R), id = threadIdx.x % (C * R);
                    float total = 0.f;
                    for (uint32_t s = 0; s < dm.S; ++s) total += buf[(s * dm.T + tl) * (C * R) + id];
                    const uint32_t col = (tg * dm.T + tl) * C + id / R;
                    if (col < dm.N) y[size_t(id % R) * dm.N + col] = total;
                }
            }
#pragma unroll
            for (int i = 0; i < C * R; ++i) acc[i] = 0.f;
        }
    }
}

// ---------------------------------------------------------------------------------
// Q6_K
// ---------------------------------------------------------------------------------
template <int R, int C>
__global__ void __launch_bounds__(1024)
gemv_q6k_kernel(const uint8_t* __restrict__ w, const float* __restrict__ x, float* __restrict__ y,
                GemvDims dm) {
    extern __shared__ float4 lds4[];
    const uint32_t f4_per_row = dm.nchunks * 512u;
    float* sums = reinterpret_cast<float*>(lds4 + R * f4_per_row);
    float* red = sums + R * dm.nchunks * 128u;

    const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
    const uint32_t slice = wv % dm.S, tile = wv / dm.S;
    const uint32_t bl = lane >> 3, h = (lane >> 2) & 1, t = lane & 3;
    const uint32_t passes = (dm.nchunks + dm.S - 1) / dm.S;
    const size_t col_bytes = size_t(dm.nblk) * 210u;
    const uint32_t shift_lo = 2 * (t >> 1), shift_hi = 4 + 2 * (t >> 1);

    auto load = [&](Q6Regs (&regs)[C], uint32_t tg, uint32_t pass) {
        const uint32_t chunk = pass * dm.S + slice;
        const uint32_t b = chunk * 8u + bl;
        const uint32_t col0 = (tg * dm.T + tile) * C;
#pragma unroll
        for (int c = 0; c < C; ++c) {
            const uint32_t col = col0 + c;
            if (chunk < dm.nchunks && b < dm.nblk && col < dm.N) {
                const uint8_t* blk = w + col * col_bytes + size_t(b) * 210u;
                regs[c].ql = ld16_a2(blk + h * 64 + 16 * t);
                regs[c].qh = ld16_a2(blk + 128 + h * 32 + 16 * (t & 1));
                regs[c].sc = ld8_a2(blk + 192 + h * 8);
                regs[c].d = ld_u16(blk + 208);
            } else {
                zero(regs[c]);
            }
        }
    };

    const uint32_t n_items = dm.ntilegroups > blockIdx.x
        ? ((dm.ntilegroups - blockIdx.x + gridDim.x - 1) / gridDim.x) * passes : 0;
    Q6Regs cur[C];
    if (n_items) load(cur, blockIdx.x, 0);  // in flight while the activations are staged
    stage_q6k(x, lds4, sums, R, dm.K, dm.nchunks);
    __syncthreads();

    float acc[C * R];
#pragma unroll
    for (int i = 0; i < C * R; ++i) acc[i] = 0.f;

    for (uint32_t it = 0; it < n_items; ++it) {
        const uint32_t tg = blockIdx.x + (it / passes) * gridDim.x, pass = it % passes;
        if (it) load(cur, tg, pass);

        const uint32_t chunk = pass * dm.S + slice;
        if (chunk < dm.nchunks) {
            const float4* xl = lds4 + chunk * 512u + lane;
            const float* sm = sums + chunk * 128u + lane;
#pragma unroll
            for (int which = 0; which < 2; ++which) {
                float4 xv[R][4];
                float sx[R];
#pragma unroll
                for (int r = 0; r < R; ++r) {
#pragma unroll
                    for (int q4 = 0; q4 < 4; ++q4) xv[r][q4] = xl[r * f4_per_row + (which * 4 + q4) * 64];
                    sx[r] = -32.f * sm[r * dm.nchunks * 128u + which * 64];  // sum (q-32) x = sum q x - 32 sum x
                }
                const uint32_t hshift = which ? shift_hi : shift_lo;
#pragma unroll
                for (int c = 0; c < C; ++c) {
                    const uint32_t ql[4] = {cur[c].ql.x, cur[c].ql.y, cur[c].ql.z, cur[c].ql.w};
                    const uint32_t qh[4] = {cur[c].qh.x, cur[c].qh.y, cur[c].qh.z, cur[c].qh.w};
                    uint32_t v[4];
#pragma unroll
                    for (int k = 0; k < 4; ++k) {
                        const uint32_t nib = which ? ((ql[k] >> 4) & 0x0F0F0F0Fu) : (ql[k] & 0x0F0F0F0Fu);
                        v[k] = nib | (((qh[k] >> hshift) & 0x03030303u) << 4);
                    }
                    float p[R];
#pragma unroll
                    for (int r = 0; r < R; ++r) p[r] = sx[r];
                    dot16<R>(v, xv, p);
                    const uint32_t scw = which ? cur[c].sc.y : cur[c].sc.x;
                    const float sf = h2f(cur[c].d) * static_cast<float>(static_cast<int>(static_cast<int8_t>(scw >> (8 * t))));
#pragma unroll
                    for (int r = 0; r < R; ++r) acc[c * R + r] = fmaf(sf, p[r], acc[c * R + r]);
                }
            }
        }

        if (pass + 1 == passes) {
            wave_reduce_multi<C * R>(acc, lane);
            constexpr int shift = reduce_multi_shift<C * R>();
            const uint32_t idx = lane >> shift;
            const bool owner = (lane & ((1 << shift) - 1)) == 0;
            if (dm.S == 1) {
                const uint32_t col = (tg * dm.T + tile) * C + idx / R;
                if (owner && col < dm.N) y[size_t(idx % R) * dm.N + col] = acc[0];
            } else {
                float* buf = red + ((it / passes) & 1u) * (dm.S * dm.T * C * R);
                if (owner) buf[(slice * dm.T + tile) * (C * R) + idx] = acc[0];
                __syncthreads();
                if (threadIdx.x < dm.T * C * R) {
                    const uint32_t tl = threadIdx.x / (C * R), id = threadIdx.x % (C * R);
                    float total = 0.f;
                    for (uint32_t s = 0; s < dm.S; ++s) total += buf[(s * dm.T + tl) * (C * R) + id];
                    const uint32_t col = (tg * dm.T + tl) * C + id / R;
                    if (col < dm.N) y[size_t(id % R) * dm.N + col] = total;
                }
            }
#pragma unroll
            for (int i = 0; i < C * R; ++i) acc[i] = 0.f;
        }
    }
}

// ---------------------------------------------------------------------------------
// Q8_0: one lane per 34-byte block; a wave owns CT consecutive columns (a contiguous
// byte range), block partials go to LDS and each column is summed in block order.
// Activations sit in LDS with a 4-float pad per 32 so that lanes reading different
// blocks hit different banks.
// ---------------------------------------------------------------------------------
template <int R>
__global__ void __launch_bounds__(256)
gemv_q80_kernel(const uint8_t* __restrict__ w, const float* __restrict__ x, float* __restrict__ y,
                uint32_t K, uint32_t N, uint32_t nblk, uint32_t CT, uint32_t ntiles) {
    extern __shared__ float4 lds4[];
    float* xs = reinterpret_cast<float*>(lds4);                    // [R][nblk*36]
    float* part = xs + R * nblk * 36u;                              // [waves][R][CT*nblk]
    const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6, nw = blockDim.x >> 6;
    for (uint32_t f = threadIdx.x; f < R * (K / 4); f += blockDim.x) {
        const uint32_t r = f / (K / 4), k4 = f - r * (K / 4);
        const float4 v = ldf4_a4(x + size_t(r) * K + k4 * 4);
        *reinterpret_cast<float4*>(xs + r * nblk * 36u + (k4 >> 3) * 36u + (k4 & 7u) * 4u) = v;
    }
    __syncthreads();
    float* mypart = part + wv * R * CT * nblk;
    const uint32_t units = CT * nblk;
    for (uint32_t tile = blockIdx.x * nw + wv; tile < ntiles; tile += gridDim.x * nw) {
        const uint32_t col0 = tile * CT;
        const uint32_t valid_units = (col0 + CT <= N ? CT : N - col0) * nblk;
        const uint8_t* base = w + size_t(col0) * nblk * 34u;
        for (uint32_t u = lane; u < units; u += 64) {
            float p[R];
#pragma unroll
            for (int r = 0; r < R; ++r) p[r] = 0.f;
            if (u < valid_units) {
                const uint8_t* blk = base + size_t(u) * 34u;
                const float d = h2f(ld_u16(blk));
                const uint4 qa = ld16_a2(blk + 2), qb = ld16_a2(blk + 18);
                const uint32_t q[8] = {qa.x, qa.y, qa.z, qa.w, qb.x, qb.y, qb.z, qb.w};
                const uint32_t b = u % nblk;
#pragma unroll
                for (int k = 0; k < 8; ++k) {
                    const float f0 = sb0(q[k]), f1 = sb1(q[k]), f2 = sb2(q[k]), f3 = sb3(q[k]);
#pragma unroll
                    for (int r = 0; r < R; ++r) {
                        const float4 xv = *reinterpret_cast<const float4*>(xs + r * nblk * 36u + b * 36u + k * 4);
                        p[r] = fmaf(f0, xv.x, p[r]);
                        p[r] = fmaf(f1, xv.y, p[r]);
                        p[r] = fmaf(f2, xv.z, p[r]);
                        p[r] = fmaf(f3, xv.w, p[r]);
                    }
                }
#pragma unroll
                for (int r = 0; r < R; ++r) p[r] *= d;
            }
#pragma unroll
            for (int r = 0; r < R; ++r) mypart[r * units + u] = p[r];
        }
        // wave-local LDS hand-off: every lane of the wave has stored before any lane reads
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        for (uint32_t o = lane; o < CT * R; o += 64) {
            const uint32_t c = o / R, r = o % R;
            if (col0 + c < N) {
                float total = 0.f;
                for (uint32_t b = 0; b < nblk; ++b) total += mypart[r * units + c * nblk + b];
                y[size_t(r) * N + col0 + c] = total;
            }
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    }
}

// ---------------------------------------------------------------------------------
// Host side
// ---------------------------------------------------------------------------------
constexpr size_t kMaxLds = 160 * 1024;
int g_cu_count = 256;

template <typename Kernel>
int raise_lds_limit(Kernel kernel) {
    return hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                               hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(kMaxLds)) == hipSuccess
        ? 0 : -1;
}

struct KPlan { GemvDims dm; uint32_t C, grid, threads; size_t lds; };

// Chooses the slice/tile split: enough waves to fill 256 CUs, k-slices so that a wave
// needs few passes, and a persistent grid when there are far more tiles than CUs.
KPlan plan_kquant(uint32_t rows, uint32_t K, uint32_t N, uint32_t blocks_per_chunk,
                  uint32_t floats_per_chunk_row, uint32_t sums_per_chunk_row) {
    KPlan p {};
    GemvDims& dm = p.dm;
    dm.K = K; dm.N = N; dm.nblk = K / 256;
    dm.nchunks = (dm.nblk + blocks_per_chunk - 1) / blocks_per_chunk;
    dm.S = dm.nchunks < 4 ? dm.nchunks : 4;
    // columns per wave: 4 when that still yields >= 2048 waves, else 2
    p.C = (uint64_t(N) * dm.S / 4 >= 2048) ? 4 : 2;
    dm.T = dm.S >= 4 ? 4 : (dm.S == 2 ? 4 : 4);
    dm.ntilegroups = (N + dm.T * p.C - 1) / (dm.T * p.C);
    p.threads = dm.S * dm.T * 64;
    p.lds = size_t(rows) * dm.nchunks * (floats_per_chunk_row + sums_per_chunk_row) * 4
        + size_t(2) * dm.S * dm.T * p.C * rows * 4;
    const uint32_t max_grid = g_cu_count * 8;
    p.grid = dm.ntilegroups < max_grid ? dm.ntilegroups : max_grid;
    return p;
}

template <int R>
int launch_q4k(hipStream_t s, const uint8_t* w, const float* x, float* y, uint32_t K, uint32_t N) {
    const KPlan p = plan_kquant(R, K, N, 16, 4096, 256);
    if (p.lds > kMaxLds) return fail(GUFFIN_E_CAPACITY, "gemv_q4k: activation rows do not fit in LDS");
    if (p.C == 4) launch((gemv_q4k_kernel<R, 4>), dim3(p.grid), dim3(p.threads), p.lds, s, w, x, y, p.dm);
    else launch((gemv_q4k_kernel<R, 2>), dim3(p.grid), dim3(p.threads), p.lds, s, w, x, y, p.dm);
    return check_launch("gemv_q4k");
}

template <int R>
int launch_q6k(hipStream_t s, const uint8_t* w, const float* x, float* y, uint32_t K, uint32_t N) {
    const KPlan p = plan_kquant(R, K, N, 8, 2048, 128);
    if (p.lds > kMaxLds) return fail(GUFFIN_E_CAPACITY, "gemv_q6k: activation rows do not fit in LDS");
    if (p.C == 4) launch((gemv_q6k_kernel<R, 4>), dim3(p.grid), dim3(p.threads), p.lds, s, w, x, y, p.dm);
    else launch((gemv_q6k_kernel<R, 2>), dim3(p.grid), dim3(p.threads), p.lds, s, w, x, y, p.dm);
    return check_launch("gemv_q6k");
}

template <int R>
int launch_q80(hipStream_t s, const uint8_t* w, const float* x, float* y, uint32_t K, uint32_t N) {
    const uint32_t nblk = K / 32;
    // a wave covers about 256 blocks per tile (4 rounds of 64 lanes)
    uint32_t CT = 256 / nblk;
    if (CT == 0) CT = 1;
    if (CT > 16) CT = 16;
    const uint32_t ntiles = (N + CT - 1) / CT;
    const uint32_t waves = 4;
    const size_t lds = (size_t(R) * nblk * 36 + size_t(waves) * R * CT * nblk) * 4;
    if (lds > kMaxLds) return fail(GUFFIN_E_CAPACITY, "gemv_q80: activation rows do not fit in LDS");
    uint32_t grid = (ntiles + waves - 1) / waves;
    const uint32_t max_grid = g_cu_count * 8;
    if (grid > max_grid) grid = max_grid;
    launch((gemv_q80_kernel<R>), dim3(grid), dim3(waves * 64), lds, s, w, x, y, K, N, nblk, CT, ntiles);
    return check_launch("gemv_q80");
}

}  // namespace

int gemv_init(int cu_count) {
    g_cu_count = cu_count > 0 ? cu_count : 256;
    int rc = 0;
    rc |= raise_lds_limit(gemv_q4k_kernel<1, 2>); rc |= raise_lds_limit(gemv_q4k_kernel<1, 4>);
    rc |= raise_lds_limit(gemv_q4k_kernel<2, 2>); rc |= raise_lds_limit(gemv_q4k_kernel<2, 4>);
    rc |= raise_lds_limit(gemv_q6k_kernel<1, 2>); rc |= raise_lds_limit(gemv_q6k_kernel<1, 4>);
    rc |= raise_lds_limit(gemv_q6k_kernel<2, 2>); rc |= raise_lds_limit(gemv_q6k_kernel<2, 4>);
    rc |= raise_lds_limit(gemv_q80_kernel<1>); rc |= raise_lds_limit(gemv_q80_kernel<2>);
    return rc;
}

}  // namespace guffin

using namespace guffin;

extern "C" int guffin_hip_dequant(void* stream, int dtype, const void* blocks, uint64_t n_blocks, float* out) {
    if (!blocks || !out) return fail(GUFFIN_E_ARG, "dequant: null pointer");
    if (dtype < GUFFIN_Q8_0 || dtype > GUFFIN_Q6_K) return fail(GUFFIN_E_ARG, "dequant: unknown dtype");
    if (reinterpret_cast<uintptr_t>(blocks) & 1u) return fail(GUFFIN_E_ALIGN, "dequant: blocks must be 2-byte aligned");
    if (n_blocks == 0) return GUFFIN_OK;
    const uint64_t n = n_blocks * (dtype == GUFFIN_Q8_0 ? 32u : 256u);
    const uint32_t grid = static_cast<uint32_t>(n / 256 < 65535 ? (n + 255) / 256 : 65535);
    const uint8_t* b = static_cast<const uint8_t*>(blocks);
    hipStream_t s = as_stream(stream);
    if (dtype == GUFFIN_Q8_0) launch(dequant_kernel<GUFFIN_Q8_0>, dim3(grid), dim3(256), 0, s, b, n, out);
    else if (dtype == GUFFIN_Q4_K) launch(dequant_kernel<GUFFIN_Q4_K>, dim3(grid), dim3(256), 0, s, b, n, out);
    else launch(dequant_kernel<GUFFIN_Q6_K>, dim3(grid), dim3(256), 0, s, b, n, out);
    return check_launch("dequant");
}

extern "C" int guffin_hip_gemv(void* stream, int dtype, const void* w, const float* x, float* y,
                               uint32_t rows, uint32_t K, uint32_t N) {
    if (!w || !x || !y) return fail(GUFFIN_E_ARG, "gemv: null pointer");
    if (dtype < GUFFIN_Q8_0 || dtype > GUFFIN_Q6_K) return fail(GUFFIN_E_ARG, "gemv: unknown dtype");
    const uint32_t be = dtype == GUFFIN_Q8_0 ? 32u : 256u;
    if (rows == 0 || rows > 8) return fail(GUFFIN_E_SHAPE, "gemv: rows must be in [1, 8]");
    if (K == 0 || N == 0 || K % be != 0) return fail(GUFFIN_E_SHAPE, "gemv: K must be a positive multiple of the block size");
    const uintptr_t wa = reinterpret_cast<uintptr_t>(w);
    if (dtype == GUFFIN_Q4_K ? (wa & 3u) : (wa & 1u)) return fail(GUFFIN_E_ALIGN, "gemv: weight pointer under-aligned for its block stream");
    if ((reinterpret_cast<uintptr_t>(x) & 3u) || (reinterpret_cast<uintptr_t>(y) & 3u)) return fail(GUFFIN_E_ALIGN, "gemv: fp32 pointers must be 4-byte aligned");
    const uint8_t* wb = static_cast<const uint8_t*>(w);
    hipStream_t s = as_stream(stream);
    // rows are processed in pairs; every row runs the same arithmetic in either width
    for (uint32_t r0 = 0; r0 < rows; r0 += 2) {
        const bool two = r0 + 1 < rows;
        const float* xr = x + size_t(r0) * K;
        float* yr = y + size_t(r0) * N;
        int rc;
        // a 2-row launch writes rows r0, r0+1 of y, which are contiguous [2, N]
        if (dtype == GUFFIN_Q4_K) rc = two ? launch_q4k<2>(s, wb, xr, yr, K, N) : launch_q4k<1>(s, wb, xr, yr, K, N);
        else if (dtype == GUFFIN_Q6_K) rc = two ? launch_q6k<2>(s, wb, xr, yr, K, N) : launch_q6k<1>(s, wb, xr, yr, K, N);
        else rc = two ? launch_q80<2>(s, wb, xr, yr, K, N) : launch_q80<1>(s, wb, xr, yr, K, N);
        if (rc) return rc;
    }
    return GUFFIN_OK;
}

extern "C" int guffin_hip_gemv_q4k(void* stream, const void* w, const float* x, float* y, uint32_t rows, uint32_t K, uint32_t N) {
    return guffin_hip_gemv(stream, GUFFIN_Q4_K, w, x, y, rows, K, N);
}
extern "C" int guffin_hip_gemv_q6k(void* stream, const void* w, const float* x, float* y, uint32_t rows, uint32_t K, uint32_t N) {
    return guffin_hip_gemv(stream, GUFFIN_Q6_K, w, x, y, rows, K, N);
}
extern "C" int guffin_hip_gemv_q80(void* stream, const void* w, const float* x, float* y, uint32_t rows, uint32_t K, uint32_t N) {
    return guffin_hip_gemv(stream, GUFFIN_Q8_0, w, x, y, rows, K, N);
}
