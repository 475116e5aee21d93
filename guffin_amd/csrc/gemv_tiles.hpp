// Wave-tile operand code shared by the kernels that stream repacked weights: tile registers, the
// matrix-core product of one tile with the activation image, and the walk over a run of blocks.
// The layout of a tile and of the activation receipt is described in gemv_packed.hip / receipt.hpp.
#pragma once
#include "common.hpp"
#include "receipt.hpp"

namespace guffin {
namespace {

typedef _Float16 half2_t __attribute__((ext_vector_type(2)));

constexpr uint32_t kTileCols = 64;

__host__ __device__ constexpr uint32_t block_bytes(int dtype) {
    return dtype == GUFFIN_Q8_0 ? 34u : dtype == GUFFIN_Q4_K ? 144u : 210u;
}
__host__ __device__ constexpr uint32_t block_elems(int dtype) { return dtype == GUFFIN_Q8_0 ? 32u : 256u; }

// bytes {0,2} and {1,3} of v as 16-bit fields
__device__ __forceinline__ uint32_t even_bytes(uint32_t v) { return __builtin_amdgcn_perm(0u, v, 0x0c020c00u); }
__device__ __forceinline__ uint32_t odd_bytes(uint32_t v) { return __builtin_amdgcn_perm(0u, v, 0x0c030c01u); }


// =======================================================================================
// Q4_K
// =======================================================================================
// Matrix-core path.  A wave covers 64 columns x one 256-element block as four column groups
// of 16; lane (j = lane % 16, s = lane / 16) holds, for every column group, the bytes 8s..8s+7
// of each 32-byte quant chunk of column 16*cg + j, and owns column `lane` for the scales and
// the result.  For each 32-element sub-block and column group one v_mfma_f32_16x16x32_f16
// multiplies the activation image (A: 16 rows = the 4 variants hi/lo x row, repeated; lane
// (i, s) holds variant i % 4, k-slice s) with the nibbles as fp16 subnormals (B: q * 2^-24,
// or 16q * 2^-24 for high nibbles, both exact).  Every lane group then holds the four variant
// sums of the 16 columns of that group; lane group g keeps those of column group g and scales
// them by d*sc of its own column in fp32.  The -dmin*m term uses the 32-sums.
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef float float4_t __attribute__((ext_vector_type(4)));

// Weight bytes are used once: streaming (non-temporal) loads keep the caches for the activation
// image, which every wave re-reads.
typedef uint32_t uint4_t __attribute__((ext_vector_type(4)));
__device__ __forceinline__ uint4 stream_load(const uint8_t* p) {
    const uint4_t v = __builtin_nontemporal_load(reinterpret_cast<const uint4_t*>(p));
    return make_uint4(v.x, v.y, v.z, v.w);
}

struct Q4Tile { uint4 q[8]; uint4 hdr; };

// Loads come back in the order of their requests: the scales and the pieces of the first four sub-blocks go
// first, so that their products run while the other half of the tile is still on its way.
__device__ __forceinline__ void load_tile(Q4Tile& t, const uint8_t* p) {
    t.hdr = stream_load(p + 8192);
#pragma unroll
    for (int i = 0; i < 8; i += 2) t.q[i] = stream_load(p + 1024 * i);
#pragma unroll
    for (int i = 1; i < 8; i += 2) t.q[i] = stream_load(p + 1024 * i);
}

__device__ __forceinline__ half8_t as_half8(uint32_t a, uint32_t b, uint32_t c, uint32_t d) {
    return __builtin_bit_cast(half8_t, make_uint4(a, b, c, d));
}

// image: this block's 8 groups of the activation image, already offset for this lane;
// mult / xs32: this block's 8 multipliers / 32-sums of row 0 (rows `per_mult` / `per_row` apart)
struct Q4Operand { half8_t a[8]; };
__device__ __forceinline__ void load_operand(Q4Operand& o, const uint8_t* __restrict__ image) {
#pragma unroll
    for (int g = 0; g < 8; ++g) o.a[g] = __builtin_bit_cast(half8_t, *reinterpret_cast<const uint4*>(image + 256 * g));
}

template <int R>
__device__ __forceinline__ void compute_tile(const Q4Tile& t, const Q4Operand& op,
                                             const float* __restrict__ mult, uint32_t per_mult,
                                             const float* __restrict__ xs32, uint32_t per_row,
                                             uint32_t lane_group, float (&acc)[R]) {
    const half8_t (&a)[8] = op.a;
    const float d = h2f(t.hdr.x & 0xFFFFu), dmin = h2f(t.hdr.x >> 16);
    const uint32_t s0 = t.hdr.y, s1 = t.hdr.z, s2 = t.hdr.w;
    const uint32_t sc_a = s0 & 0x3F3F3F3Fu, mn_a = s1 & 0x3F3F3F3Fu;
    const uint32_t sc_b = (s2 & 0x0F0F0F0Fu) | ((s0 >> 2) & 0x30303030u);
    const uint32_t mn_b = ((s2 >> 4) & 0x0F0F0F0Fu) | ((s1 >> 2) & 0x30303030u);
    const float d_q = d * 0.0625f;  // nibbles enter as 16 q
    float mt[R];
#pragma unroll
    for (int r = 0; r < R; ++r) mt[r] = 0.f;
    const float4_t zero = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int ch = 0; ch < 4; ++ch) {  // 32-byte chunk: sub-blocks 2ch (low nibbles) and 2ch+1 (high)
        float4_t lo = zero, hi = zero;
#pragma unroll
        for (int cg = 0; cg < 4; ++cg) {
            const uint4 piece = t.q[2 * cg + (ch >> 1)];
            const uint32_t w0 = (ch & 1) ? piece.z : piece.x, w1 = (ch & 1) ? piece.w : piece.y;
            // every nibble sits in bits 4-7 of its half (16 q as a bit pattern below 2048, which reads as
            // 16 q 2^-24): the matrix instruction does not normalise such operands, so a pattern with leading
            // zeros loses that many bits of every product it meets once the products of a sum are aligned.
            // (In bits 0-3 the low nibbles cost up to 200 eps of a group's sum|q x| on activations with a wide
            // range inside the group; bits 6-9 would gain two more bits for one more shift per word.)
            constexpr uint32_t M = 0x00F000F0u;
            const half8_t blo = as_half8((w0 << 4) & M, (w0 >> 4) & M, (w1 << 4) & M, (w1 >> 4) & M);
            const half8_t bhi = as_half8(w0 & M, (w0 >> 8) & M, w1 & M, (w1 >> 8) & M);
            const float4_t dlo = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[2 * ch], blo, zero, 0, 0, 0);
            const float4_t dhi = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[2 * ch + 1], bhi, zero, 0, 0, 0);
            if (lane_group == uint32_t(cg)) { lo = dlo; hi = dhi; }
        }
        const uint32_t scw = ch < 2 ? sc_a : sc_b, mnw = ch < 2 ? mn_a : mn_b;
        const float sc_lo = (ch & 1) ? ub2(scw) : ub0(scw), sc_hi = (ch & 1) ? ub3(scw) : ub1(scw);
        const float mn_lo = (ch & 1) ? ub2(mnw) : ub0(mnw), mn_hi = (ch & 1) ? ub3(mnw) : ub1(mnw);
        const float f_lo = d_q * sc_lo, f_hi = d_q * sc_hi;
#pragma unroll
        for (int r = 0; r < R; ++r) {
            const float m_lo = mult[r * per_mult + 2 * ch], m_hi = mult[r * per_mult + 2 * ch + 1];
            acc[r] = fmaf(f_lo * m_lo, lo[2 * r] + lo[2 * r + 1], acc[r]);
            acc[r] = fmaf(f_hi * m_hi, hi[2 * r] + hi[2 * r + 1], acc[r]);
            mt[r] = fmaf(mn_lo, xs32[r * per_row + 2 * ch], mt[r]);
            mt[r] = fmaf(mn_hi, xs32[r * per_row + 2 * ch + 1], mt[r]);
        }
    }
#pragma unroll
    for (int r = 0; r < R; ++r) acc[r] = fmaf(-dmin, mt[r], acc[r]);
}

// =======================================================================================
// Q6_K
// =======================================================================================
// Same operand scheme as Q4_K with two differences.  A scale covers 16 elements, so the A rows
// of one 32-element MFMA are split: rows 0-3 carry the variants with the second 16 elements
// zeroed, rows 4-7 the other half (rows 8-15 repeat them); lane group g then holds the sums of
// k-half g % 2.  Lane (j, g) owns columns 32*(g/2) + j and + 16 for that k-half, keeps column
// groups 2*(g/2) and 2*(g/2)+1, and the two k-halves are added across lanes at the end.
struct Q6Tile { uint4 ql[8]; uint4 qh[4]; uint4 sc[2]; uint32_t d[2]; };

// EARLY: the request order of the Q4_K tile (what the first 128 elements need, then the low nibbles of the other
// half).  It pays where the operand groups are requested ahead of the tile; the one-tile-at-a-time walk reads
// them behind the tile, where a group's wait covers every earlier request anyway, and is slower with it.
template <bool EARLY>
__device__ __forceinline__ void load_tile(Q6Tile& t, const uint8_t* p, uint32_t lane) {
#pragma unroll
    for (int i = 0; i < 8; i += EARLY ? 2 : 1) t.ql[i] = stream_load(p + 1024 * i);
#pragma unroll
    for (int i = 0; i < 4; ++i) t.qh[i] = stream_load(p + 8192 + 1024 * i);
    const uint8_t* base = p - lane * 16;
    const uint32_t col = 32u * (lane >> 5) + (lane & 15u);
#pragma unroll
    for (int c = 0; c < 2; ++c) {
        t.sc[c] = *reinterpret_cast<const uint4*>(base + 12288 + (col + 16 * c) * 16);
        t.d[c] = *reinterpret_cast<const uint16_t*>(base + 13312 + (col + 16 * c) * 2);
    }
    if constexpr (EARLY) {
#pragma unroll
        for (int i = 1; i < 8; i += 2) t.ql[i] = stream_load(p + 1024 * i);
    }
}

__device__ __forceinline__ float sbyte(uint32_t w, int i) {
    return i == 0 ? sb0(w) : i == 1 ? sb1(w) : i == 2 ? sb2(w) : sb3(w);
}

template <int R>
__device__ __forceinline__ void compute_tile(const Q6Tile& t, const uint8_t* __restrict__ image, uint32_t keep,
                                             const float* __restrict__ mult, uint32_t per_mult,
                                             const float* __restrict__ xs16, uint32_t per_row,
                                             uint32_t lane, float (&acc)[2][R]) {
    const uint32_t khalf = (lane >> 4) & 1u;
    const bool upper = lane >= 32;
    const float4_t zero = {0.f, 0.f, 0.f, 0.f};
    float part[2][R], off[2][R];
#pragma unroll
    for (int c = 0; c < 2; ++c)
#pragma unroll
        for (int r = 0; r < R; ++r) { part[c][r] = 0.f; off[c][r] = 0.f; }
#pragma unroll
    for (int g = 0; g < 8; ++g) {  // 32-element group: half n, quadrant qd
        const int n = g >> 2, qd = g & 3;
        uint4 av = *reinterpret_cast<const uint4*>(image + 256 * g);
        av.x &= keep; av.y &= keep; av.z &= keep; av.w &= keep;
        const half8_t a = __builtin_bit_cast(half8_t, av);
        float4_t D[4];
#pragma unroll
        for (int cg = 0; cg < 4; ++cg) {
            const uint4 lq = t.ql[2 * cg + n], hq = t.qh[cg];
            const uint32_t w0 = (qd & 1) ? lq.z : lq.x, w1 = (qd & 1) ? lq.w : lq.y;
            const uint32_t h0 = n ? hq.z : hq.x, h1 = n ? hq.w : hq.y;
            const int ls = qd >= 2 ? 4 : 0;  // nibble shift
            uint32_t b[4];
#pragma unroll
            for (int k = 0; k < 2; ++k) {
                const uint32_t w = k ? w1 : w0, h = k ? h1 : h0;
                // the 6-bit quant sits in bits 4-9 of its half (16 q as a bit pattern: see the Q4_K tile)
                const uint32_t lo0 = (ls ? w : w << 4) & 0x00F000F0u, lo1 = (w >> (ls + 4)) & 0x00F000F0u;
                // 2-bit field of quadrant qd moved to bits 8-9 of each half
                const uint32_t hs0 = h << (8 - 2 * qd);
                const uint32_t hs1 = qd == 0 ? h : h >> (2 * qd);
                b[2 * k] = (hs0 & 0x03000300u) | lo0;
                b[2 * k + 1] = (hs1 & 0x03000300u) | lo1;
            }
            D[cg] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, as_half8(b[0], b[1], b[2], b[3]), zero, 0, 0, 0);
        }
        const float4_t da = upper ? D[2] : D[0], db = upper ? D[3] : D[1];
        // int8 scale of 16-element group 2g + khalf for the lane's two columns
        const int word = g >> 1;  // scales 4*word .. 4*word+3 hold groups 2g-(g&1)*2 ...
        float sc[2];
#pragma unroll
        for (int c = 0; c < 2; ++c) {
            const uint32_t wv = word == 0 ? t.sc[c].x : word == 1 ? t.sc[c].y : word == 2 ? t.sc[c].z : t.sc[c].w;
            const float s_even = sbyte(wv, 2 * (g & 1)), s_odd = sbyte(wv, 2 * (g & 1) + 1);
            sc[c] = khalf ? s_odd : s_even;
        }
#pragma unroll
        for (int r = 0; r < R; ++r) {
            const float m = mult[r * per_mult + g];
            const float s16_first = xs16[r * per_row + 2 * g], s16_second = xs16[r * per_row + 2 * g + 1];
            const float s16 = khalf ? s16_second : s16_first;
            part[0][r] = fmaf(sc[0] * m, da[2 * r] + da[2 * r + 1], part[0][r]);
            part[1][r] = fmaf(sc[1] * m, db[2 * r] + db[2 * r + 1], part[1][r]);
            off[0][r] = fmaf(sc[0], s16, off[0][r]);
            off[1][r] = fmaf(sc[1], s16, off[1][r]);
        }
    }
#pragma unroll
    for (int c = 0; c < 2; ++c) {
        const float d = h2f(t.d[c]);
#pragma unroll
        for (int r = 0; r < R; ++r) acc[c][r] = fmaf(d, fmaf(-32.0f, off[c][r], 0.0625f * part[c][r]), acc[c][r]);
    }
}

// adds the two k-halves and hands every lane the sum of its own column
template <int R>
__device__ __forceinline__ void q6_gather(const float (&acc2)[2][R], uint32_t lane, float (&acc)[R]) {
    const uint32_t src = 32u * (lane >> 5) + (lane & 15u);  // lane (j, group 2*(q/2)) holds column 16q + j as a (q even) or b
#pragma unroll
    for (int r = 0; r < R; ++r) {
        const float a = acc2[0][r] + __shfl_xor(acc2[0][r], 16, kWave);
        const float b = acc2[1][r] + __shfl_xor(acc2[1][r], 16, kWave);
        const float ga = __shfl(a, src, kWave), gb = __shfl(b, src, kWave);
        acc[r] = ((lane >> 4) & 1u) ? gb : ga;
    }
}

// =======================================================================================
// Q8_0
// =======================================================================================
// One 32-element block per MFMA and column group; the int8 quants enter biased by 128 as fp16
// subnormals, the bias comes back through the 32-sum.
struct Q8Tile { uint4 q[2]; uint32_t d; };

__device__ __forceinline__ void load_tile(Q8Tile& t, const uint8_t* p, uint32_t lane) {
    t.q[0] = stream_load(p);
    t.q[1] = stream_load(p + 1024);
    t.d = *reinterpret_cast<const uint16_t*>(p - lane * 16 + 2048 + lane * 2);
}

template <int R>
__device__ __forceinline__ void compute_tile(const Q8Tile& t, const half8_t a,
                                             const float* __restrict__ mult, uint32_t per_mult,
                                             const float* __restrict__ xs32, uint32_t per_row,
                                             uint32_t lane_group, float (&acc)[R]) {
    const float4_t zero = {0.f, 0.f, 0.f, 0.f};
    float4_t own = zero;
#pragma unroll
    for (int cg = 0; cg < 4; ++cg) {
        const uint4 piece = t.q[cg >> 1];
        const uint32_t w0 = ((cg & 1) ? piece.z : piece.x) ^ 0x80808080u, w1 = ((cg & 1) ? piece.w : piece.y) ^ 0x80808080u;
        // the biased byte sits in bits 3-10 of its half (8 (q + 128) as a bit pattern: see the Q4_K tile)
        const float4_t d4 = __builtin_amdgcn_mfma_f32_16x16x32_f16(
            a, as_half8(even_bytes(w0) << 3, odd_bytes(w0) << 3, even_bytes(w1) << 3, odd_bytes(w1) << 3), zero, 0, 0, 0);
        if (lane_group == uint32_t(cg)) own = d4;
    }
    const float d = h2f(t.d);
#pragma unroll
    for (int r = 0; r < R; ++r) {
        const float v = fmaf(0.125f * mult[r * per_mult], own[2 * r] + own[2 * r + 1], -128.0f * xs32[r * per_row]);
        acc[r] = fmaf(d, v, acc[r]);
    }
}

// =======================================================================================
// The streaming kernel: one wave = one (column tile, k-slice)
// =======================================================================================
// One wave: `count` consecutive blocks of one column tile, the first at `tiles` (its 64 x block bytes),
// against the operand blocks ob0 .. ob0 + count - 1 of the receipt `xsums` (a blob laid out for R rows
// of K activations, in global memory or in LDS); returns the per-lane column sums.
template <int DTYPE, int R, bool SINGLE = false>
__device__ __forceinline__ void run_blocks_at(const uint8_t* __restrict__ tiles, const float* __restrict__ xsums,
                                              uint32_t K, uint32_t ob0, uint32_t count, float (&acc)[R],
                                              uint32_t lane = threadIdx.x & 63) {
    constexpr uint32_t TB = kTileCols * block_bytes(DTYPE);
    const uint32_t n16 = K / 16, per_row = n16 + K / 32;
    // Q6_K consumes 16-sums (16 per block), Q4_K 32-sums (8 per block), Q8_0 one 32-sum per block
    const float* xs = DTYPE == GUFFIN_Q6_K ? xsums : xsums + n16;
    const uint8_t* tp = tiles + lane * 16;
#pragma unroll
    for (int r = 0; r < R; ++r) acc[r] = 0.f;
    const ReceiptLayout L = receipt_layout(R, K);
    const uint8_t* blob = reinterpret_cast<const uint8_t*>(xsums);
    const float* mult = reinterpret_cast<const float*>(blob + L.mult_off);
    // lane (i = lane % 16, s = lane / 16) of the A operand: variant i % 4, k-slice s
    const uint8_t* image = blob + L.image_off + (lane & 3u) * 64u + (lane >> 4) * 16u;
    const uint32_t ob1 = ob0 + count;
    if constexpr (DTYPE == GUFFIN_Q4_K) {
        // the first block's operand (a hit in the caches) is requested ahead of the weight tiles, which
        // come from HBM: behind them it would cost every wave a second trip before its first product
        Q4Tile cur, nxt;
        Q4Operand op;
        if (count) { load_operand(op, image + size_t(ob0) * 2048u); load_tile(cur, tp); }
        for (uint32_t b = ob0; b < ob1; ++b) {
            if (b + 1 < ob1) load_tile(nxt, tp + size_t(b + 1 - ob0) * TB);
            if (b != ob0) load_operand(op, image + size_t(b) * 2048u);
            compute_tile<R>(cur, op, mult + b * 8u, K / 32, xs + b * 8u, per_row, lane >> 4, acc);
            cur = nxt;
        }
    } else if constexpr (DTYPE == GUFFIN_Q6_K) {
        // A rows 0-3 / 8-11 see the first 16 elements of a group, rows 4-7 / 12-15 the second 16
        const uint32_t keep = (((lane & 15u) >> 2) & 1u) == (lane >> 5) ? 0xFFFFFFFFu : 0u;
        float acc2[2][R];
#pragma unroll
        for (int c = 0; c < 2; ++c)
#pragma unroll
            for (int r = 0; r < R; ++r) acc2[c][r] = 0.f;
        // (this tile and its operand together do not fit the registers: the operand is read group by group)
        if constexpr (SINGLE) {  // one tile in registers at a time: 16 waves fit a workgroup
            for (uint32_t b = ob0; b < ob1; ++b) {
                Q6Tile cur;
                load_tile<false>(cur, tp + size_t(b - ob0) * TB, lane);
                compute_tile<R>(cur, image + size_t(b) * 2048u, keep, mult + b * 8u, K / 32, xs + b * 16u, per_row, lane, acc2);
            }
        } else {
            Q6Tile cur, nxt;
            if (count) load_tile<true>(cur, tp, lane);
            for (uint32_t b = ob0; b < ob1; ++b) {
                if (b + 1 < ob1) load_tile<true>(nxt, tp + size_t(b + 1 - ob0) * TB, lane);
                compute_tile<R>(cur, image + size_t(b) * 2048u, keep, mult + b * 8u, K / 32, xs + b * 16u, per_row, lane, acc2);
                cur = nxt;
            }
        }
        q6_gather<R>(acc2, lane, acc);
    } else {
        Q8Tile cur, nxt;
        auto operand = [&](uint32_t b) { return __builtin_bit_cast(half8_t, *reinterpret_cast<const uint4*>(image + size_t(b) * 256u)); };
        half8_t a = {}, an = {};
        if (count) { a = operand(ob0); load_tile(cur, tp, lane); }
        for (uint32_t b = ob0; b < ob1; ++b) {
            if (b + 1 < ob1) { an = operand(b + 1); load_tile(nxt, tp + size_t(b + 1 - ob0) * TB, lane); }
            compute_tile<R>(cur, a, mult + b, K / 32, xs + b, per_row, lane >> 4, acc);
            cur = nxt;
            a = an;
        }
    }
}

// The first two Q8_0 tiles of a wave's run, requested ahead of time (before a wait that the operand needs
// and the weights do not), and the run itself starting from them.
struct Q8Ahead { Q8Tile t[2]; };

__device__ __forceinline__ void load_ahead(Q8Ahead& ahead, const uint8_t* __restrict__ tiles, uint32_t count, uint32_t lane) {
    constexpr uint32_t TB = kTileCols * block_bytes(GUFFIN_Q8_0);
    const uint8_t* tp = tiles + lane * 16;
    ahead.t[0] = Q8Tile{};
    ahead.t[1] = Q8Tile{};
    if (count > 0) load_tile(ahead.t[0], tp, lane);
    if (count > 1) load_tile(ahead.t[1], tp + TB, lane);
}

template <int R>
__device__ __forceinline__ void run_blocks_ahead(const Q8Ahead& ahead, const uint8_t* __restrict__ tiles,
                                                 const float* __restrict__ xsums, uint32_t K, uint32_t ob0, uint32_t count,
                                                 float (&acc)[R], uint32_t lane = threadIdx.x & 63) {
    constexpr uint32_t TB = kTileCols * block_bytes(GUFFIN_Q8_0);
    const uint32_t n16 = K / 16, per_row = n16 + K / 32;
    const float* xs = xsums + n16;
    const uint8_t* tp = tiles + lane * 16;
#pragma unroll
    for (int r = 0; r < R; ++r) acc[r] = 0.f;
    const ReceiptLayout L = receipt_layout(R, K);
    const uint8_t* blob = reinterpret_cast<const uint8_t*>(xsums);
    const float* mult = reinterpret_cast<const float*>(blob + L.mult_off);
    const uint8_t* image = blob + L.image_off + (lane & 3u) * 64u + (lane >> 4) * 16u;
    const uint32_t ob1 = ob0 + count;
    auto operand = [&](uint32_t b) { return __builtin_bit_cast(half8_t, *reinterpret_cast<const uint4*>(image + size_t(b) * 256u)); };
    Q8Tile cur = ahead.t[0], nxt = ahead.t[1], far = Q8Tile{};
    half8_t a = {}, an = {};
    if (count) a = operand(ob0);
    for (uint32_t b = ob0; b < ob1; ++b) {
        if (b + 1 < ob1) an = operand(b + 1);
        if (b + 2 < ob1) load_tile(far, tp + size_t(b + 2 - ob0) * TB, lane);
        compute_tile<R>(cur, a, mult + b, K / 32, xs + b, per_row, lane >> 4, acc);
        cur = nxt;
        nxt = far;
        a = an;
    }
}

// One wave: blocks [b0, b1) of column tile `ct` of a whole matrix whose operand is the receipt of its K inputs.
template <int DTYPE, int R, bool SINGLE = false>
__device__ __forceinline__ void run_blocks(const uint8_t* __restrict__ wt, const float* __restrict__ x,
                                           const float* __restrict__ xsums, uint32_t K, uint32_t nblk,
                                           uint32_t ct, uint32_t b0, uint32_t b1, float (&acc)[R]) {
    constexpr uint32_t TB = kTileCols * block_bytes(DTYPE);
    run_blocks_at<DTYPE, R, SINGLE>(wt + (size_t(ct) * nblk + b0) * TB, xsums, K, b0, b1 > b0 ? b1 - b0 : 0u, acc);
}

}  // namespace
}  // namespace guffin
