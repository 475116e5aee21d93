// Activation receipt: what every producer of a GEMV input leaves next to the fp32 rows.
//
//   sums   float [rows][K/16 + K/32]   sums of 16 and of 32 consecutive activations (the
//                                      reference's producers emit the same kind of receipt for
//                                      its Q4_K kernels, metal_kernels.mm:16-27)
//   mult   float [rows][K/32]          per 32-group multiplier 2^(E+24) of the image below
//   image  half  [K/32][4][32]         matrix-core operand: variant 2r = hi, 2r+1 = lo of row r,
//                                      hi + lo = x * 2^-E to 22 bits, E chosen per 32-group so that
//                                      |x| 2^-E < 2^15; inside a group the 8 halves of k-slice s
//                                      (elements 8s..8s+7) sit at 8s + {0,2,1,3,4,6,5,7}, the
//                                      order in which nibble pairs fall out of a weight dword
// All three start on 256-byte boundaries of one blob; K must be a multiple of 32.
#pragma once
#include "common.hpp"

namespace guffin {

// gelu_tanh(g) * u with the reference's operation order (src/tensor/ops/elementwise.cpp:79-94, 50-63)
__device__ __forceinline__ float geglu_value(float g, float u) {
    constexpr float k0 = 0.7978845608028654f, k1 = 0.044715f;
    const float inner = __fmul_rn(k0, __fadd_rn(g, __fmul_rn(__fmul_rn(__fmul_rn(k1, g), g), g)));
    const float t = tanhf(inner);
    return __fmul_rn(__fmul_rn(__fmul_rn(0.5f, g), __fadd_rn(1.0f, t)), u);
}

struct ReceiptLayout { size_t mult_off, image_off, bytes; };

__host__ __device__ inline ReceiptLayout receipt_layout(uint32_t rows, uint32_t K) {
    const size_t sums = size_t(rows) * (K / 16 + K / 32) * 4;
    const size_t mult = (sums + 255) & ~size_t{255};
    const size_t image = (mult + size_t(rows) * (K / 32) * 4 + 255) & ~size_t{255};
    return {mult, image, image + size_t(K / 32) * 256};
}

// One item: the 8 consecutive activations v[] of row r, elements k0 + 8t .. k0 + 8t + 7.  The four
// lanes of a 32-group (t % 4 = 0..3 in consecutive lanes) must run it together.
__device__ __forceinline__ void emit_receipt_values(const float (&v)[8], uint32_t k0, uint32_t t, uint32_t r, uint32_t rows,
                                                    uint32_t K, void* blob) {
    const ReceiptLayout L = receipt_layout(rows, K);
    const uint32_t n16 = K / 16;
    float* sums = static_cast<float*>(blob) + size_t(r) * (n16 + K / 32);
    float* mult = reinterpret_cast<float*>(static_cast<uint8_t*>(blob) + L.mult_off) + size_t(r) * (K / 32);
    uint8_t* image = static_cast<uint8_t*>(blob) + L.image_off;
    {
        const uint32_t g = (k0 >> 5) + (t >> 2), s = t & 3;
        float sum = v[0], m = fabsf(v[0]);
#pragma unroll
        for (int i = 1; i < 8; ++i) { sum += v[i]; m = fmaxf(m, fabsf(v[i])); }
        // the four lanes of the group exchange inside their quad (lane ^ 1, then lane ^ 2)
        m = fmaxf(m, lane_cross<0xB1>(m));
        m = fmaxf(m, lane_cross<0x4E>(m));
        const float sum16 = sum + lane_cross<0xB1>(sum);
        const float sum32 = sum16 + lane_cross<0x4E>(sum16);
        // biased exponent of the group maximum, clamped so that both scale factors are normal floats
        uint32_t eb = __float_as_uint(m) >> 23;
        eb = eb < 14u ? 14u : eb > 244u ? 244u : eb;
        const float inv = __uint_as_float((268u - eb) << 23);      // 2^-E, E = eb - 141: |x| 2^-E < 2^15
        if (s == 0) { mult[g] = __uint_as_float((eb + 10u) << 23); sums[n16 + g] = sum32; }  // 2^(E+24)
        if ((s & 1u) == 0) sums[2 * g + (s >> 1)] = sum16;
        uint32_t hi[4], lo[4];
        constexpr int order[8] = {0, 2, 1, 3, 4, 6, 5, 7};
#pragma unroll
        for (int p = 0; p < 4; ++p) {
            uint32_t hw = 0, lw = 0;
#pragma unroll
            for (int q = 0; q < 2; ++q) {
                const float x = v[order[2 * p + q]] * inv;
                const _Float16 h = static_cast<_Float16>(x);
                const _Float16 l = static_cast<_Float16>(x - static_cast<float>(h));
                hw |= uint32_t(__builtin_bit_cast(uint16_t, h)) << (16 * q);
                lw |= uint32_t(__builtin_bit_cast(uint16_t, l)) << (16 * q);
            }
            hi[p] = hw; lo[p] = lw;
        }
        uint8_t* base = image + (size_t(g) * 4 + 2 * r) * 64 + s * 16;
        *reinterpret_cast<uint4*>(base) = make_uint4(hi[0], hi[1], hi[2], hi[3]);
        *reinterpret_cast<uint4*>(base + 64) = make_uint4(lo[0], lo[1], lo[2], lo[3]);
        if (rows == 1) {  // the operand always has four variants; a single row leaves two empty
            *reinterpret_cast<uint4*>(base + 128) = make_uint4(0, 0, 0, 0);
            *reinterpret_cast<uint4*>(base + 192) = make_uint4(0, 0, 0, 0);
        }
    }
}

// Writes the part of row r's receipt that covers elements k0 .. k0+count (both multiples of 32)
// from vals[0 .. count) (LDS or global).  Called by every thread of a workgroup whose size is a
// multiple of 64; four consecutive lanes share a group.
__device__ __forceinline__ void emit_receipt(const float* vals, uint32_t k0, uint32_t count, uint32_t r, uint32_t rows,
                                             uint32_t K, void* blob, uint32_t tid = threadIdx.x, uint32_t nthreads = blockDim.x) {
    for (uint32_t t = tid; t < count / 8; t += nthreads) {
        float v[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) v[i] = vals[t * 8 + i];
        emit_receipt_values(v, k0, t, r, rows, K, blob);
    }
}

}  // namespace guffin
