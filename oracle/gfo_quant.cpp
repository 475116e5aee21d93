// CPU oracle (test infrastructure only, see gfo.h): block decoders and the
// sequential-fp32 GEMV of the reference CPU backend.
//
// Follows:
//   src/tensor/f16.cpp:7-37                     fp16 bits -> fp32 (exact)
//   src/tensor/quantization.cpp:338-357         Q4_K 6-bit scale/min unpack
//   src/tensor/quantization.cpp:457-459         Q8_0 value  = d * int8
//   src/tensor/quantization.cpp:507-521         Q4_K nibble order and value
//   src/tensor/quantization.cpp:558-593         Q6_K bit planes and value
//   src/tensor/backends/cpu_backend.cpp:43-72   column-major block addressing
//   src/tensor/backends/cpu_backend.cpp:301-323 GEMV: sum=0.0f; sum += x*w, k ascending
// Build with -ffp-contract=off: every multiply and add rounds separately.
#include "gfo.h"

#include <cmath>
#include <cstring>
#include <stdexcept>
#include <thread>
#include <vector>

namespace {

constexpr uint32_t kBytes[3] = {34, 144, 210};
constexpr uint32_t kElems[3] = {32, 256, 256};

inline uint16_t load_u16(const uint8_t* p) { return static_cast<uint16_t>(p[0] | (p[1] << 8)); }

// One element of a Q8_0 block: 2-byte fp16 scale, then 32 signed bytes.
inline float q8_0_value(const uint8_t* b, uint32_t i) {
    const float d = gfo_f16_to_f32(load_u16(b));
    const int8_t q = static_cast<int8_t>(b[2 + i]);
    return d * static_cast<float>(q);
}

// Group g of a Q4_K block has a 6-bit scale and a 6-bit min packed in 12 bytes.
inline void q4_k_scale_min(const uint8_t* s, uint32_t g, uint8_t& sc, uint8_t& mn) {
    if (g < 4) {
        sc = s[g] & 63;
        mn = s[g + 4] & 63;
    } else {
        sc = static_cast<uint8_t>((s[g + 4] & 0x0F) | ((s[g - 4] >> 6) << 4));
        mn = static_cast<uint8_t>((s[g + 4] >> 4) | ((s[g] >> 6) << 4));
    }
}

inline float q4_k_value(const uint8_t* b, uint32_t i) {
    const float d = gfo_f16_to_f32(load_u16(b));
    const float dmin = gfo_f16_to_f32(load_u16(b + 2));
    uint8_t sc, mn;
    q4_k_scale_min(b + 4, i / 32, sc, mn);
    const uint8_t byte = b[16 + (i / 64) * 32 + (i % 32)];
    const uint8_t q = (i % 64) < 32 ? (byte & 0x0F) : (byte >> 4);
    // left-to-right: (d*sc)*q - (dmin*m)
    return d * static_cast<float>(sc) * static_cast<float>(q) - dmin * static_cast<float>(mn);
}

inline float q6_k_value(const uint8_t* b, uint32_t i) {
    const uint32_t half = i / 128, r = i % 128, lane = r % 32;
    const uint8_t lo_byte = b[half * 64 + ((r / 32) % 2) * 32 + lane];
    const uint8_t lo = r < 64 ? (lo_byte & 0x0F) : (lo_byte >> 4);
    const uint8_t hi = (b[128 + half * 32 + lane] >> ((r / 32) * 2)) & 3;
    const int q = static_cast<int>(lo | (hi << 4)) - 32;
    const int8_t scale = static_cast<int8_t>(b[192 + i / 16]);
    const float d = gfo_f16_to_f32(load_u16(b + 208));
    // left-to-right: (d*scale)*q
    return d * static_cast<float>(scale) * static_cast<float>(static_cast<int8_t>(q));
}

inline float block_value(int dtype, const uint8_t* b, uint32_t i) {
    switch (dtype) {
        case GFO_Q8_0: return q8_0_value(b, i);
        case GFO_Q4_K: return q4_k_value(b, i);
        default: return q6_k_value(b, i);
    }
}

void dequant_column(int dtype, const uint8_t* col, uint32_t K, float* out) {
    const uint32_t be = kElems[dtype], bb = kBytes[dtype];
    for (uint32_t blk = 0; blk < K / be; ++blk)
        for (uint32_t i = 0; i < be; ++i) out[blk * be + i] = block_value(dtype, col + size_t(blk) * bb, i);
}

void gemv_columns(int dtype, const uint8_t* w, const float* x, float* y, uint32_t rows,
                  uint32_t K, uint32_t N, uint32_t n0, uint32_t n1) {
    const size_t col_bytes = size_t(K / kElems[dtype]) * kBytes[dtype];
    std::vector<float> wcol(K);
    for (uint32_t n = n0; n < n1; ++n) {
        dequant_column(dtype, w + n * col_bytes, K, wcol.data());
        for (uint32_t r = 0; r < rows; ++r) {
            const float* xr = x + size_t(r) * K;
            float sum = 0.0f;
            for (uint32_t k = 0; k < K; ++k) sum += xr[k] * wcol[k];
            y[size_t(r) * N + n] = sum;
        }
    }
}

}  // namespace

extern "C" {

float gfo_f16_to_f32(uint16_t h) {
    const uint32_t sign = uint32_t(h & 0x8000u) << 16;
    const uint32_t e = (h >> 10) & 0x1F;
    uint32_t f = h & 0x3FF;
    uint32_t bits;
    if (e == 0) {
        if (f == 0) {
            bits = sign;
        } else {  // subnormal half: renormalise
            int ex = -14;
            while (!(f & 0x400)) { f <<= 1; --ex; }
            bits = sign | (uint32_t(ex + 127) << 23) | ((f & 0x3FF) << 13);
        }
    } else if (e == 31) {
        bits = sign | 0x7F800000u | (f << 13);
    } else {
        bits = sign | ((e + 112) << 23) | (f << 13);
    }
    float out;
    std::memcpy(&out, &bits, 4);
    return out;
}

uint32_t gfo_block_bytes(int dtype) { return kBytes[dtype]; }
uint32_t gfo_block_elems(int dtype) { return kElems[dtype]; }

void gfo_dequant(int dtype, const uint8_t* blocks, uint64_t n_blocks, float* out) {
    const uint32_t be = kElems[dtype], bb = kBytes[dtype];
    for (uint64_t b = 0; b < n_blocks; ++b)
        for (uint32_t i = 0; i < be; ++i) out[b * be + i] = block_value(dtype, blocks + b * bb, i);
}

void gfo_gemv(int dtype, const uint8_t* w, const float* x, float* y, uint32_t rows, uint32_t K,
              uint32_t N) {
    gemv_columns(dtype, w, x, y, rows, K, N, 0, N);
}

void gfo_gemv_mt(int dtype, const uint8_t* w, const float* x, float* y, uint32_t rows,
                 uint32_t K, uint32_t N, uint32_t threads) {
    if (threads <= 1) { gemv_columns(dtype, w, x, y, rows, K, N, 0, N); return; }
    std::vector<std::thread> pool;
    const uint32_t per = (N + threads - 1) / threads;
    for (uint32_t t = 0; t < threads; ++t) {
        const uint32_t n0 = t * per, n1 = n0 + per < N ? n0 + per : N;
        if (n0 >= n1) break;
        pool.emplace_back(gemv_columns, dtype, w, x, y, rows, K, N, n0, n1);
    }
    for (auto& th : pool) th.join();
}

// The reference's loop nest verbatim in behaviour: for every (row, column, inner)
// it locates the block from the column-major index and decodes ONE element, with
// the block-index bounds check its block view performs.
void gfo_gemv_as_written(int dtype, const uint8_t* w, const float* x, float* y, uint32_t rows,
                         uint32_t K, uint32_t N) {
    const uint32_t be = kElems[dtype], bb = kBytes[dtype];
    const uint64_t blocks_per_column = K / be;
    const uint64_t block_count = blocks_per_column * N;
    for (uint32_t r = 0; r < rows; ++r) {
        for (uint32_t n = 0; n < N; ++n) {
            float sum = 0.0f;
            for (uint32_t k = 0; k < K; ++k) {
                const uint64_t block = n * blocks_per_column + k / be;
                if (block >= block_count) throw std::out_of_range("block index");
                sum += x[size_t(r) * K + k] * block_value(dtype, w + block * bb, k % be);
            }
            y[size_t(r) * N + n] = sum;
        }
    }
}

}  // extern "C"
