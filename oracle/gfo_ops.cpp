// CPU oracle (test infrastructure only, see gfo.h): the small per-layer operators.
//
// Follows:
//   src/tensor/ops/normalization.cpp:70-99   rms_norm_f32 (fp32 sequential sum, 1/sqrt)
//   src/tensor/backends/metal/metal_kernels.mm:2109-2158  rms_norm_add = norm*gamma + residual
//   src/tensor/backends/metal/metal_kernels.mm:1916-1932  per-head RMS norm over head_dim
//   src/tensor/ops/rope.cpp:109-117, 242-283 split-half RoPE, angle in double
//   src/tensor/backends/metal/metal_kernels.mm:2406-2486  per-row positions, frequency_scale,
//                                            K narrowed to fp16 AFTER rotation, V narrowed
//   tests/tensor/gemma3_metal_tests.cpp:87-128  binary16 round-to-nearest-even contract
//   src/tensor/ops/elementwise.cpp:79-94, 50-63  gelu_tanh(g) * u
//   src/tensor/ops/attention.cpp:482-618 + softmax.cpp:42-71  scores (fp32 sequential dot
//                                            * scale), softmax (double exp, double sum,
//                                            stored as float), values (fp32 sequential)
//   src/tensor/backends/metal/metal_kernels.mm:3061-3147  token order: ring then ancestors
//   src/tensor/ops/reduction.cpp:93-117      argmax, strict '>' (lowest id wins ties)
//   src/engine/sampling.cpp:25-30            candidate order: logit desc, token asc
//   src/tensor/backends/metal/metal_kernels.mm:452-474   embedding = dequant row * scale
#include "gfo.h"

#include <algorithm>
#include <cmath>
#include <cstring>
#include <limits>
#include <vector>

extern "C" {

uint16_t gfo_f32_to_f16_rne(float value) {
    uint32_t x;
    std::memcpy(&x, &value, 4);
    const uint16_t sign = static_cast<uint16_t>((x >> 16) & 0x8000u);
    const uint32_t mag = x & 0x7FFFFFFFu;
    if (mag >= 0x7F800000u) {  // inf / nan
        return static_cast<uint16_t>(sign | (mag > 0x7F800000u ? 0x7E00u : 0x7C00u));
    }
    const int32_t exp = static_cast<int32_t>(mag >> 23) - 127;
    if (exp > 15) return static_cast<uint16_t>(sign | 0x7C00u);
    if (exp >= -14) {  // normal half candidate
        const uint32_t mant = mag & 0x7FFFFFu;
        uint32_t half = (static_cast<uint32_t>(exp + 15) << 10) | (mant >> 13);
        const uint32_t rest = mant & 0x1FFFu;
        if (rest > 0x1000u || (rest == 0x1000u && (half & 1u))) ++half;  // carries into exponent
        return static_cast<uint16_t>(sign | half);
    }
    if (exp < -25) return sign;  // below half of the smallest subnormal
    // subnormal half: value = m * 2^-24, m in [0, 1024]
    const uint32_t mant = (mag & 0x7FFFFFu) | 0x800000u;  // 24-bit significand, value = mant * 2^(exp-23)
    const uint32_t shift = static_cast<uint32_t>(-exp - 1);  // mant >> shift gives units of 2^-24
    uint32_t half = mant >> shift;
    const uint32_t rest = mant & ((1u << shift) - 1u);
    const uint32_t halfway = 1u << (shift - 1u);
    if (rest > halfway || (rest == halfway && (half & 1u))) ++half;
    return static_cast<uint16_t>(sign | half);
}

void gfo_rms_norm(const float* x, const float* gamma, float* y, uint32_t rows, uint32_t width,
                  float eps) {
    for (uint32_t r = 0; r < rows; ++r) {
        const float* in = x + size_t(r) * width;
        float ss = 0.0f;
        for (uint32_t c = 0; c < width; ++c) ss += in[c] * in[c];
        const float mean = ss / static_cast<float>(width);
        const float inv = 1.0f / std::sqrt(mean + eps);
        for (uint32_t c = 0; c < width; ++c) y[size_t(r) * width + c] = in[c] * inv * gamma[c];
    }
}

void gfo_rms_norm_add(const float* x, const float* gamma, const float* residual, float* y,
                      uint32_t rows, uint32_t width, float eps) {
    for (uint32_t r = 0; r < rows; ++r) {
        const float* in = x + size_t(r) * width;
        float ss = 0.0f;
        for (uint32_t c = 0; c < width; ++c) ss += in[c] * in[c];
        const float mean = ss / static_cast<float>(width);
        const float inv = 1.0f / std::sqrt(mean + eps);
        for (uint32_t c = 0; c < width; ++c)
            y[size_t(r) * width + c] = in[c] * inv * gamma[c] + residual[size_t(r) * width + c];
    }
}

void gfo_head_rms_norm(const float* x, const float* gamma, float* y, uint32_t rows,
                       uint32_t heads, uint32_t head_dim, float eps) {
    gfo_rms_norm(x, gamma, y, rows * heads, head_dim, eps);
}

static inline double rope_angle(uint32_t position, uint32_t pair, uint32_t rope_dim, float base,
                                float scale) {
    const double exponent = static_cast<double>(2u * pair) / static_cast<double>(rope_dim);
    return static_cast<double>(position) / std::pow(static_cast<double>(base), exponent)
        * static_cast<double>(scale);
}

void gfo_rope_neox(const float* in, float* out, const uint32_t* positions, uint32_t rows,
                   uint32_t heads, uint32_t head_dim, uint32_t rope_dim, float base, float scale) {
    const uint32_t width = heads * head_dim, half = rope_dim / 2;
    if (out != in) std::memcpy(out, in, size_t(rows) * width * sizeof(float));
    std::vector<float> tmp(head_dim);
    for (uint32_t r = 0; r < rows; ++r)
        for (uint32_t h = 0; h < heads; ++h) {
            const float* src = in + size_t(r) * width + size_t(h) * head_dim;
            float* dst = out + size_t(r) * width + size_t(h) * head_dim;
            std::memcpy(tmp.data(), src, head_dim * sizeof(float));
            for (uint32_t p = 0; p < half; ++p) {
                const double a = rope_angle(positions[r], p, rope_dim, base, scale);
                const float c = static_cast<float>(std::cos(a)), s = static_cast<float>(std::sin(a));
                const float first = tmp[p], second = tmp[p + half];
                dst[p] = first * c - second * s;
                dst[p + half] = first * s + second * c;
            }
        }
}

void gfo_kv_store_f16(const float* raw_k, const float* raw_v, const uint32_t* positions,
                      uint16_t* out_k, uint16_t* out_v, uint32_t rows, uint32_t heads,
                      uint32_t head_dim, uint32_t rope_dim, float base, float scale) {
    const size_t n = size_t(rows) * heads * head_dim;
    std::vector<float> rotated(n);
    if (rope_dim)
        gfo_rope_neox(raw_k, rotated.data(), positions, rows, heads, head_dim, rope_dim, base, scale);
    else
        std::memcpy(rotated.data(), raw_k, n * sizeof(float));
    for (size_t i = 0; i < n; ++i) {
        out_k[i] = gfo_f32_to_f16_rne(rotated[i]);
        out_v[i] = gfo_f32_to_f16_rne(raw_v[i]);
    }
}

void gfo_geglu(const float* gate, const float* up, float* out, uint64_t n) {
    constexpr float k0 = 0.7978845608028654f, k1 = 0.044715f;
    for (uint64_t i = 0; i < n; ++i) {
        const float v = gate[i];
        const float inner = k0 * (v + k1 * v * v * v);
        const float g = 0.5f * v * (1.0f + std::tanh(inner));
        out[i] = g * up[i];
    }
}

void gfo_embed(int dtype, const uint8_t* w, const uint32_t* tokens, float* out, uint32_t rows,
               uint32_t width, float scale) {
    const uint32_t be = gfo_block_elems(dtype), bb = gfo_block_bytes(dtype);
    const size_t row_bytes = size_t(width / be) * bb;
    for (uint32_t r = 0; r < rows; ++r) {
        gfo_dequant(dtype, w + tokens[r] * row_bytes, width / be, out + size_t(r) * width);
        for (uint32_t c = 0; c < width; ++c) out[size_t(r) * width + c] *= scale;
    }
}

void gfo_attention(const float* q, const uint16_t* ring_k, const uint16_t* ring_v,
                   const uint16_t* priv_k, const uint16_t* priv_v, const uint32_t* schedule,
                   const uint32_t* ancestors, float* out, uint32_t rows, uint32_t row_mask,
                   uint32_t q_heads, uint32_t kv_heads, uint32_t head_dim, float scale) {
    const uint32_t group = q_heads / kv_heads, kv_width = kv_heads * head_dim;
    std::vector<float> scores, probs;
    std::vector<const uint16_t*> krow, vrow;
    for (uint32_t r = 0; r < rows; ++r) {
        const uint32_t* s = schedule + 4 * r;
        const uint32_t count = s[1] + s[3];
        krow.resize(count); vrow.resize(count); scores.resize(count); probs.resize(count);
        for (uint32_t h = 0; h < q_heads; ++h) {
            const uint32_t kvh = h / group;
            for (uint32_t t = 0; t < count; ++t) {
                if (t < s[1]) {
                    const size_t slot = (s[0] + t) & row_mask;
                    krow[t] = ring_k + slot * kv_width + kvh * head_dim;
                    vrow[t] = ring_v + slot * kv_width + kvh * head_dim;
                } else {
                    const size_t slot = ancestors[s[2] + t - s[1]];
                    krow[t] = priv_k + slot * kv_width + kvh * head_dim;
                    vrow[t] = priv_v + slot * kv_width + kvh * head_dim;
                }
            }
            const float* qh = q + (size_t(r) * q_heads + h) * head_dim;
            for (uint32_t t = 0; t < count; ++t) {
                float dot = 0.0f;
                for (uint32_t c = 0; c < head_dim; ++c) dot += qh[c] * gfo_f16_to_f32(krow[t][c]);
                scores[t] = dot * scale;
            }
            float mx = scores[0];
            for (uint32_t t = 1; t < count; ++t) mx = std::max(mx, scores[t]);
            double sum = 0.0;
            for (uint32_t t = 0; t < count; ++t) {
                const double e = std::exp(static_cast<double>(scores[t] - mx));
                sum += e;
                probs[t] = static_cast<float>(e);
            }
            for (uint32_t t = 0; t < count; ++t)
                probs[t] = static_cast<float>(static_cast<double>(probs[t]) / sum);
            float* oh = out + (size_t(r) * q_heads + h) * head_dim;
            for (uint32_t c = 0; c < head_dim; ++c) {
                float acc = 0.0f;
                for (uint32_t t = 0; t < count; ++t) acc += probs[t] * gfo_f16_to_f32(vrow[t][c]);
                oh[c] = acc;
            }
        }
    }
}

uint32_t gfo_argmax(const float* logits, uint32_t vocab) {
    uint32_t best = 0;
    float best_logit = logits[0];
    for (uint32_t t = 1; t < vocab; ++t)
        if (logits[t] > best_logit) { best = t; best_logit = logits[t]; }
    return best;
}

int gfo_select_candidates(const float* logits, uint32_t vocab, uint32_t k, const uint32_t* history,
                          uint32_t history_count, gfo_token_logit* out) {
    const uint32_t keep = std::min(vocab, k);
    std::vector<gfo_token_logit> all(vocab);
    for (uint32_t t = 0; t < vocab; ++t) all[t] = {t, logits[t]};
    auto better = [](const gfo_token_logit& a, const gfo_token_logit& b) {
        if (a.logit != b.logit) return a.logit > b.logit;
        return a.token < b.token;
    };
    std::partial_sort(all.begin(), all.begin() + keep, all.end(), better);
    uint32_t n = 0;
    for (uint32_t i = 0; i < keep; ++i) {
        if (!std::isfinite(all[i].logit)) return -1;
        out[n++] = all[i];
    }
    for (uint32_t i = 0; i < history_count; ++i) {
        const float l = logits[history[i]];
        if (!std::isfinite(l)) return -1;
        out[n++] = {history[i], l};
    }
    return static_cast<int>(n);
}

}  // extern "C"
