// Per-layer operators of the Gemma-3 block graph on gfx950: RMS norms, NeoX RoPE,
// fp16 KV narrowing, GeGLU, embedding gather, KV publication.
//
// Reference behaviour:
//   rms_norm / rms_norm_add / head_rms_norm  src/tensor/backends/metal/metal_kernels.mm:1915-2158
//                                            (CPU: src/tensor/ops/normalization.cpp:70-99)
//   rope by positions, kv store              metal_kernels.mm:2406-2486 (CPU angle in double:
//                                            src/tensor/ops/rope.cpp:109-117, 242-283)
//   gelu_tanh * up                           metal_kernels.mm:1827-1843 (CPU: ops/elementwise.cpp:79-94)
//   embedding                                metal_kernels.mm:452-474, src/engine/gemma3_draft.mm:61-71
//   kv scatter (publish private rows)        metal_kernels.mm:2519-2557
//
// Every operator that produces a GEMV input can also emit the per-16 / per-32 activation
// sums the packed GEMV consumes, and every operator that consumes a GEMV output can sum
// `planes` k-slice partial planes (stride plane_stride floats) while it loads.
#include "common.hpp"
#include "receipt.hpp"

namespace guffin {
namespace {

__device__ __forceinline__ float block_sum(float v, float* scratch) {
    v = wave_sum(v);
    const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6, nw = (blockDim.x + 63) >> 6;
    __syncthreads();  // scratch may still be read from a previous call
    if (lane == 0) scratch[wv] = v;
    __syncthreads();
    float t = 0.f;
    for (int i = 0; i < nw; ++i) t += scratch[i];  // same order on every thread
    return t;
}

// Loads the row (summing partial planes) into LDS and returns this thread's share of the
// squared sum.  Four columns per thread are in flight at a time, plane loads in batches of
// four, so a row of a few thousand columns costs two or three memory round trips.
__device__ __forceinline__ float stage_row(const float* __restrict__ xr, uint32_t planes, size_t plane_stride,
                                           float* row, uint32_t width) {
    float ss = 0.f;
    const uint32_t step = blockDim.x;
    for (uint32_t c0 = threadIdx.x; c0 < width; c0 += 4 * step) {
        float v[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) v[u] = c0 + u * step < width ? xr[c0 + u * step] : 0.f;
        uint32_t s = 1;
        for (; s + 4 <= planes; s += 4) {
            float t[4][4];
#pragma unroll
            for (int u = 0; u < 4; ++u)
#pragma unroll
                for (int k = 0; k < 4; ++k) t[u][k] = c0 + u * step < width ? xr[(s + k) * plane_stride + c0 + u * step] : 0.f;
#pragma unroll
            for (int u = 0; u < 4; ++u)
#pragma unroll
                for (int k = 0; k < 4; ++k) v[u] += t[u][k];
        }
        for (; s < planes; ++s) {
            float t[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) t[u] = c0 + u * step < width ? xr[s * plane_stride + c0 + u * step] : 0.f;
#pragma unroll
            for (int u = 0; u < 4; ++u) v[u] += t[u];
        }
#pragma unroll
        for (int u = 0; u < 4; ++u)
            if (c0 + u * step < width) { row[c0 + u * step] = v[u]; ss = fmaf(v[u], v[u], ss); }
    }
    return ss;
}

// y = x * rsqrt(mean(x^2) + eps) * gamma [+ residual]; one workgroup per row.
// x may be `planes` partial planes.  Optional outputs: y_sums (group sums of y).
__global__ void __launch_bounds__(1024)
rms_norm_kernel(const float* __restrict__ x, uint32_t planes, size_t plane_stride,
                const float* __restrict__ gamma, const float* __restrict__ residual,
                float* __restrict__ y, float* __restrict__ y_sums, uint32_t width, float eps,
                uint32_t* __restrict__ status) {
    extern __shared__ float lds[];  // [width] row image + [16] scratch
    float* row = lds;
    float* scratch = lds + width;
    const uint32_t r = blockIdx.x;
    // operands of the second pass are requested before the first reduction
    constexpr int PF = 4;
    float gm[PF], rs[PF];
#pragma unroll
    for (int u = 0; u < PF; ++u) {
        const uint32_t c = threadIdx.x + u * blockDim.x;
        gm[u] = c < width ? gamma[c] : 0.f;
        rs[u] = (residual && c < width) ? residual[size_t(r) * width + c] : 0.f;
    }
    const float ss = stage_row(x + size_t(r) * width, planes, plane_stride, row, width);
    const float total = block_sum(ss, scratch);
    const float inv = 1.0f / sqrtf(total / static_cast<float>(width) + eps);
    bool bad = false;
    auto second = [&](uint32_t c, float g, float res) {
        float v = row[c] * inv * g;
        if (residual) v += res;
        bad |= !isfinite(v);
        row[c] = v;
        y[size_t(r) * width + c] = v;
    };
#pragma unroll
    for (int u = 0; u < PF; ++u) {
        const uint32_t c = threadIdx.x + u * blockDim.x;
        if (c < width) second(c, gm[u], rs[u]);
    }
    for (uint32_t c = threadIdx.x + PF * blockDim.x; c < width; c += blockDim.x)
        second(c, gamma[c], residual ? residual[size_t(r) * width + c] : 0.f);
    if (bad && status) atomicOr(status, GUFFIN_STATUS_NONFINITE);
    if (y_sums) {
        __syncthreads();
        emit_receipt(row, 0, width, r, gridDim.x, width, y_sums);
    }
}

// Fused tail of one sub-block and head of the next:
//   out_residual = residual + rms(x, gamma_post);  out_norm = rms(out_residual, gamma_next)
// (reference order: encode_rms_norm_add then encode_rms_norm, gemma_target_runtime.cpp:156-173, 201-213)
__global__ void __launch_bounds__(1024)
rms_norm_add_norm_kernel(const float* __restrict__ x, uint32_t planes, size_t plane_stride,
                         const float* __restrict__ gamma_post, const float* __restrict__ residual,
                         float* __restrict__ out_residual, const float* __restrict__ gamma_next,
                         float* __restrict__ out_norm, float* __restrict__ out_sums, uint32_t width,
                         float eps, uint32_t* __restrict__ status) {
    extern __shared__ float lds[];
    float* row = lds;
    float* scratch = lds + width;
    const uint32_t r = blockIdx.x;
    // operands of the second and third pass are requested before the first reduction
    constexpr int PF = 4;
    float gp[PF], rs[PF], gn[PF];
#pragma unroll
    for (int u = 0; u < PF; ++u) {
        const uint32_t c = threadIdx.x + u * blockDim.x;
        const bool in = c < width;
        gp[u] = in ? gamma_post[c] : 0.f;
        rs[u] = in ? residual[size_t(r) * width + c] : 0.f;
        gn[u] = in ? gamma_next[c] : 0.f;
    }
    float ss = stage_row(x + size_t(r) * width, planes, plane_stride, row, width);
    float total = block_sum(ss, scratch);
    float inv = 1.0f / sqrtf(total / static_cast<float>(width) + eps);
    ss = 0.f;
    bool bad = false;
    auto second = [&](uint32_t c, float g, float res) {
        const float v = row[c] * inv * g + res;
        bad |= !isfinite(v);
        row[c] = v;
        out_residual[size_t(r) * width + c] = v;
        ss = fmaf(v, v, ss);
    };
#pragma unroll
    for (int u = 0; u < PF; ++u) {
        const uint32_t c = threadIdx.x + u * blockDim.x;
        if (c < width) second(c, gp[u], rs[u]);
    }
    for (uint32_t c = threadIdx.x + PF * blockDim.x; c < width; c += blockDim.x)
        second(c, gamma_post[c], residual[size_t(r) * width + c]);
    total = block_sum(ss, scratch);
    inv = 1.0f / sqrtf(total / static_cast<float>(width) + eps);
    auto third = [&](uint32_t c, float g) {
        const float v = row[c] * inv * g;
        row[c] = v;
        out_norm[size_t(r) * width + c] = v;
    };
#pragma unroll
    for (int u = 0; u < PF; ++u) {
        const uint32_t c = threadIdx.x + u * blockDim.x;
        if (c < width) third(c, gn[u]);
    }
    for (uint32_t c = threadIdx.x + PF * blockDim.x; c < width; c += blockDim.x) third(c, gamma_next[c]);
    if (bad && status) atomicOr(status, GUFFIN_STATUS_NONFINITE);
    if (out_sums) {
        __syncthreads();
        emit_receipt(row, 0, width, r, gridDim.x, width, out_sums);
    }
}

// The same for the common shape (at most four planes, 16-byte aligned rows, width a multiple of 8
// and at most 8 x 1024): a thread owns 8 consecutive columns from the operands to the receipt, so
// every operand is requested at once (one trip to memory instead of one per plane batch) and
// nothing is staged in LDS but the per-wave sums.
constexpr int kFastPlanes = 4;
__device__ __forceinline__ float4 ld4(const float* p, bool on) {
    return on ? *reinterpret_cast<const float4*>(p) : make_float4(0.f, 0.f, 0.f, 0.f);
}
__device__ __forceinline__ void unpack4(const float4& a, float* o) { o[0] = a.x; o[1] = a.y; o[2] = a.z; o[3] = a.w; }

__global__ void __launch_bounds__(1024)
rms_norm_add_norm_regs_kernel(const float* __restrict__ x, uint32_t planes, size_t plane_stride,
                              const float* __restrict__ gamma_post, const float* __restrict__ residual,
                              float* __restrict__ out_residual, const float* __restrict__ gamma_next,
                              float* __restrict__ out_norm, float* __restrict__ out_sums, uint32_t width,
                              float eps, uint32_t* __restrict__ status) {
    __shared__ float scratch[16];
    const uint32_t r = blockIdx.x, item = threadIdx.x;
    const bool active = item < width / 8;
    const size_t col = active ? item * 8u : 0u, at = size_t(r) * width + col;
    float4 p[kFastPlanes][2], res4[2], gp4[2], gn4[2];
#pragma unroll
    for (int h = 0; h < 2; ++h) {
        gp4[h] = ld4(gamma_post + col + 4 * h, active);
        gn4[h] = ld4(gamma_next + col + 4 * h, active);
        res4[h] = ld4(residual + at + 4 * h, active);
#pragma unroll
        for (int s = 0; s < kFastPlanes; ++s) p[s][h] = ld4(x + s * plane_stride + at + 4 * h, active && uint32_t(s) < planes);
    }
    float v[8], a[8], gp[8], gn[8], res[8];
    unpack4(p[0][0], v); unpack4(p[0][1], v + 4);
#pragma unroll
    for (int s = 1; s < kFastPlanes; ++s) {  // plane order
        if (uint32_t(s) < planes) {
            unpack4(p[s][0], a); unpack4(p[s][1], a + 4);
#pragma unroll
            for (int i = 0; i < 8; ++i) v[i] += a[i];
        }
    }
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i) ss = fmaf(v[i], v[i], ss);
    float total = block_sum(ss, scratch);
    float inv = 1.0f / sqrtf(total / static_cast<float>(width) + eps);
    unpack4(gp4[0], gp); unpack4(gp4[1], gp + 4);
    unpack4(gn4[0], gn); unpack4(gn4[1], gn + 4);
    unpack4(res4[0], res); unpack4(res4[1], res + 4);
    bool bad = false;
    ss = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const float t = active ? v[i] * inv * gp[i] + res[i] : 0.f;
        bad |= !isfinite(t);
        v[i] = t;
        ss = fmaf(t, t, ss);
    }
    if (active) {
        *reinterpret_cast<float4*>(out_residual + at) = make_float4(v[0], v[1], v[2], v[3]);
        *reinterpret_cast<float4*>(out_residual + at + 4) = make_float4(v[4], v[5], v[6], v[7]);
    }
    total = block_sum(ss, scratch);
    inv = 1.0f / sqrtf(total / static_cast<float>(width) + eps);
    float y[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) y[i] = v[i] * inv * gn[i];
    if (active) {
        *reinterpret_cast<float4*>(out_norm + at) = make_float4(y[0], y[1], y[2], y[3]);
        *reinterpret_cast<float4*>(out_norm + at + 4) = make_float4(y[4], y[5], y[6], y[7]);
        if (out_sums) emit_receipt_values(y, 0, item, r, gridDim.x, width, out_sums);
    }
    if (bad && status) atomicOr(status, GUFFIN_STATUS_NONFINITE);
}

// Per-head RMS norm over head_dim (one wave per (row, head)); in place allowed.
__global__ void __launch_bounds__(64)
head_rms_norm_kernel(const float* __restrict__ x, const float* __restrict__ gamma, float* __restrict__ y,
                     uint32_t head_dim, float eps) {
    const size_t base = size_t(blockIdx.x) * head_dim;
    float ss = 0.f;
    for (uint32_t c = threadIdx.x; c < head_dim; c += 64) { const float v = x[base + c]; ss = fmaf(v, v, ss); }
    ss = wave_sum(ss);
    const float inv = 1.0f / sqrtf(ss / static_cast<float>(head_dim) + eps);
    for (uint32_t c = threadIdx.x; c < head_dim; c += 64) y[base + c] = x[base + c] * inv * gamma[c];
}

// Fused q/k head norm + NeoX RoPE + fp16 KV narrowing for `rows` new tokens:
//   q_out = rope(headnorm(q_raw)) fp32;  k_out = f16(rope(headnorm(k_raw)));  v_out = f16(v_raw)
// One wave per (row, head); q heads first, then k heads, then v heads.  Any of the three
// sections can be disabled with a null pointer; q_norm/k_norm null skips the head norm.
// Inputs may be `planes` partial planes of a GEMV.
// cos/sin of every (row, pair) once per forward pass: table[row][pair] = {cos, sin}
__global__ void rope_table_kernel(const uint32_t* positions, float2* table, uint32_t rows, uint32_t rope_dim,
                                  float base, float scale) {
    const uint32_t half = rope_dim / 2, i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= rows * half) return;
    float c, s;
    rope_sincos(positions[i / half], i % half, rope_dim, base, scale, c, s);
    table[i] = make_float2(c, s);
}

struct QkvArgs {
    const float2* rope_table;  // optional [rows][rope_dim/2] from rope_table_kernel; else computed here
    const float* q_raw; const float* k_raw; const float* v_raw;
    uint32_t q_planes, k_planes, v_planes; size_t q_plane_stride, k_plane_stride, v_plane_stride;
    const float* q_norm; const float* k_norm;
    const uint32_t* positions;
    float* q_out; uint16_t* k_out; uint16_t* v_out;
    uint32_t rows, q_heads, kv_heads, head_dim, rope_dim;
    float base, scale, eps;
    uint32_t* status;
};

__global__ void __launch_bounds__(64) qkv_post_kernel(QkvArgs a) {
    extern __shared__ float lds[];  // [head_dim]
    const uint32_t per_row = a.q_heads + 2 * a.kv_heads;
    const uint32_t r = blockIdx.x / per_row, h = blockIdx.x % per_row, lane = threadIdx.x;
    const bool is_q = h < a.q_heads, is_k = !is_q && h < a.q_heads + a.kv_heads;
    const uint32_t hh = is_q ? h : is_k ? h - a.q_heads : h - a.q_heads - a.kv_heads;
    const uint32_t heads = is_q ? a.q_heads : a.kv_heads;
    const float* src = is_q ? a.q_raw : is_k ? a.k_raw : a.v_raw;
    if (!src) return;
    const size_t stride = is_q ? a.q_plane_stride : is_k ? a.k_plane_stride : a.v_plane_stride;
    const uint32_t planes = is_q ? a.q_planes : is_k ? a.k_planes : a.v_planes;
    const size_t off = (size_t(r) * heads + hh) * a.head_dim;
    float ss = 0.f;
    for (uint32_t c = lane; c < a.head_dim; c += 64) {
        const float v = load_planes(src + off + c, planes, stride);
        lds[c] = v;
        ss = fmaf(v, v, ss);
    }
    bool bad = false;
    if (!is_q && !is_k) {  // V: narrow only
        for (uint32_t c = lane; c < a.head_dim; c += 64) {
            const _Float16 hv = static_cast<_Float16>(lds[c]);
            bad |= !isfinite(static_cast<float>(hv));
            a.v_out[off + c] = __builtin_bit_cast(uint16_t, hv);
        }
        if (bad && a.status) atomicOr(a.status, GUFFIN_STATUS_KV_NONFINITE);
        return;
    }
    const float* gamma = is_q ? a.q_norm : a.k_norm;
    if (gamma) {
        ss = wave_sum(ss);
        const float inv = 1.0f / sqrtf(ss / static_cast<float>(a.head_dim) + a.eps);
        for (uint32_t c = lane; c < a.head_dim; c += 64) lds[c] = lds[c] * inv * gamma[c];
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    const uint32_t half = a.rope_dim / 2, pos = a.rope_table ? 0u : a.positions[r];
    auto emit = [&](uint32_t c, float v) {
        if (is_q) {
            a.q_out[off + c] = v;
        } else {
            const _Float16 hv = static_cast<_Float16>(v);  // round-to-nearest-even, after rotation
            bad |= !isfinite(static_cast<float>(hv));
            a.k_out[off + c] = __builtin_bit_cast(uint16_t, hv);
        }
    };
    for (uint32_t pair = lane; pair < half; pair += 64) {
        float cs, sn;
        if (a.rope_table) { const float2 t = a.rope_table[size_t(r) * half + pair]; cs = t.x; sn = t.y; }
        else rope_sincos(pos, pair, a.rope_dim, a.base, a.scale, cs, sn);
        const float first = lds[pair], second = lds[pair + half];
        emit(pair, __fsub_rn(__fmul_rn(first, cs), __fmul_rn(second, sn)));
        emit(pair + half, __fadd_rn(__fmul_rn(first, sn), __fmul_rn(second, cs)));
    }
    for (uint32_t c = a.rope_dim + lane; c < a.head_dim; c += 64) emit(c, lds[c]);
    if (bad && a.status) atomicOr(a.status, GUFFIN_STATUS_KV_NONFINITE);
}

// out = gelu_tanh(gate) * up, element-wise; gate/up may be partial planes.  One workgroup
// per row when sums are requested (row image in LDS), grid-stride otherwise.
__global__ void __launch_bounds__(256)
geglu_kernel(const float* __restrict__ gate, const float* __restrict__ up, uint32_t planes, size_t plane_stride,
             float* __restrict__ out, float* __restrict__ out_sums, uint32_t width) {
    extern __shared__ float lds[];  // [chunk] when sums are requested
    // grid: (chunks_per_row, rows); a chunk is a multiple of 32 columns
    const uint32_t chunk = (width + gridDim.x - 1) / gridDim.x;
    const uint32_t c0 = blockIdx.x * chunk, c1 = c0 + chunk < width ? c0 + chunk : width;
    const size_t rbase = size_t(blockIdx.y) * width;
    for (uint32_t c = c0 + threadIdx.x; c < c1; c += blockDim.x) {
        const float g = load_planes(gate + rbase + c, planes, plane_stride);
        const float u = load_planes(up + rbase + c, planes, plane_stride);
        const float v = geglu_value(g, u);
        out[rbase + c] = v;
        if (out_sums) lds[c - c0] = v;
    }
    if (out_sums) {
        __syncthreads();
        emit_receipt(lds, c0, c1 - c0, blockIdx.y, gridDim.y, width, out_sums);
    }
}

// out[r, :] = dequant(row tokens[r] of W) * scale; canonical block stream (one row = width/elems blocks)
template <int DTYPE>
__global__ void __launch_bounds__(256)
embed_kernel(const uint8_t* __restrict__ w, const uint32_t* __restrict__ tokens, float* __restrict__ out,
             uint32_t width, float scale, uint32_t vocab, uint32_t* __restrict__ status) {
    constexpr uint32_t be = DTYPE == GUFFIN_Q8_0 ? 32 : 256;
    constexpr uint32_t bb = DTYPE == GUFFIN_Q8_0 ? 34 : DTYPE == GUFFIN_Q4_K ? 144 : 210;
    uint32_t token = tokens[blockIdx.x];
    if (token >= vocab) {
        if (threadIdx.x == 0 && status) atomicOr(status, GUFFIN_STATUS_BAD_TOKEN);
        token = 0;
    }
    const uint8_t* row = w + size_t(token) * (width / be) * bb;
    bool bad = false;
    for (uint32_t c = threadIdx.x; c < width; c += blockDim.x) {
        const uint8_t* b = row + size_t(c / be) * bb;
        const uint32_t i = c % be;
        float v;
        if constexpr (DTYPE == GUFFIN_Q8_0) {
            v = __fmul_rn(h2f(ld_u16(b)), static_cast<float>(static_cast<int8_t>(b[2 + i])));
        } else if constexpr (DTYPE == GUFFIN_Q6_K) {
            const uint32_t half = i >> 7, rr = i & 127, l = rr & 31;
            const uint32_t lo_byte = b[half * 64 + ((rr >> 5) & 1) * 32 + l];
            const uint32_t lo = rr < 64 ? (lo_byte & 0x0Fu) : (lo_byte >> 4);
            const uint32_t hi = (b[128 + half * 32 + l] >> ((rr >> 5) * 2)) & 3u;
            const int q = static_cast<int>(lo | (hi << 4)) - 32;
            const float sc = static_cast<float>(static_cast<int8_t>(b[192 + (i >> 4)]));
            v = __fmul_rn(__fmul_rn(h2f(ld_u16(b + 208)), sc), static_cast<float>(q));
        } else {
            const float d = h2f(ld_u16(b)), dmin = h2f(ld_u16(b + 2));
            const uint8_t* s = b + 4;
            const uint32_t g = i >> 5;
            uint32_t sc, mn;
            if (g < 4) { sc = s[g] & 63u; mn = s[g + 4] & 63u; }
            else { sc = (s[g + 4] & 0x0Fu) | ((s[g - 4] >> 6) << 4); mn = (s[g + 4] >> 4) | ((s[g] >> 6) << 4); }
            const uint32_t byte = b[16 + (i >> 6) * 32 + (i & 31)];
            const uint32_t q = (i & 63) < 32 ? (byte & 0x0Fu) : (byte >> 4);
            v = __fsub_rn(__fmul_rn(__fmul_rn(d, static_cast<float>(sc)), static_cast<float>(q)),
                          __fmul_rn(dmin, static_cast<float>(mn)));
        }
        v = __fmul_rn(v, scale);
        bad |= !isfinite(v);
        out[size_t(blockIdx.x) * width + c] = v;
    }
    if (bad && status) atomicOr(status, GUFFIN_STATUS_NONFINITE);
}

// ring[(position + i) & mask] = private[selected[i]] for both K and V (16-bit elements)
__global__ void kv_scatter_kernel(const uint16_t* __restrict__ priv_k, const uint16_t* __restrict__ priv_v,
                                  const uint32_t* __restrict__ selected, uint16_t* __restrict__ ring_k,
                                  uint16_t* __restrict__ ring_v, uint32_t position, uint32_t rows,
                                  uint32_t row_width, uint32_t mask) {
    const uint32_t i = blockIdx.y;
    if (i >= rows) return;
    // when more rows than ring slots are published only the newest owner of a slot writes it
    if (rows > mask + 1 && i + mask + 1 < rows) return;
    const size_t src = size_t(selected[i]) * row_width, dst = size_t((position + i) & mask) * row_width;
    for (uint32_t c = blockIdx.x * blockDim.x + threadIdx.x; c < row_width; c += gridDim.x * blockDim.x) {
        ring_k[dst + c] = priv_k[src + c];
        ring_v[dst + c] = priv_v[src + c];
    }
}

// one thread per four columns, whole waves, at most 1024 threads
uint32_t norm_threads(uint32_t width) {
    const uint32_t t = ((width + 3) / 4 + 63) / 64 * 64;
    return t < 64 ? 64 : t > 1024 ? 1024 : t;
}

bool aligned4(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 3u) == 0; }

}  // namespace

int ops_init(int) {
    int rc = 0;
    rc |= hipFuncSetAttribute(reinterpret_cast<const void*>(rms_norm_kernel),
                              hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024) != hipSuccess;
    rc |= hipFuncSetAttribute(reinterpret_cast<const void*>(rms_norm_add_norm_kernel),
                              hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024) != hipSuccess;
    return rc;
}

}  // namespace guffin

using namespace guffin;

extern "C" int guffin_hip_rms_norm(void* stream, const float* x, uint32_t planes, uint64_t plane_stride,
                                   const float* gamma, const float* residual, float* y, float* y_sums,
                                   uint32_t rows, uint32_t width, float eps, uint32_t* status) {
    if (!x || !gamma || !y) return fail(GUFFIN_E_ARG, "rms_norm: null pointer");
    if (rows == 0 || width == 0 || planes == 0) return fail(GUFFIN_E_SHAPE, "rms_norm: empty shape");
    if (y_sums && (width % 32 != 0 || rows > 2)) return fail(GUFFIN_E_SHAPE, "rms_norm: a receipt needs width % 32 == 0 and rows <= 2");
    if (reinterpret_cast<uintptr_t>(y_sums) & 255u) return fail(GUFFIN_E_ALIGN, "rms_norm: the receipt must be 256-byte aligned");
    if (!(eps > 0.f)) return fail(GUFFIN_E_ARG, "rms_norm: epsilon must be positive");
    if (!aligned4(x) || !aligned4(y) || !aligned4(gamma)) return fail(GUFFIN_E_ALIGN, "rms_norm: fp32 pointers must be 4-byte aligned");
    const size_t lds = (size_t(width) + 16) * 4;
    if (lds > 160 * 1024) return fail(GUFFIN_E_CAPACITY, "rms_norm: row does not fit in LDS");
    launch(rms_norm_kernel, dim3(rows), dim3(norm_threads(width)), lds, as_stream(stream), x, planes,
                       static_cast<size_t>(plane_stride), gamma, residual, y, y_sums, width, eps, status);
    return check_launch("rms_norm");
}

extern "C" int guffin_hip_rms_norm_add_norm(void* stream, const float* x, uint32_t planes, uint64_t plane_stride,
                                            const float* gamma_post, const float* residual, float* out_residual,
                                            const float* gamma_next, float* out_norm, float* out_sums,
                                            uint32_t rows, uint32_t width, float eps, uint32_t* status) {
    if (!x || !gamma_post || !residual || !out_residual || !gamma_next || !out_norm)
        return fail(GUFFIN_E_ARG, "rms_norm_add_norm: null pointer");
    if (rows == 0 || width == 0 || planes == 0) return fail(GUFFIN_E_SHAPE, "rms_norm_add_norm: empty shape");
    if (out_sums && (width % 32 != 0 || rows > 2)) return fail(GUFFIN_E_SHAPE, "rms_norm_add_norm: a receipt needs width % 32 == 0 and rows <= 2");
    if (reinterpret_cast<uintptr_t>(out_sums) & 255u) return fail(GUFFIN_E_ALIGN, "rms_norm_add_norm: the receipt must be 256-byte aligned");
    if (!(eps > 0.f)) return fail(GUFFIN_E_ARG, "rms_norm_add_norm: epsilon must be positive");
    auto a16 = [](const void* q) { return (reinterpret_cast<uintptr_t>(q) & 15u) == 0; };
    if (planes <= uint32_t(kFastPlanes) && width % 8 == 0 && width / 8 <= 1024 && (!out_sums || width % 32 == 0)
        && plane_stride % 4 == 0 && a16(x) && a16(gamma_post) && a16(residual) && a16(out_residual) && a16(gamma_next) && a16(out_norm)) {
        const uint32_t threads = (width / 8 + 63) / 64 * 64;
        launch(rms_norm_add_norm_regs_kernel, dim3(rows), dim3(threads), 0, as_stream(stream), x, planes,
                           static_cast<size_t>(plane_stride), gamma_post, residual, out_residual, gamma_next, out_norm,
                           out_sums, width, eps, status);
        return check_launch("rms_norm_add_norm");
    }
    const size_t lds = (size_t(width) + 16) * 4;
    if (lds > 160 * 1024) return fail(GUFFIN_E_CAPACITY, "rms_norm_add_norm: row does not fit in LDS");
    launch(rms_norm_add_norm_kernel, dim3(rows), dim3(norm_threads(width)), lds, as_stream(stream), x, planes,
                       static_cast<size_t>(plane_stride), gamma_post, residual, out_residual, gamma_next,
                       out_norm, out_sums, width, eps, status);
    return check_launch("rms_norm_add_norm");
}

extern "C" int guffin_hip_head_rms_norm(void* stream, const float* x, const float* gamma, float* y,
                                        uint32_t rows, uint32_t heads, uint32_t head_dim, float eps) {
    if (!x || !gamma || !y) return fail(GUFFIN_E_ARG, "head_rms_norm: null pointer");
    if (rows == 0 || heads == 0 || head_dim == 0) return fail(GUFFIN_E_SHAPE, "head_rms_norm: empty shape");
    if (!(eps > 0.f)) return fail(GUFFIN_E_ARG, "head_rms_norm: epsilon must be positive");
    launch(head_rms_norm_kernel, dim3(rows * heads), dim3(64), 0, as_stream(stream), x, gamma, y, head_dim, eps);
    return check_launch("head_rms_norm");
}

static int launch_qkv(void* stream, const QkvArgs& a) {
    if (!a.positions && !a.rope_table) return fail(GUFFIN_E_ARG, "rope/kv: null positions");
    if (a.rows == 0 || a.head_dim == 0 || a.head_dim > 4096) return fail(GUFFIN_E_SHAPE, "rope/kv: bad head shape");
    if (a.rope_dim > a.head_dim || (a.rope_dim & 1u)) return fail(GUFFIN_E_SHAPE, "rope/kv: rope_dim must be even and <= head_dim");
    if (a.rope_dim && !a.rope_table && !(a.base > 0.f)) return fail(GUFFIN_E_ARG, "rope/kv: frequency base must be positive");
    const uint32_t blocks = a.rows * (a.q_heads + 2 * a.kv_heads);
    if (blocks == 0) return fail(GUFFIN_E_SHAPE, "rope/kv: no heads");
    launch(qkv_post_kernel, dim3(blocks), dim3(64), a.head_dim * sizeof(float), as_stream(stream), a);
    return check_launch("qkv_post");
}

extern "C" int guffin_hip_rope_neox(void* stream, const float* in, const uint32_t* positions, float* out,
                                    uint32_t rows, uint32_t heads, uint32_t head_dim, uint32_t rope_dim,
                                    float freq_base, float freq_scale) {
    if (!in || !out) return fail(GUFFIN_E_ARG, "rope_neox: null pointer");
    QkvArgs a {};
    a.q_raw = in; a.q_planes = 1; a.positions = positions; a.q_out = out;
    a.rows = rows; a.q_heads = heads; a.kv_heads = 0; a.head_dim = head_dim; a.rope_dim = rope_dim;
    a.base = freq_base; a.scale = freq_scale; a.eps = 1e-6f;
    return launch_qkv(stream, a);
}

extern "C" int guffin_hip_kv_store_f16(void* stream, const float* raw_k, const float* raw_v, const uint32_t* positions,
                                       void* out_k, void* out_v, uint32_t rows, uint32_t heads, uint32_t head_dim,
                                       uint32_t rope_dim, float freq_base, float freq_scale, uint32_t* status) {
    if (!raw_k || !raw_v || !out_k || !out_v) return fail(GUFFIN_E_ARG, "kv_store_f16: null pointer");
    QkvArgs a {};
    a.k_raw = raw_k; a.v_raw = raw_v; a.k_planes = a.v_planes = 1; a.positions = positions;
    a.k_out = static_cast<uint16_t*>(out_k); a.v_out = static_cast<uint16_t*>(out_v);
    a.rows = rows; a.q_heads = 0; a.kv_heads = heads; a.head_dim = head_dim; a.rope_dim = rope_dim;
    a.base = freq_base; a.scale = freq_scale; a.eps = 1e-6f; a.status = status;
    return launch_qkv(stream, a);
}

extern "C" int guffin_hip_qkv_post(void* stream, const float* q_raw, const float* k_raw, const float* v_raw,
                                   uint32_t q_planes, uint32_t k_planes, uint32_t v_planes,
                                   uint64_t q_plane_stride, uint64_t k_plane_stride,
                                   uint64_t v_plane_stride, const float* q_norm, const float* k_norm,
                                   const uint32_t* positions, float* q_out, void* k_out, void* v_out,
                                   uint32_t rows, uint32_t q_heads, uint32_t kv_heads, uint32_t head_dim,
                                   uint32_t rope_dim, float freq_base, float freq_scale, float eps,
                                   const float* rope_table, uint32_t* status) {
    if (!q_raw || !k_raw || !v_raw || !q_out || !k_out || !v_out) return fail(GUFFIN_E_ARG, "qkv_post: null pointer");
    if (!rope_table && !positions) return fail(GUFFIN_E_ARG, "qkv_post: need positions or a rope table");
    if (q_planes == 0 || k_planes == 0 || v_planes == 0) return fail(GUFFIN_E_SHAPE, "qkv_post: planes must be >= 1");
    if (!(eps > 0.f)) return fail(GUFFIN_E_ARG, "qkv_post: epsilon must be positive");
    QkvArgs a {};
    a.q_raw = q_raw; a.k_raw = k_raw; a.v_raw = v_raw; a.q_planes = q_planes; a.k_planes = k_planes; a.v_planes = v_planes;
    a.q_plane_stride = q_plane_stride; a.k_plane_stride = k_plane_stride; a.v_plane_stride = v_plane_stride;
    a.q_norm = q_norm; a.k_norm = k_norm; a.positions = positions;
    a.q_out = q_out; a.k_out = static_cast<uint16_t*>(k_out); a.v_out = static_cast<uint16_t*>(v_out);
    a.rows = rows; a.q_heads = q_heads; a.kv_heads = kv_heads; a.head_dim = head_dim; a.rope_dim = rope_dim;
    a.base = freq_base; a.scale = freq_scale; a.eps = eps; a.status = status;
    a.rope_table = reinterpret_cast<const float2*>(rope_table);
    return launch_qkv(stream, a);
}

extern "C" int guffin_hip_rope_table(void* stream, const uint32_t* positions, float* table, uint32_t rows,
                                     uint32_t rope_dim, float freq_base, float freq_scale) {
    if (!positions || !table) return fail(GUFFIN_E_ARG, "rope_table: null pointer");
    if (rows == 0 || rope_dim == 0 || rope_dim % 2) return fail(GUFFIN_E_SHAPE, "rope_table: rope_dim must be even and rows >= 1");
    if (reinterpret_cast<uintptr_t>(table) & 7u) return fail(GUFFIN_E_ALIGN, "rope_table: table must be 8-byte aligned");
    const uint32_t n = rows * (rope_dim / 2);
    launch(rope_table_kernel, dim3((n + 63) / 64), dim3(64), 0, as_stream(stream), positions,
                       reinterpret_cast<float2*>(table), rows, rope_dim, freq_base, freq_scale);
    return check_launch("rope_table");
}

extern "C" int guffin_hip_geglu(void* stream, const float* gate, const float* up, uint32_t planes, uint64_t plane_stride,
                                float* out, float* out_sums, uint32_t rows, uint32_t width) {
    if (!gate || !up || !out) return fail(GUFFIN_E_ARG, "geglu: null pointer");
    if (rows == 0 || width == 0 || planes == 0) return fail(GUFFIN_E_SHAPE, "geglu: empty shape");
    if (out_sums && (width % 32 != 0 || rows > 2)) return fail(GUFFIN_E_SHAPE, "geglu: a receipt needs width % 32 == 0 and rows <= 2");
    if (reinterpret_cast<uintptr_t>(out_sums) & 255u) return fail(GUFFIN_E_ALIGN, "geglu: the receipt must be 256-byte aligned");
    // chunks of 512 columns (a multiple of 32) per workgroup
    const uint32_t chunk = 512, chunks = (width + chunk - 1) / chunk;
    const uint32_t per = out_sums ? chunk : (width + chunks - 1) / chunks;
    const uint32_t gx = (width + per - 1) / per;
    launch(geglu_kernel, dim3(gx, rows), dim3(256), out_sums ? per * sizeof(float) : 0, as_stream(stream),
                       gate, up, planes, static_cast<size_t>(plane_stride), out, out_sums, width);
    return check_launch("geglu");
}

extern "C" int guffin_hip_embed(void* stream, int dtype, const void* w, const uint32_t* tokens, float* out,
                                uint32_t rows, uint32_t width, float scale, uint32_t vocab, uint32_t* status) {
    if (!w || !tokens || !out) return fail(GUFFIN_E_ARG, "embed: null pointer");
    if (dtype < GUFFIN_Q8_0 || dtype > GUFFIN_Q6_K) return fail(GUFFIN_E_ARG, "embed: unknown dtype");
    const uint32_t be = dtype == GUFFIN_Q8_0 ? 32u : 256u;
    if (rows == 0 || width == 0 || width % be != 0 || vocab == 0) return fail(GUFFIN_E_SHAPE, "embed: bad shape");
    if (reinterpret_cast<uintptr_t>(w) & 1u) return fail(GUFFIN_E_ALIGN, "embed: weights must be 2-byte aligned");
    const uint8_t* wb = static_cast<const uint8_t*>(w);
    hipStream_t s = as_stream(stream);
    if (dtype == GUFFIN_Q8_0) launch(embed_kernel<GUFFIN_Q8_0>, dim3(rows), dim3(256), 0, s, wb, tokens, out, width, scale, vocab, status);
    else if (dtype == GUFFIN_Q4_K) launch(embed_kernel<GUFFIN_Q4_K>, dim3(rows), dim3(256), 0, s, wb, tokens, out, width, scale, vocab, status);
    else launch(embed_kernel<GUFFIN_Q6_K>, dim3(rows), dim3(256), 0, s, wb, tokens, out, width, scale, vocab, status);
    return check_launch("embed");
}

extern "C" int guffin_hip_kv_scatter(void* stream, const void* priv_k, const void* priv_v, const uint32_t* selected,
                                     void* ring_k, void* ring_v, uint32_t position, uint32_t rows,
                                     uint32_t row_width, uint32_t ring_mask) {
    if (!priv_k || !priv_v || !selected || !ring_k || !ring_v) return fail(GUFFIN_E_ARG, "kv_scatter: null pointer");
    if (rows == 0 || row_width == 0) return fail(GUFFIN_E_SHAPE, "kv_scatter: empty shape");
    if ((ring_mask & (ring_mask + 1)) != 0) return fail(GUFFIN_E_ARG, "kv_scatter: ring capacity must be a power of two");
    launch(kv_scatter_kernel, dim3((row_width + 255) / 256, rows), dim3(256), 0, as_stream(stream),
                       static_cast<const uint16_t*>(priv_k), static_cast<const uint16_t*>(priv_v), selected,
                       static_cast<uint16_t*>(ring_k), static_cast<uint16_t*>(ring_v), position, rows, row_width, ring_mask);
    return check_launch("kv_scatter");
}
