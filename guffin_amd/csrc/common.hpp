// Shared device helpers for the gfx950 kernels of the H1 step.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/guffin_hip.h"
#include "chain.hpp"

namespace guffin {

constexpr int kWave = 64;

// ---- error plumbing (host) -------------------------------------------------
void set_last_error(const char* message);
int fail(int code, const char* message);
int check_launch(const char* what);

inline hipStream_t as_stream(void* s) { return reinterpret_cast<hipStream_t>(s); }

// Layer policy of src/engine/model.cpp:607-610: with a period above one, every layer but the last of
// each period uses the sliding window (local ring, local rotation base); otherwise every layer is global.
__host__ __device__ inline bool layer_is_local(uint32_t global_period, uint32_t layer) {
    return global_period > 1 && (layer % global_period) != global_period - 1;
}

// ---- resident forward pass (resident.hip), used by the block graph of plan.hip ------------------
constexpr uint32_t kResidentLayers = 6;   // blocks per launch (their pointers travel as kernel arguments)
extern uint32_t g_spin_limit;
extern unsigned long long* g_resident_stamps;
extern int g_forward_mode;
bool resident_fits(const guffin_model_desc& m, uint32_t rows);
// Whether forward_rows runs the resident pass for this model now: the model fits, the mode asks for it (2) or leaves
// the choice open (0) for a model with one KV head, and no earlier pass of this process gave up a wait.
bool resident_chosen(const guffin_model_desc& m, uint32_t rows);
// Host code that reads a device status word reports it here: GUFFIN_STATUS_SYNC switches the automatic choice of
// the resident pass off for the rest of the process (a device shared with other work, or one whose dispatcher does
// not place the workgroups as the pass assumes, would raise it on every pass).
void resident_note_status(uint32_t status_word);
int resident_init(int cu_count);
uint64_t resident_scratch_bytes(const guffin_model_desc& m, uint32_t rows);
uint32_t resident_sync_words(const guffin_model_desc& m);
int resident_launch(hipStream_t stream, const guffin_model_desc& m, uint32_t rows, uint32_t first, uint32_t count,
                    uint8_t* exchange, uint32_t* sync_words, const float* rope_local, const float* rope_global,
                    const uint32_t* schedule, const uint32_t* ancestors, void* priv_k, void* priv_v, const float* x_in,
                    const void* u_receipt_in, float* x_out, float* u_out, void* u_receipt_out, uint32_t max_ring_tokens,
                    uint32_t* status);

// ---- attention with a host-known schedule (attention.hip), used by the block graph of plan.hip --------
int qkv_attention_scheduled(void* stream, const float* q_raw, const float* k_raw, const float* v_raw, uint32_t planes,
                            uint64_t q_plane_stride, uint64_t k_plane_stride, uint64_t v_plane_stride, const float* q_norm,
                            const float* k_norm, const float* rope_table, float eps, const void* ring_k, const void* ring_v,
                            void* priv_k, void* priv_v, const uint32_t* schedule, const uint32_t* ancestors,
                            const uint32_t* host_schedule, const uint32_t* host_amask, float* out, float* out_sums,
                            float* partial_out, float* partial_ml, uint32_t rows, uint32_t max_tokens, uint32_t ring_mask,
                            uint32_t q_heads, uint32_t kv_heads, uint32_t head_dim, float scale, uint32_t* status);

// ---- typed loads at the alignment a GGUF block stream guarantees ------------
struct __attribute__((packed, aligned(4))) U4a4 { uint32_t x, y, z, w; };
struct __attribute__((packed, aligned(2))) U4a2 { uint32_t x, y, z, w; };
struct __attribute__((packed, aligned(2))) U2a2 { uint32_t x, y; };
struct __attribute__((packed, aligned(4))) F4a4 { float x, y, z, w; };

__device__ __forceinline__ uint4 ld16_a4(const uint8_t* p) {
    const U4a4 t = *reinterpret_cast<const U4a4*>(p);
    return make_uint4(t.x, t.y, t.z, t.w);
}
__device__ __forceinline__ uint4 ld16_a2(const uint8_t* p) {
    const U4a2 t = *reinterpret_cast<const U4a2*>(p);
    return make_uint4(t.x, t.y, t.z, t.w);
}
__device__ __forceinline__ uint2 ld8_a2(const uint8_t* p) {
    const U2a2 t = *reinterpret_cast<const U2a2*>(p);
    return make_uint2(t.x, t.y);
}
__device__ __forceinline__ float4 ldf4_a4(const float* p) {
    const F4a4 t = *reinterpret_cast<const F4a4*>(p);
    return make_float4(t.x, t.y, t.z, t.w);
}
__device__ __forceinline__ uint32_t ld_u16(const uint8_t* p) { return *reinterpret_cast<const uint16_t*>(p); }

// fp16 bits -> fp32, exact (IEEE widening, subnormals included)
__device__ __forceinline__ float h2f(uint32_t bits) {
    return static_cast<float>(__builtin_bit_cast(_Float16, static_cast<unsigned short>(bits)));
}

// Hides a value from the optimiser so that a following (v >> 8k) & 0xFF selects
// v_cvt_f32_ubyteK instead of being re-derived from the unmasked source.
__device__ __forceinline__ uint32_t opaque(uint32_t v) {
    asm volatile("" : "+v"(v));
    return v;
}
__device__ __forceinline__ float ub0(uint32_t v) { return static_cast<float>(v & 0xFFu); }
__device__ __forceinline__ float ub1(uint32_t v) { return static_cast<float>((v >> 8) & 0xFFu); }
__device__ __forceinline__ float ub2(uint32_t v) { return static_cast<float>((v >> 16) & 0xFFu); }
__device__ __forceinline__ float ub3(uint32_t v) { return static_cast<float>(v >> 24); }
__device__ __forceinline__ float sb0(uint32_t v) { return static_cast<float>(static_cast<int8_t>(v)); }
__device__ __forceinline__ float sb1(uint32_t v) { return static_cast<float>(static_cast<int8_t>(v >> 8)); }
__device__ __forceinline__ float sb2(uint32_t v) { return static_cast<float>(static_cast<int8_t>(v >> 16)); }
__device__ __forceinline__ float sb3(uint32_t v) { return static_cast<float>(static_cast<int8_t>(v >> 24)); }

// Sums and maxima over the 16 lanes of a row on the vector unit's lane-crossing modifiers (two quad permutations,
// then the mirror of 8 and of 16 lanes: every lane ends with the row's total), and over the wave with two more
// steps through the LDS crossbar.  A crossbar shuffle costs a wave that is alone on its SIMD more than a hundred
// cycles, and the reductions sit in dependent chains; every lane of the wave must be active.
template <int CTRL>
__device__ __forceinline__ float lane_cross(float v) {   // a lane outside the modifier's reach reads 0
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, true));
}
__device__ __forceinline__ float row16_sum(float v) {
    v += lane_cross<0xB1>(v);    // quad_perm [1,0,3,2]
    v += lane_cross<0x4E>(v);    // quad_perm [2,3,0,1]
    v += lane_cross<0x141>(v);   // row_half_mirror
    v += lane_cross<0x140>(v);   // row_mirror
    return v;
}
__device__ __forceinline__ float row16_max(float v) {
    v = fmaxf(v, lane_cross<0xB1>(v));
    v = fmaxf(v, lane_cross<0x4E>(v));
    v = fmaxf(v, lane_cross<0x141>(v));
    v = fmaxf(v, lane_cross<0x140>(v));
    return v;
}
// Inclusive prefix sum over the 64 lanes, the same way: four shifts inside the rows of 16 (a lane past the row's
// start reads 0), then lane 15's total into the next row and lane 31's into the upper half.
template <int CTRL, int ROWS>
__device__ __forceinline__ uint32_t lane_cross_u32(uint32_t v) {
    return static_cast<uint32_t>(__builtin_amdgcn_update_dpp(0, static_cast<int>(v), CTRL, ROWS, 0xF, ROWS == 0xF));
}
__device__ __forceinline__ uint32_t wave_inclusive_scan(uint32_t v) {
    v += lane_cross_u32<0x111, 0xF>(v);   // row_shr:1
    v += lane_cross_u32<0x112, 0xF>(v);   // row_shr:2
    v += lane_cross_u32<0x114, 0xF>(v);   // row_shr:4
    v += lane_cross_u32<0x118, 0xF>(v);   // row_shr:8
    v += lane_cross_u32<0x142, 0xA>(v);   // row_bcast:15 into rows 1 and 3
    v += lane_cross_u32<0x143, 0xC>(v);   // row_bcast:31 into rows 2 and 3
    return v;
}
__device__ __forceinline__ uint32_t wave_max_u32(uint32_t v) {
    v = max(v, lane_cross_u32<0xB1, 0xF>(v));
    v = max(v, lane_cross_u32<0x4E, 0xF>(v));
    v = max(v, lane_cross_u32<0x141, 0xF>(v));
    v = max(v, lane_cross_u32<0x140, 0xF>(v));
    v = max(v, static_cast<uint32_t>(__shfl_xor(static_cast<int>(v), 16, kWave)));
    return max(v, static_cast<uint32_t>(__shfl_xor(static_cast<int>(v), 32, kWave)));
}

__device__ __forceinline__ float wave_sum(float v) {
    v = row16_sum(v);
    v += __shfl_xor(v, 16, kWave);
    return v + __shfl_xor(v, 32, kWave);
}
__device__ __forceinline__ float wave_max(float v) {
    v = row16_max(v);
    v = fmaxf(v, __shfl_xor(v, 16, kWave));
    return fmaxf(v, __shfl_xor(v, 32, kWave));
}

// Sum of `planes` partial planes in plane order; loads are issued four at a time so that the
// adds, not the memory latency, form the dependent chain.
__device__ __forceinline__ float load_planes(const float* p, uint32_t planes, size_t plane_stride) {
    float v = p[0];
    uint32_t s = 1;
    for (; s + 4 <= planes; s += 4) {
        const float a = p[s * plane_stride], b = p[(s + 1) * plane_stride], c = p[(s + 2) * plane_stride],
                    d = p[(s + 3) * plane_stride];
        v += a; v += b; v += c; v += d;
    }
    for (; s < planes; ++s) v += p[s * plane_stride];
    return v;
}

// Reduces NV per-lane values across the 64 lanes with NV-1 + (6 - log2 NV) exchanges
// instead of 6*NV: at each level the upper half-wave keeps one half of the values and
// the lower half-wave the other.  Afterwards v[0] on lane l holds the wave total of
// value index l >> (6 - log2 NV); the summation order is fixed, so results repeat.
template <int NV>
__device__ __forceinline__ void wave_reduce_multi(float (&v)[NV], int lane) {
    static_assert(NV >= 1 && NV <= 64 && (NV & (NV - 1)) == 0, "NV must be a power of two");
    int stride = 32;
#pragma unroll
    for (int m = NV; m > 1; m >>= 1) {
        const int half = m >> 1;
        const bool upper = (lane & stride) != 0;
#pragma unroll
        for (int i = 0; i < half; ++i) {
            const float send = upper ? v[i] : v[i + half];
            const float keep = upper ? v[i + half] : v[i];
            v[i] = keep + __shfl_xor(send, stride, kWave);
        }
        stride >>= 1;
    }
#pragma unroll
    for (; stride > 0; stride >>= 1) v[0] += __shfl_xor(v[0], stride, kWave);
}

template <int NV>
__device__ __forceinline__ constexpr int reduce_multi_shift() {
    int s = 6, n = NV;
    while (n > 1) { n >>= 1; --s; }
    return s;
}

// cos and sin of the NeoX rotation of (position, pair)
__device__ __forceinline__ void rope_sincos(uint32_t position, uint32_t pair, uint32_t rope_dim, float base,
                                            float scale, float& c, float& s) {
    // angle in double, as the CPU operator forms it (rope.cpp:109-117), times the layer's frequency scale
    const double exponent = static_cast<double>(2u * pair) / static_cast<double>(rope_dim);
    const double angle = static_cast<double>(position) / pow(static_cast<double>(base), exponent)
        * static_cast<double>(scale);
    c = static_cast<float>(cos(angle));
    s = static_cast<float>(sin(angle));
}

}  // namespace guffin
