// Chunked prefill on the matrix core (gfx950): M rows x quantised weights, and causal GQA
// attention over the fp16 KV rings for a run of consecutive positions.
//
// Replaces the reference's prefill matrix path (src/tensor/backends/metal/metal_kernels.mm:
// 1031-1199, dispatch rules metal_command_context.mm:384-401) and encode_f16_prefill_attention
// (metal_command_context.hpp:185, kernels metal_kernels.mm:2593-2800).
//
// GEMM.  Same wave tiles and the same exact-operand idea as the packed GEMV: quants enter
// v_mfma_f32_16x16x32_f16 as fp16 subnormals (B), activations as an fp16 hi/lo image (A).  With
// many rows the 16 A rows are 8 activation rows x {hi, lo}, so nothing is replicated: after
// one MFMA lane (j, g) holds, for column 16*cg + j, rows 2g and 2g+1 of the row group as
// (hi, lo) pairs.  A wave owns 32 rows (4 row groups) of 64 columns (Q4_K, Q8_0) or 32 columns
// (Q6_K).  For Q8_0 a workgroup is 4 waves on the same tile (128 rows), each loading its own
// operands; for Q4_K it is 4 waves on 4 neighbouring tiles and the same 32 rows, for Q6_K 4 waves
// on the halves of 2 neighbouring tiles, which share the A operands through LDS (the vector
// memory path, not the matrix core, bounds the kernel that does not).  The K-quants fold their
// scales into B (Q4_K: sc * q <= 945; Q6_K: |scale| times the low four and the high two bits of q,
// sign in bit 15 -- all still exact fp16 bit patterns) and accumulate a whole 256-element block
// inside the MFMA chain; Q8_0 applies the block scale and the activation multiplier to each MFMA
// result in fp32.  The offset terms (-dmin m, -32 d scale) are one more MFMA per block on an image
// of the block's group sums (Q6_K: half-group sums); Q8_0 uses per-(row, 32-group) sums in fp32.
//
// Attention.  A workgroup serves 16 consecutive query rows of one KV head (all query heads of the
// group) and walks the visible key range in tiles of 32 tokens through LDS with an online
// softmax, fp32 math on fp16 keys/values: positions before the run come from the ring, the run's
// own positions from its private rows, which are published to the ring afterwards.
#include "common.hpp"

namespace guffin {
namespace {

typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef float float4_t __attribute__((ext_vector_type(4)));

constexpr uint32_t kCols = 64;       // columns per wave tile
constexpr uint32_t kWaveRows = 32;   // rows per wave (4 row groups of 8)
constexpr uint32_t kChunkRows = 128; // rows per workgroup

__host__ __device__ constexpr uint32_t block_bytes(int dtype) {
    return dtype == GUFFIN_Q8_0 ? 34u : dtype == GUFFIN_Q4_K ? 144u : 210u;
}
__host__ __device__ constexpr uint32_t block_elems(int dtype) { return dtype == GUFFIN_Q8_0 ? 32u : 256u; }

// ---- activation image of M rows --------------------------------------------------------
// image: half [K/32][Mpad/8][16][32]   A row 2*(row % 8) + {0 hi, 1 lo}; inside a group the halves
//                                      of elements 8s..8s+7 sit at 8s + {0,2,1,3,4,6,5,7}
// mult : float [K/32][Mpad]            2^(E+24) of (row, group); E is shared by the 8 groups of a
//                                      256-element block when K is a multiple of 256
// s32  : float [K/32][Mpad]            sum of the group's 32 activations
// sumi : half  [K/256][Mpad/8][16][8]   (K % 256 == 0) the 8 group sums of a block as an A operand:
//                                      same A rows, halves of groups t at {0,2,1,3,4,6,5,7}[t]
// smul : float [K/256][Mpad]           2^(Es+24) of (row, block) for sumi
// sumh : half  [K/256][Mpad/8][16][16]  (K % 256 == 0) the 16 half-group sums of a block as an A
//                                      operand: same A rows, the sum of elements 16t..16t+15 at t
// shml : float [K/256][Mpad]           2^(Eh+24) of (row, block) for sumh
struct ImageLayout { size_t mult_off, s32_off, sumi_off, smul_off, sumh_off, shml_off, bytes; uint32_t mpad; };

__host__ __device__ inline ImageLayout image_layout(uint32_t M, uint32_t K) {
    const uint32_t mpad = (M + kChunkRows - 1) / kChunkRows * kChunkRows;
    ImageLayout L {};
    L.mpad = mpad;
    L.mult_off = size_t(K / 32) * mpad * 128;  // 16 A rows x 64 B per 8 rows = 128 B per row and group
    L.s32_off = L.mult_off + size_t(K / 32) * mpad * 4;
    L.sumi_off = L.s32_off + size_t(K / 32) * mpad * 4;
    L.smul_off = L.sumi_off + size_t(K / 256) * mpad * 32;   // 16 A rows x 16 B per 8 rows
    L.sumh_off = L.smul_off + size_t(K / 256) * mpad * 4;
    L.shml_off = L.sumh_off + size_t(K / 256) * mpad * 64;   // 16 A rows x 32 B per 8 rows
    L.bytes = L.shml_off + size_t(K / 256) * mpad * 4;
    return L;
}

// one thread per (row, group, k-slice); four consecutive lanes share a group
__global__ void __launch_bounds__(256)
prefill_pack_kernel(const float* __restrict__ x, uint8_t* __restrict__ blob, uint32_t M, uint32_t K) {
    const ImageLayout L = image_layout(M, K);
    const uint32_t groups = K / 32;
    const uint64_t t = uint64_t(blockIdx.x) * blockDim.x + threadIdx.x;
    if (t >= uint64_t(L.mpad) * groups * 4) return;
    const uint32_t s = t & 3u, g = (t >> 2) % groups, row = static_cast<uint32_t>((t >> 2) / groups);
    float v[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) v[i] = row < M ? x[size_t(row) * K + g * 32 + s * 8 + i] : 0.f;
    float sum = v[0], m = fabsf(v[0]);
#pragma unroll
    for (int i = 1; i < 8; ++i) { sum += v[i]; m = fmaxf(m, fabsf(v[i])); }
    m = fmaxf(m, __shfl_xor(m, 1, kWave));
    m = fmaxf(m, __shfl_xor(m, 2, kWave));
    if (K % 256 == 0) {  // one exponent per 256 elements (32 consecutive threads): K-quant blocks
        m = fmaxf(m, __shfl_xor(m, 4, kWave));
        m = fmaxf(m, __shfl_xor(m, 8, kWave));
        m = fmaxf(m, __shfl_xor(m, 16, kWave));
    }
    const float sum16 = sum + __shfl_xor(sum, 1, kWave);
    const float sum32 = sum16 + __shfl_xor(sum16, 2, kWave);
    uint32_t eb = __float_as_uint(m) >> 23;
    eb = eb < 14u ? 14u : eb > 244u ? 244u : eb;
    const float inv = __uint_as_float((268u - eb) << 23);
    float* mult = reinterpret_cast<float*>(blob + L.mult_off);
    float* s32 = reinterpret_cast<float*>(blob + L.s32_off);
    if (s == 0) { mult[size_t(g) * L.mpad + row] = __uint_as_float((eb + 10u) << 23); s32[size_t(g) * L.mpad + row] = sum32; }
    constexpr int order[8] = {0, 2, 1, 3, 4, 6, 5, 7};
    if (K % 256 == 0) {  // the block's 8 group sums as a second small A operand (hi/lo, own exponent)
        float sm = fabsf(sum32);
        sm = fmaxf(sm, __shfl_xor(sm, 4, kWave));
        sm = fmaxf(sm, __shfl_xor(sm, 8, kWave));
        sm = fmaxf(sm, __shfl_xor(sm, 16, kWave));
        uint32_t es = __float_as_uint(sm) >> 23;
        es = es < 14u ? 14u : es > 244u ? 244u : es;
        if (s == 0) {
            const float sv = sum32 * __uint_as_float((268u - es) << 23);
            const _Float16 h = static_cast<_Float16>(sv);
            const _Float16 l = static_cast<_Float16>(sv - static_cast<float>(h));
            const uint32_t blk = g >> 3, t8 = g & 7u;
            uint8_t* rec = blob + L.sumi_off + ((size_t(blk) * (L.mpad / 8) + row / 8) * 16 + 2 * (row % 8)) * 16 + order[t8] * 2;
            *reinterpret_cast<uint16_t*>(rec) = __builtin_bit_cast(uint16_t, h);
            *reinterpret_cast<uint16_t*>(rec + 16) = __builtin_bit_cast(uint16_t, l);
            if (t8 == 0) reinterpret_cast<float*>(blob + L.smul_off)[size_t(blk) * L.mpad + row] = __uint_as_float((es + 10u) << 23);
        }
        // and its 16 half-group sums (Q6_K scales cover 16 elements); lanes s and s ^ 1 hold the same sum
        float sh = fabsf(sum16);
        sh = fmaxf(sh, __shfl_xor(sh, 2, kWave));
        sh = fmaxf(sh, __shfl_xor(sh, 4, kWave));
        sh = fmaxf(sh, __shfl_xor(sh, 8, kWave));
        sh = fmaxf(sh, __shfl_xor(sh, 16, kWave));
        uint32_t eh = __float_as_uint(sh) >> 23;
        eh = eh < 14u ? 14u : eh > 244u ? 244u : eh;
        if ((s & 1u) == 0) {
            const float sv = sum16 * __uint_as_float((268u - eh) << 23);
            const _Float16 h = static_cast<_Float16>(sv);
            const _Float16 l = static_cast<_Float16>(sv - static_cast<float>(h));
            const uint32_t blk = g >> 3, t16 = 2 * (g & 7u) + (s >> 1);
            uint8_t* rec = blob + L.sumh_off + ((size_t(blk) * (L.mpad / 8) + row / 8) * 16 + 2 * (row % 8)) * 32 + t16 * 2;
            *reinterpret_cast<uint16_t*>(rec) = __builtin_bit_cast(uint16_t, h);
            *reinterpret_cast<uint16_t*>(rec + 32) = __builtin_bit_cast(uint16_t, l);
            if (t16 == 0) reinterpret_cast<float*>(blob + L.shml_off)[size_t(blk) * L.mpad + row] = __uint_as_float((eh + 10u) << 23);
        }
    }
    uint32_t hi[4], lo[4];
#pragma unroll
    for (int p = 0; p < 4; ++p) {
        uint32_t hw = 0, lw = 0;
#pragma unroll
        for (int q = 0; q < 2; ++q) {
            const float xv = v[order[2 * p + q]] * inv;
            const _Float16 h = static_cast<_Float16>(xv);
            const _Float16 l = static_cast<_Float16>(xv - static_cast<float>(h));
            hw |= uint32_t(__builtin_bit_cast(uint16_t, h)) << (16 * q);
            lw |= uint32_t(__builtin_bit_cast(uint16_t, l)) << (16 * q);
        }
        hi[p] = hw; lo[p] = lw;
    }
    uint8_t* base = blob + ((size_t(g) * (L.mpad / 8) + row / 8) * 16 + 2 * (row % 8)) * 64 + s * 16;
    *reinterpret_cast<uint4*>(base) = make_uint4(hi[0], hi[1], hi[2], hi[3]);
    *reinterpret_cast<uint4*>(base + 64) = make_uint4(lo[0], lo[1], lo[2], lo[3]);
}

__device__ __forceinline__ half8_t as_half8(uint32_t a, uint32_t b, uint32_t c, uint32_t d) {
    return __builtin_bit_cast(half8_t, make_uint4(a, b, c, d));
}
__device__ __forceinline__ uint32_t even_bytes(uint32_t v) { return __builtin_amdgcn_perm(0u, v, 0x0c020c00u); }
__device__ __forceinline__ uint32_t odd_bytes(uint32_t v) { return __builtin_amdgcn_perm(0u, v, 0x0c030c01u); }
typedef unsigned short ushort2_t __attribute__((ext_vector_type(2)));
// products of the two 16-bit fields of a and b (v_pk_mul_lo_u16)
__device__ __forceinline__ uint32_t pk_mul(uint32_t a, uint32_t b) {
    return __builtin_bit_cast(uint32_t, __builtin_bit_cast(ushort2_t, a) * __builtin_bit_cast(ushort2_t, b));
}
// a * b + c on both 16-bit fields
__device__ __forceinline__ uint32_t pk_mad(uint32_t a, uint32_t b, uint32_t c) {
    // vector arithmetic rather than inline assembly: the compiler's hazard handling around matrix
    // instructions does not look into an asm statement
    return __builtin_bit_cast(uint32_t, __builtin_bit_cast(ushort2_t, a) * __builtin_bit_cast(ushort2_t, b)
                                            + __builtin_bit_cast(ushort2_t, c));
}

// what a wave needs of the image for one 32-group: the A operands of its 4 row groups and the
// multipliers / sums of the lane's two rows per row group
struct GroupOperands {
    half8_t a[4];
    float2 mult[4];
};

struct WaveCtx {
    const uint8_t* image;   // + lane offset inside a (group, row group) record
    const float* mult; const float* s32;
    uint32_t mpad, rg0, row0;  // first row group / first of the lane's rows of row group 0
};

__device__ __forceinline__ void load_group(const WaveCtx& c, uint32_t g, GroupOperands& o) {
#pragma unroll
    for (int rg = 0; rg < 4; ++rg) {
        o.a[rg] = __builtin_bit_cast(half8_t, *reinterpret_cast<const uint4*>(
            c.image + (size_t(g) * (c.mpad / 8) + c.rg0 + rg) * 1024));
        o.mult[rg] = *reinterpret_cast<const float2*>(c.mult + size_t(g) * c.mpad + c.row0 + 8 * rg);
    }
}

// acc[rg][2] += f * mult * (hi + lo sums) for the lane's two rows of every row group
__device__ __forceinline__ void mfma_scale(const GroupOperands& o, half8_t b, float f, float (&acc)[4][2]) {
    const float4_t zero = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int rg = 0; rg < 4; ++rg) {
        const float4_t d = __builtin_amdgcn_mfma_f32_16x16x32_f16(o.a[rg], b, zero, 0, 0, 0);
        acc[rg][0] = fmaf(f * o.mult[rg].x, d[0] + d[1], acc[rg][0]);
        acc[rg][1] = fmaf(f * o.mult[rg].y, d[2] + d[3], acc[rg][1]);
    }
}

__device__ __forceinline__ void add_offset(const float* sums, const WaveCtx& c, uint32_t index, float f, float (&acc)[4][2]) {
#pragma unroll
    for (int rg = 0; rg < 4; ++rg) {
        const float2 s = *reinterpret_cast<const float2*>(sums + size_t(index) * c.mpad + c.row0 + 8 * rg);
        acc[rg][0] = fmaf(f, s.x, acc[rg][0]);
        acc[rg][1] = fmaf(f, s.y, acc[rg][1]);
    }
}

// The image and the weight tile are read through buffer resources: an address is the resource
// (scalar registers) + a wave-uniform byte offset (a scalar register) + the lane's 32-bit offset,
// so a load costs one address register however many groups the loop walks.
typedef uint32_t uint4_t __attribute__((ext_vector_type(4)));

__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_resource(const void* base, uint32_t bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, static_cast<int>(bytes), 0x00020000);
}
__device__ __forceinline__ uint4 ld16(__amdgpu_buffer_rsrc_t r, uint32_t lane_off, uint32_t uniform_off) {
    const uint4_t v = __builtin_amdgcn_raw_buffer_load_b128(r, static_cast<int>(lane_off), static_cast<int>(uniform_off), 0);
    return make_uint4(v[0], v[1], v[2], v[3]);
}
__device__ __forceinline__ float2 ld8(__amdgpu_buffer_rsrc_t r, uint32_t lane_off, uint32_t uniform_off) {
    typedef uint32_t uint2_t __attribute__((ext_vector_type(2)));
    const uint2_t v = __builtin_amdgcn_raw_buffer_load_b64(r, static_cast<int>(lane_off), static_cast<int>(uniform_off), 0);
    return make_float2(__uint_as_float(v[0]), __uint_as_float(v[1]));
}

// the A operands of one 32-group for the wave's 4 row groups
struct GroupA { half8_t a[4]; };


// chunk CH (64 elements of K) of a Q4_K block: D[cg][rg] += A(lo group) * (sc * low nibbles) +
// A(hi group) * (sc * high nibbles); scw holds the scale bytes of chunks 0-1 or 2-3
template <int CH>
__device__ __forceinline__ void q4_chunk(const GroupA& lo, const GroupA& hi, const uint4 (&q)[8], const uint32_t (&scw)[4],
                                         float4_t (&D)[4][4]) {
    constexpr uint32_t M = 0x000F000Fu;
    // all low-nibble groups first, then all high-nibble groups: an accumulator is used again 16
    // matrix instructions later rather than 4
#pragma unroll
    for (int cg = 0; cg < 4; ++cg) {
        // the scale byte in both 16-bit fields
        const uint32_t pair_lo = __builtin_amdgcn_perm(0u, scw[cg], (CH & 1) ? 0x0c020c02u : 0x0c000c00u);
        const uint4 piece = q[2 * cg + (CH >> 1)];
        const uint32_t w0 = (CH & 1) ? piece.z : piece.x, w1 = (CH & 1) ? piece.w : piece.y;
        const half8_t blo = as_half8(pk_mul(w0 & M, pair_lo), pk_mul((w0 >> 8) & M, pair_lo),
                                     pk_mul(w1 & M, pair_lo), pk_mul((w1 >> 8) & M, pair_lo));
#pragma unroll
        for (int rg = 0; rg < 4; ++rg) D[cg][rg] = __builtin_amdgcn_mfma_f32_16x16x32_f16(lo.a[rg], blo, D[cg][rg], 0, 0, 0);
    }
#pragma unroll
    for (int cg = 0; cg < 4; ++cg) {
        const uint32_t pair_hi = __builtin_amdgcn_perm(0u, scw[cg], (CH & 1) ? 0x0c030c03u : 0x0c010c01u);
        const uint4 piece = q[2 * cg + (CH >> 1)];
        const uint32_t w0 = (CH & 1) ? piece.z : piece.x, w1 = (CH & 1) ? piece.w : piece.y;
        const half8_t bhi = as_half8(pk_mul((w0 >> 4) & M, pair_hi), pk_mul((w0 >> 12) & M, pair_hi),
                                     pk_mul((w1 >> 4) & M, pair_hi), pk_mul((w1 >> 12) & M, pair_hi));
#pragma unroll
        for (int rg = 0; rg < 4; ++rg) D[cg][rg] = __builtin_amdgcn_mfma_f32_16x16x32_f16(hi.a[rg], bhi, D[cg][rg], 0, 0, 0);
    }
    // one MFMA occupies the matrix pipe for four issue slots: the next column group's operands
    // are built in the other three
#pragma unroll
    for (int i = 0; i < 32; ++i) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x002, 3, 0);
    }
}

// Q4_K with the activations shared through LDS.  The four waves of a workgroup own four
// neighbouring column tiles and the SAME 32 rows: each wave fetches a quarter of a chunk's A
// operands (64 elements of K: a low-nibble and a high-nibble group x 4 row groups = 8 records of
// 1 KB) and all four read the whole chunk from LDS, which cuts the bytes that pass the vector
// memory path per MFMA by more than half -- that path, not the matrix core, bounds the kernel
// that loads every operand itself.  Three LDS buffers rotate: chunk c is read, c + 1 is complete,
// c + 2 is written after the one barrier of the step.  grid (Mpad/32, ceil(N/256)), 256 threads;
// consecutive workgroups walk the rows, so one XCD's L2 keeps an eighth of the image.
__device__ __forceinline__ void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

__global__ void __launch_bounds__(256, 2)
prefill_gemm_q4k_kernel(const uint8_t* __restrict__ tiles, const uint8_t* __restrict__ blob, float* __restrict__ y,
                        uint32_t M, uint32_t K, uint32_t N) {
    constexpr uint32_t TB = kCols * block_bytes(GUFFIN_Q4_K);
    constexpr uint32_t kStage = 8192;  // one chunk of A operands
    __shared__ __attribute__((aligned(16))) uint8_t stage[3 * kStage];
    const ImageLayout L = image_layout(M, K);
    const uint32_t lane = threadIdx.x & 63, wv = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t j = lane & 15, lg = lane >> 4;
    const uint32_t nblk = K / 256, nchunk = nblk * 4;
    const uint32_t wave_row = blockIdx.x * kWaveRows;
    if (wave_row >= M) return;  // padding rows only (the whole workgroup)
    const uint32_t tile_index = blockIdx.y * 4 + wv;
    const bool valid = tile_index < N / kCols;  // a wave past the last tile works on tile 0 and stores nothing
    // addresses into the image: the resource, a wave-uniform byte offset and the lane's offset
    struct { __amdgpu_buffer_rsrc_t blob; uint32_t image, mult, a_off, r_off, mpad, rg0, row0; } c;
    c.mpad = L.mpad;
    c.rg0 = wave_row / 8;
    c.row0 = wave_row + 2 * lg;
    c.a_off = j * 64 + lg * 16;  // A lane (i = lane % 16, s = lane / 16): row i, k-slice s
    c.r_off = 8 * lg;            // the lane's first row inside a row group, in bytes of a float row
    c.blob = make_resource(blob, static_cast<uint32_t>(L.bytes));
    c.image = c.rg0 * 1024;      // the wave's first row group of group 0
    c.mult = static_cast<uint32_t>(L.mult_off) + wave_row * 4;
    const uint32_t smul = static_cast<uint32_t>(L.smul_off) + wave_row * 4;
    const uint32_t sumi = static_cast<uint32_t>(L.sumi_off) + c.rg0 * 256;
    // the sums image fills k-slice 0 only: the other lanes read past the resource's end, which a
    // buffer load answers with zeros
    const uint32_t sums_off = lane < 16 ? lane * 16 : 0x80000000u;
    const __amdgpu_buffer_rsrc_t tile = make_resource(tiles + size_t(valid ? tile_index : 0) * nblk * TB, nblk * TB);
    // this wave's share of chunk n: row group wv of its two groups
    const uint32_t share = c.image + wv * 1024;
    auto fetch = [&](uint32_t n, uint4& lo, uint4& hi) {
        const uint32_t g = 2 * (n < nchunk ? n : nchunk - 1);  // past the end: the last chunk again, never read
        lo = ld16(c.blob, c.a_off, share + g * c.mpad * 128);
        hi = ld16(c.blob, c.a_off, share + (g + 1) * c.mpad * 128);
    };
    auto deposit = [&](uint32_t buffer, const uint4& lo, const uint4& hi) {
        *reinterpret_cast<uint4*>(stage + buffer * kStage + wv * 1024 + lane * 16) = lo;
        *reinterpret_cast<uint4*>(stage + buffer * kStage + 4096 + wv * 1024 + lane * 16) = hi;
    };
    float acc[4][4][2];  // [column group][row group][row of the lane]
#pragma unroll
    for (int cg = 0; cg < 4; ++cg)
#pragma unroll
        for (int rg = 0; rg < 4; ++rg) { acc[cg][rg][0] = 0.f; acc[cg][rg][1] = 0.f; }
    uint4 q[8], hd[4], slo, shi;
#pragma unroll
    for (int i = 0; i < 8; ++i) q[i] = ld16(tile, lane * 16, 1024 * i);
#pragma unroll
    for (int cg = 0; cg < 4; ++cg) hd[cg] = ld16(tile, j * 16, 8192 + 256 * cg);
    fetch(0, slo, shi); deposit(0, slo, shi);
    fetch(1, slo, shi); deposit(1, slo, shi);
    fetch(2, slo, shi);
    lds_barrier();  // chunks 0 and 1 are complete
    uint32_t rd = 0, wr = 2;  // buffers of the chunk to read and of the chunk to deposit
    float4_t D[4][4];
    uint32_t sc_a[4], sc_b[4];
    // one step: read chunk n's operands, barrier, deposit chunk n + 2, ask for chunk n + 3
    auto step = [&](uint32_t n, GroupA& lo, GroupA& hi) {
#pragma unroll
        for (int rg = 0; rg < 4; ++rg) {
            lo.a[rg] = __builtin_bit_cast(half8_t, *reinterpret_cast<const uint4*>(stage + rd * kStage + rg * 1024 + lane * 16));
            hi.a[rg] = __builtin_bit_cast(half8_t, *reinterpret_cast<const uint4*>(stage + rd * kStage + 4096 + rg * 1024 + lane * 16));
        }
        lds_barrier();
        deposit(wr, slo, shi);
        fetch(n + 3, slo, shi);
        rd = rd == 2 ? 0 : rd + 1;
        wr = wr == 2 ? 0 : wr + 1;
    };
    for (uint32_t b = 0; b < nblk; ++b) {
        const uint32_t bn = b + 1 < nblk ? b + 1 : b;   // the last block requests itself again
        const uint32_t tn = bn * TB;
        GroupA lo, hi;
#pragma unroll
        for (int cg = 0; cg < 4; ++cg) {
            const uint4 hdr = hd[cg];
            sc_a[cg] = hdr.y & 0x3F3F3F3Fu;
            sc_b[cg] = (hdr.w & 0x0F0F0F0Fu) | ((hdr.y >> 2) & 0x30303030u);
#pragma unroll
            for (int rg = 0; rg < 4; ++rg) D[cg][rg] = float4_t{0.f, 0.f, 0.f, 0.f};
        }
        step(4 * b, lo, hi);
        __builtin_amdgcn_sched_barrier(0);
        q4_chunk<0>(lo, hi, q, sc_a, D);
        __builtin_amdgcn_sched_barrier(0);
        step(4 * b + 1, lo, hi);
        __builtin_amdgcn_sched_barrier(0);
        q4_chunk<1>(lo, hi, q, sc_a, D);
        __builtin_amdgcn_sched_barrier(0);
        step(4 * b + 2, lo, hi);
        // the weights of the next block: after the A request that is awaited first
#pragma unroll
        for (int i = 0; i < 8; i += 2) q[i] = ld16(tile, lane * 16, tn + 1024 * i);
#pragma unroll
        for (int cg = 0; cg < 4; ++cg) hd[cg] = ld16(tile, j * 16, tn + 8192 + 256 * cg);
        __builtin_amdgcn_sched_barrier(0);
        q4_chunk<2>(lo, hi, q, sc_b, D);
        __builtin_amdgcn_sched_barrier(0);
        step(4 * b + 3, lo, hi);
        // what the block's end needs travels during the last chunk: the sums image (its 8 halves
        // are k-slice 0; the other k-slices are zero), the multipliers, and d, dmin and the minima,
        // which are read again rather than held through the block
        half8_t as[4];
        float2 ms[4], mult[4];
        uint4 hb[4];
#pragma unroll
        for (int rg = 0; rg < 4; ++rg) {
            as[rg] = __builtin_bit_cast(half8_t, ld16(c.blob, sums_off + rg * 256, sumi + b * L.mpad * 32));
            ms[rg] = ld8(c.blob, c.r_off + rg * 32, smul + b * L.mpad * 4);
            mult[rg] = ld8(c.blob, c.r_off + rg * 32, c.mult + b * 8 * c.mpad * 4);  // shared by the block's 8 groups
        }
        __builtin_amdgcn_sched_barrier(0);
        q4_chunk<3>(lo, hi, q, sc_b, D);
        __builtin_amdgcn_sched_barrier(0);
        // the odd quants are consumed: the header again and the next block's quants take their registers
#pragma unroll
        for (int cg = 0; cg < 4; ++cg) hb[cg] = ld16(tile, j * 16, b * TB + 8192 + 256 * cg);
#pragma unroll
        for (int i = 1; i < 8; i += 2) q[i] = ld16(tile, lane * 16, tn + 1024 * i);
        __builtin_amdgcn_sched_barrier(0);
        // block done: -dmin * sum_g m_g * (sum of group g) as one more MFMA per tile, then one scale step
#pragma unroll
        for (int cg = 0; cg < 4; ++cg) {
            const float d = h2f(hb[cg].x & 0xFFFFu), dmin = h2f(hb[cg].x >> 16);
            const uint32_t mn_a = hb[cg].z & 0x3F3F3F3Fu;
            const uint32_t mn_b = ((hb[cg].w >> 4) & 0x0F0F0F0Fu) | ((hb[cg].z >> 2) & 0x30303030u);
            const half8_t bm = as_half8(even_bytes(mn_a), odd_bytes(mn_a), even_bytes(mn_b), odd_bytes(mn_b));
#pragma unroll
            for (int rg = 0; rg < 4; ++rg) {
                const float4_t dm = __builtin_amdgcn_mfma_f32_16x16x32_f16(as[rg], bm, float4_t{0.f, 0.f, 0.f, 0.f}, 0, 0, 0);
                const float4_t dv = D[cg][rg];
                acc[cg][rg][0] = fmaf(d * mult[rg].x, dv[0] + dv[1], fmaf(-dmin * ms[rg].x, dm[0] + dm[1], acc[cg][rg][0]));
                acc[cg][rg][1] = fmaf(d * mult[rg].y, dv[2] + dv[3], fmaf(-dmin * ms[rg].y, dm[2] + dm[3], acc[cg][rg][1]));
            }
        }
        __builtin_amdgcn_sched_barrier(0);
    }
    if (!valid) return;
#pragma unroll
    for (int cg = 0; cg < 4; ++cg)
#pragma unroll
        for (int rg = 0; rg < 4; ++rg)
#pragma unroll
            for (int r = 0; r < 2; ++r) {
                const uint32_t row = c.row0 + 8 * rg + r;
                if (row < M) y[size_t(row) * N + tile_index * kCols + 16 * cg + j] = acc[cg][rg][r];
            }
}

// ---- Q6_K with the activations shared through LDS ------------------------------------------
__device__ __forceinline__ uint32_t ld4(__amdgpu_buffer_rsrc_t r, uint32_t lane_off, uint32_t uniform_off) {
    return __builtin_amdgcn_raw_buffer_load_b32(r, static_cast<int>(lane_off), static_cast<int>(uniform_off), 0);
}

typedef short short2_t __attribute__((ext_vector_type(2)));
// two int8 scales (one per 16-bit field, as unsigned bytes) -> two fp16 bit patterns |s| with the
// sign in bit 15: the half reads as s * 2^-24
__device__ __forceinline__ uint32_t scale_patterns(uint32_t fields) {
    const short2_t sv = __builtin_bit_cast(short2_t, fields ^ 0x00800080u) - short2_t{0x80, 0x80};
    const uint32_t mag = __builtin_bit_cast(uint32_t, __builtin_elementwise_abs(sv));
    return mag | (__builtin_bit_cast(uint32_t, sv) & 0x80008000u);
}

// group G (32 elements of K) of a Q6_K block for the wave's two column groups: q = lo + 16 hi2
// (4 + 2 bits); |scale| * lo <= 1905 and |scale| * 4 hi2 <= 1524 are exact as fp16 bit patterns
// (n < 2048 reads as n * 2^-24) and carry the scale's sign in bit 15, so both parts accumulate over
// the whole block inside the MFMA chains Dl and Dh (Dh then weighs 4).  The matrix instruction does not
// normalise such patterns -- leading zeros cost product bits once a sum's products are aligned -- which is
// why hi2 enters times 4.  A scale covers 16 elements: lanes of k-slices
// 0-1 take the group's first scale, 2-3 the second (sel picks that field of the pattern word).
template <int G>
__device__ __forceinline__ void q6_group(const GroupA& A, const uint4 (&ql)[4], const uint4 (&qh)[2], const uint32_t (&P)[2][8],
                                         uint32_t sel, float4_t (&Dl)[2][4], float4_t (&Dh)[2][4]) {
    constexpr int n = G >> 2, qd = G & 3, ls = qd >= 2 ? 4 : 0;
#pragma unroll
    for (int cc = 0; cc < 2; ++cc) {
        const uint32_t ps = __builtin_amdgcn_perm(0u, P[cc][G], sel);
        const uint32_t pair = ps & 0x7FFF7FFFu, sign = ps & 0x80008000u;
        const uint4 lq = ql[2 * cc + n], hq = qh[cc];
        const uint32_t w0 = (qd & 1) ? lq.z : lq.x, w1 = (qd & 1) ? lq.w : lq.y;
        const uint32_t h0 = n ? hq.z : hq.x, h1 = n ? hq.w : hq.y;
        uint32_t bl[4], bh[4];
#pragma unroll
        for (int k = 0; k < 2; ++k) {
            const uint32_t w = k ? w1 : w0, h = k ? h1 : h0;
            // the products stay below 2^11, so adding the sign bit sets it
            bl[2 * k] = pk_mad((w >> ls) & 0x000F000Fu, pair, sign);
            bl[2 * k + 1] = pk_mad((w >> (ls + 8)) & 0x000F000Fu, pair, sign);
            // the two high bits enter as 4 hi2 (|scale| 4 hi2 <= 1524): fewer leading zeros in the pattern
            bh[2 * k] = pk_mad((qd == 0 ? h << 2 : h >> (2 * qd - 2)) & 0x000C000Cu, pair, sign);
            bh[2 * k + 1] = pk_mad((h >> (6 + 2 * qd)) & 0x000C000Cu, pair, sign);
        }
        const half8_t blo = as_half8(bl[0], bl[1], bl[2], bl[3]), bhi = as_half8(bh[0], bh[1], bh[2], bh[3]);
#pragma unroll
        for (int rg = 0; rg < 4; ++rg) Dl[cc][rg] = __builtin_amdgcn_mfma_f32_16x16x32_f16(A.a[rg], blo, Dl[cc][rg], 0, 0, 0);
#pragma unroll
        for (int rg = 0; rg < 4; ++rg) Dh[cc][rg] = __builtin_amdgcn_mfma_f32_16x16x32_f16(A.a[rg], bhi, Dh[cc][rg], 0, 0, 0);
    }
}

// The four waves of a workgroup own the two halves (two column groups each) of two neighbouring
// column tiles and the SAME 32 rows, and share the A operands through LDS exactly as the Q4_K
// kernel does (three rotating buffers of one 64-element chunk, one barrier per chunk).  The offset
// term -32 d sum_t scale_t (sum of half-group t) is one more MFMA per block on the image of the 16
// half-group sums.  grid (Mpad/32, ceil(N/128)), 256 threads.
__global__ void __launch_bounds__(256, 2)
prefill_gemm_q6k_kernel(const uint8_t* __restrict__ tiles, const uint8_t* __restrict__ blob, float* __restrict__ y,
                        uint32_t M, uint32_t K, uint32_t N) {
    constexpr uint32_t TB = kCols * block_bytes(GUFFIN_Q6_K);
    constexpr uint32_t kStage = 8192;  // one chunk of A operands
    __shared__ __attribute__((aligned(16))) uint8_t stage[3 * kStage];
    const ImageLayout L = image_layout(M, K);
    const uint32_t lane = threadIdx.x & 63, wv = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t j = lane & 15, lg = lane >> 4;
    const uint32_t nblk = K / 256, nchunk = nblk * 4;
    const uint32_t wave_row = blockIdx.x * kWaveRows;
    if (wave_row >= M) return;  // padding rows only (the whole workgroup)
    const uint32_t tile_index = blockIdx.y * 2 + (wv >> 1), half = wv & 1u;
    const bool valid = tile_index < N / kCols;  // a wave past the last tile works on tile 0 and stores nothing
    const uint32_t mpad = L.mpad, rg0 = wave_row / 8, row0 = wave_row + 2 * lg;
    const uint32_t a_off = j * 64 + lg * 16;  // A lane (i = lane % 16, s = lane / 16): row i, k-slice s
    const uint32_t r_off = 8 * lg;            // the lane's first row inside a row group, in bytes of a float row
    const __amdgpu_buffer_rsrc_t img = make_resource(blob, static_cast<uint32_t>(L.bytes));
    const uint32_t mult_off = static_cast<uint32_t>(L.mult_off) + wave_row * 4;
    const uint32_t shml = static_cast<uint32_t>(L.shml_off) + wave_row * 4;
    const uint32_t sumh = static_cast<uint32_t>(L.sumh_off) + rg0 * 512;
    // the sums image fills k-slices 0 and 1 only: the other lanes read past the resource's end,
    // which a buffer load answers with zeros
    const uint32_t sums_off = lane < 32 ? j * 32 + lg * 16 : 0x80000000u;
    const __amdgpu_buffer_rsrc_t tile = make_resource(tiles + size_t(valid ? tile_index : 0) * nblk * TB, nblk * TB);
    const uint32_t sel = lane >= 32 ? 0x03020302u : 0x01000100u;
    // this wave's share of chunk n: row group wv of its two groups
    const uint32_t share = (rg0 + wv) * 1024;
    uint4 slo, shi;
    auto fetch = [&](uint32_t n) {
        const uint32_t g = 2 * (n < nchunk ? n : nchunk - 1);  // past the end: the last chunk again, never read
        slo = ld16(img, a_off, share + g * mpad * 128);
        shi = ld16(img, a_off, share + (g + 1) * mpad * 128);
    };
    auto deposit = [&](uint32_t buffer) {
        *reinterpret_cast<uint4*>(stage + buffer * kStage + wv * 1024 + lane * 16) = slo;
        *reinterpret_cast<uint4*>(stage + buffer * kStage + 4096 + wv * 1024 + lane * 16) = shi;
    };
    float acc[2][4][2];  // [column group of the half][row group][row of the lane]
#pragma unroll
    for (int cc = 0; cc < 2; ++cc)
#pragma unroll
        for (int rg = 0; rg < 4; ++rg) { acc[cc][rg][0] = 0.f; acc[cc][rg][1] = 0.f; }
    // the block's bytes of this wave's half tile: low nibbles (pieces 4 half .. 4 half + 3), high
    // bit pairs (8 + 2 half, + 1), the 16 scales of the lane's column and the dword that holds its d
    uint4 ql[4], qh[2], scv[2], qh_next[2], scv_next[2];
    uint32_t dw[2], dw_next[2];
#pragma unroll
    for (int i = 0; i < 4; ++i) ql[i] = ld16(tile, lane * 16, 1024 * (4 * half + i));
#pragma unroll
    for (int cc = 0; cc < 2; ++cc) {
        qh[cc] = ld16(tile, lane * 16, 8192 + 1024 * (2 * half + cc));
        scv[cc] = ld16(tile, j * 16, 12288 + 256 * (2 * half + cc));
        dw[cc] = ld4(tile, (j >> 1) * 4, 13312 + 32 * (2 * half + cc));
    }
    fetch(0); deposit(0);
    fetch(1); deposit(1);
    fetch(2);
    lds_barrier();  // chunks 0 and 1 are complete
    uint32_t rd = 0, wr = 2;  // buffers of the chunk to read and of the chunk to deposit
    // one step: read chunk n's operands, barrier, deposit chunk n + 2, ask for chunk n + 3
    auto step = [&](uint32_t n, GroupA& lo, GroupA& hi) {
#pragma unroll
        for (int rg = 0; rg < 4; ++rg) {
            lo.a[rg] = __builtin_bit_cast(half8_t, *reinterpret_cast<const uint4*>(stage + rd * kStage + rg * 1024 + lane * 16));
            hi.a[rg] = __builtin_bit_cast(half8_t, *reinterpret_cast<const uint4*>(stage + rd * kStage + 4096 + rg * 1024 + lane * 16));
        }
        lds_barrier();
        deposit(wr);
        fetch(n + 3);
        rd = rd == 2 ? 0 : rd + 1;
        wr = wr == 2 ? 0 : wr + 1;
    };
    // one matrix instruction keeps its pipe for four issue slots: the next operands are built in the other three
    auto interleave = [] {
#pragma unroll
        for (int i = 0; i < 32; ++i) {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            __builtin_amdgcn_sched_group_barrier(0x002, 3, 0);
        }
    };
    float4_t Dl[2][4], Dh[2][4];
    uint32_t P[2][8];  // word m: the patterns of scales 2m and 2m + 1 of the lane's column
    for (uint32_t b = 0; b < nblk; ++b) {
        const uint32_t tn = (b + 1 < nblk ? b + 1 : b) * TB;   // the last block requests itself again
        GroupA lo, hi;
#pragma unroll
        for (int cc = 0; cc < 2; ++cc) {
            const uint32_t w[4] = {scv[cc].x, scv[cc].y, scv[cc].z, scv[cc].w};
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                P[cc][2 * i] = scale_patterns(__builtin_amdgcn_perm(0u, w[i], 0x0c010c00u));
                P[cc][2 * i + 1] = scale_patterns(__builtin_amdgcn_perm(0u, w[i], 0x0c030c02u));
            }
#pragma unroll
            for (int rg = 0; rg < 4; ++rg) { Dl[cc][rg] = float4_t{0.f, 0.f, 0.f, 0.f}; Dh[cc][rg] = Dl[cc][rg]; }
        }
        step(4 * b, lo, hi);
        __builtin_amdgcn_sched_barrier(0);
        q6_group<0>(lo, ql, qh, P, sel, Dl, Dh);
        q6_group<1>(hi, ql, qh, P, sel, Dl, Dh);
        interleave();
        __builtin_amdgcn_sched_barrier(0);
        step(4 * b + 1, lo, hi);
        __builtin_amdgcn_sched_barrier(0);
        q6_group<2>(lo, ql, qh, P, sel, Dl, Dh);
        q6_group<3>(hi, ql, qh, P, sel, Dl, Dh);
        interleave();
        __builtin_amdgcn_sched_barrier(0);
        step(4 * b + 2, lo, hi);
        // the first 128 elements' nibbles are consumed: the next block's take their registers, and
        // its bit pairs, scales and d are requested beside them
        ql[0] = ld16(tile, lane * 16, tn + 1024 * (4 * half));
        ql[2] = ld16(tile, lane * 16, tn + 1024 * (4 * half + 2));
#pragma unroll
        for (int cc = 0; cc < 2; ++cc) {
            qh_next[cc] = ld16(tile, lane * 16, tn + 8192 + 1024 * (2 * half + cc));
            scv_next[cc] = ld16(tile, j * 16, tn + 12288 + 256 * (2 * half + cc));
            dw_next[cc] = ld4(tile, (j >> 1) * 4, tn + 13312 + 32 * (2 * half + cc));
        }
        __builtin_amdgcn_sched_barrier(0);
        q6_group<4>(lo, ql, qh, P, sel, Dl, Dh);
        q6_group<5>(hi, ql, qh, P, sel, Dl, Dh);
        interleave();
        __builtin_amdgcn_sched_barrier(0);
        step(4 * b + 3, lo, hi);
        // what the block's end needs travels during the last chunk: the sums image and the multipliers
        half8_t as[4];
        float2 ms[4], mult[4];
#pragma unroll
        for (int rg = 0; rg < 4; ++rg) {
            as[rg] = __builtin_bit_cast(half8_t, ld16(img, sums_off + rg * 512, sumh + b * mpad * 64));
            ms[rg] = ld8(img, r_off + rg * 32, shml + b * mpad * 4);
            mult[rg] = ld8(img, r_off + rg * 32, mult_off + b * 8 * mpad * 4);  // shared by the block's 8 groups
        }
        __builtin_amdgcn_sched_barrier(0);
        q6_group<6>(lo, ql, qh, P, sel, Dl, Dh);
        q6_group<7>(hi, ql, qh, P, sel, Dl, Dh);
        interleave();
        __builtin_amdgcn_sched_barrier(0);
        ql[1] = ld16(tile, lane * 16, tn + 1024 * (4 * half + 1));
        ql[3] = ld16(tile, lane * 16, tn + 1024 * (4 * half + 3));
        __builtin_amdgcn_sched_barrier(0);
        // block done: the offset term as one more MFMA per column group, then one scale step
#pragma unroll
        for (int cc = 0; cc < 2; ++cc) {
            const float d = h2f((dw[cc] >> (16 * (j & 1u))) & 0xFFFFu);
            const bool upper = (lg & 1u) != 0;  // k-slice 1 holds half-groups 8..15
            uint32_t bw[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const uint32_t first = P[cc][i], second = P[cc][4 + i];  // values, so that P stays in registers
                bw[i] = upper ? second : first;
            }
            const half8_t bm = as_half8(bw[0], bw[1], bw[2], bw[3]);
#pragma unroll
            for (int rg = 0; rg < 4; ++rg) {
                const float4_t dm = __builtin_amdgcn_mfma_f32_16x16x32_f16(as[rg], bm, float4_t{0.f, 0.f, 0.f, 0.f}, 0, 0, 0);
                const float4_t lo4 = Dl[cc][rg], hi4 = Dh[cc][rg];
                acc[cc][rg][0] = fmaf(d * mult[rg].x, (lo4[0] + lo4[1]) + 4.0f * (hi4[0] + hi4[1]),
                                      fmaf(-32.0f * d * ms[rg].x, dm[0] + dm[1], acc[cc][rg][0]));
                acc[cc][rg][1] = fmaf(d * mult[rg].y, (lo4[2] + lo4[3]) + 4.0f * (hi4[2] + hi4[3]),
                                      fmaf(-32.0f * d * ms[rg].y, dm[2] + dm[3], acc[cc][rg][1]));
            }
            qh[cc] = qh_next[cc]; scv[cc] = scv_next[cc]; dw[cc] = dw_next[cc];
        }
        __builtin_amdgcn_sched_barrier(0);
    }
    if (!valid) return;
#pragma unroll
    for (int cc = 0; cc < 2; ++cc)
#pragma unroll
        for (int rg = 0; rg < 4; ++rg)
#pragma unroll
            for (int r = 0; r < 2; ++r) {
                const uint32_t row = row0 + 8 * rg + r;
                if (row < M) y[size_t(row) * N + tile_index * kCols + 16 * (2 * half + cc) + j] = acc[cc][rg][r];
            }
}

// Q8_0.  grid (N/64, Mpad/128), 256 threads, four waves on the same tile (128 rows), each loading its
// own operands.  y[M][N] fp32.
template <int DTYPE>
__global__ void __launch_bounds__(256, 2)
prefill_gemm_kernel(const uint8_t* __restrict__ tiles, const uint8_t* __restrict__ blob, float* __restrict__ y,
                    uint32_t M, uint32_t K, uint32_t N) {
    constexpr uint32_t TB = kCols * block_bytes(DTYPE);
    const ImageLayout L = image_layout(M, K);
    const uint32_t lane = threadIdx.x & 63, wv = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t j = lane & 15, lg = lane >> 4;
    const uint32_t nblk = K / block_elems(DTYPE);
    WaveCtx c;
    c.mpad = L.mpad;
    c.rg0 = (blockIdx.y * kChunkRows + wv * kWaveRows) / 8;
    c.row0 = blockIdx.y * kChunkRows + wv * kWaveRows + 2 * lg;
    c.image = blob + (lane & 15u) * 64 + (lane >> 4) * 16;  // A lane (i = lane % 16, s = lane / 16): row i, k-slice s
    c.mult = reinterpret_cast<const float*>(blob + L.mult_off);
    c.s32 = reinterpret_cast<const float*>(blob + L.s32_off);
    if (blockIdx.y * kChunkRows + wv * kWaveRows >= M) return;  // a wave of padding rows only
    float acc[4][4][2];  // [column group][row group][row of the lane]
#pragma unroll
    for (int cg = 0; cg < 4; ++cg)
#pragma unroll
        for (int rg = 0; rg < 4; ++rg) { acc[cg][rg][0] = 0.f; acc[cg][rg][1] = 0.f; }
    const uint8_t* tp = tiles + size_t(blockIdx.x) * nblk * TB;
    for (uint32_t b = 0; b < nblk; ++b, tp += TB) {
        static_assert(DTYPE == GUFFIN_Q8_0, "Q4_K and Q6_K have their own kernels");
        const uint4 q0 = *reinterpret_cast<const uint4*>(tp + lane * 16);
        const uint4 q1 = *reinterpret_cast<const uint4*>(tp + 1024 + lane * 16);
        GroupOperands o;
        load_group(c, b, o);
#pragma unroll
        for (int cg = 0; cg < 4; ++cg) {
            const float d = h2f(*reinterpret_cast<const uint16_t*>(tp + 2048 + (16 * cg + j) * 2));
            const uint4 piece = cg < 2 ? q0 : q1;
            const uint32_t w0 = ((cg & 1) ? piece.z : piece.x) ^ 0x80808080u, w1 = ((cg & 1) ? piece.w : piece.y) ^ 0x80808080u;
            // 8 (q + 128) as a bit pattern: the top of the 11-bit window that reads as n 2^-24
            mfma_scale(o, as_half8(even_bytes(w0) << 3, odd_bytes(w0) << 3, even_bytes(w1) << 3, odd_bytes(w1) << 3), 0.125f * d, acc[cg]);
            add_offset(c.s32, c, b, -128.0f * d, acc[cg]);
        }
    }
#pragma unroll
    for (int cg = 0; cg < 4; ++cg)
#pragma unroll
        for (int rg = 0; rg < 4; ++rg)
#pragma unroll
            for (int r = 0; r < 2; ++r) {
                const uint32_t row = c.row0 + 8 * rg + r;
                if (row < M) y[size_t(row) * N + blockIdx.x * kCols + 16 * cg + j] = acc[cg][rg][r];
            }
}

// ---- causal attention for a run of rows ------------------------------------------------
// grid (ceil(rows / 16), kv_heads), 256 threads: thread = (query slot of 16 rows x GROUP heads, one of
// 256/(16*GROUP) interleaved dim slices).  Keys/values of positions below `position` come from the
// ring, those of the run itself from its private fp16 rows [rows][kv_heads*256].
template <int GROUP>
__global__ void __launch_bounds__(256)
prefill_attention_kernel(const float* __restrict__ q, const uint16_t* __restrict__ ring_k,
                         const uint16_t* __restrict__ ring_v, const uint16_t* __restrict__ run_k,
                         const uint16_t* __restrict__ run_v, float* __restrict__ out, uint32_t rows,
                         uint32_t position, uint32_t window, uint32_t ring_mask, uint32_t q_heads,
                         uint32_t kv_heads, float scale) {
    constexpr int HD = 256, QT = 16, NQ = QT * GROUP, KT = 32;
    constexpr int TPQ = 256 / NQ;        // threads per query: 16, 8 or 4
    constexpr int DPT = HD / TPQ;        // dims per thread, interleaved: dim = part + TPQ * i
    __shared__ _Float16 ks[KT][HD + 2];
    __shared__ _Float16 vs[KT][HD + 2];
    __shared__ float sc[NQ][KT];
    const uint32_t kvh = blockIdx.y, r0 = blockIdx.x * QT;
    const uint32_t qi = threadIdx.x / TPQ, part = threadIdx.x % TPQ;
    const uint32_t row = r0 + qi / GROUP, head = kvh * GROUP + qi % GROUP;
    const bool live = row < rows;
    const uint32_t pos = position + row;
    float qv[DPT], acc[DPT];
#pragma unroll
    for (int i = 0; i < DPT; ++i) {
        qv[i] = live ? q[(size_t(row) * q_heads + head) * HD + part + TPQ * i] * scale : 0.f;
        acc[i] = 0.f;
    }
    float mx = -INFINITY, den = 0.f;
    const uint32_t last_row = min(r0 + QT, rows) - 1;
    const uint32_t hi_pos = position + last_row;
    const uint32_t lo_first = (window && position + r0 + 1 > window) ? position + r0 + 1 - window : 0;
    const uint32_t my_first = (window && pos + 1 > window) ? pos + 1 - window : 0;
    const size_t row_stride = size_t(kv_heads) * HD;
    for (uint32_t t0 = lo_first; t0 <= hi_pos; t0 += KT) {
        __syncthreads();
        for (uint32_t i = threadIdx.x; i < KT * HD / 2; i += 256) {
            const uint32_t t = i / (HD / 2), d2 = i % (HD / 2);
            uint32_t kk = 0, vv = 0;
            const uint32_t kp = t0 + t;
            if (kp <= hi_pos) {
                const bool own = kp >= position;
                const size_t off = (own ? size_t(kp - position) : size_t(kp & ring_mask)) * row_stride + kvh * HD + 2 * d2;
                kk = *reinterpret_cast<const uint32_t*>((own ? run_k : ring_k) + off);
                vv = *reinterpret_cast<const uint32_t*>((own ? run_v : ring_v) + off);
            }
            *reinterpret_cast<uint32_t*>(&ks[t][2 * d2]) = kk;
            *reinterpret_cast<uint32_t*>(&vs[t][2 * d2]) = vv;
        }
        __syncthreads();
        float tile_max = -INFINITY;
        float s_loc[KT / TPQ];
        for (int t = 0; t < KT; ++t) {
            float s = 0.f;
#pragma unroll
            for (int i = 0; i < DPT; ++i) s = fmaf(qv[i], static_cast<float>(ks[t][part + TPQ * i]), s);
#pragma unroll
            for (int o = TPQ / 2; o > 0; o >>= 1) s += __shfl_xor(s, o, kWave);
            const uint32_t kp = t0 + t;
            const bool visible = live && kp <= pos && kp >= my_first;
            s = visible ? s : -INFINITY;
            if (uint32_t(t) % TPQ == part) s_loc[t / TPQ] = s;
            tile_max = fmaxf(tile_max, s);
        }
        const float new_max = fmaxf(mx, tile_max);
        const float rescale = new_max == -INFINITY ? 1.f : expf(mx - new_max);
        den *= rescale;
#pragma unroll
        for (int i = 0; i < DPT; ++i) acc[i] *= rescale;
        float add = 0.f;
#pragma unroll
        for (int u = 0; u < KT / TPQ; ++u) {
            const float p = s_loc[u] == -INFINITY ? 0.f : expf(s_loc[u] - new_max);
            sc[qi][u * TPQ + part] = p;
            add += p;
        }
#pragma unroll
        for (int o = TPQ / 2; o > 0; o >>= 1) add += __shfl_xor(add, o, kWave);
        den += add;
        mx = new_max;
        // the TPQ lanes of a query sit in one wave: their sc[] entries are visible after a wave barrier
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        for (int t = 0; t < KT; ++t) {
            const float p = sc[qi][t];
#pragma unroll
            for (int i = 0; i < DPT; ++i) acc[i] = fmaf(p, static_cast<float>(vs[t][part + TPQ * i]), acc[i]);
        }
    }
    if (live) {
#pragma unroll
        for (int i = 0; i < DPT; ++i) out[(size_t(row) * q_heads + head) * HD + part + TPQ * i] = acc[i] / den;
    }
}

// ---- the same attention on the matrix core ------------------------------------------------
// Values are contracted over tokens, so the B operand needs 8 consecutive tokens of one output
// dimension: a small pass first writes V^T, [kv_heads][256][T] fp16, for the virtual tokens
// base32 .. base32 + T (T a multiple of 32; tokens outside [first_visible, end) are zero).
__global__ void __launch_bounds__(256)
transpose_values_kernel(const uint16_t* __restrict__ ring_v, const uint16_t* __restrict__ run_v,
                        uint16_t* __restrict__ vt, uint32_t base32, uint32_t T, uint32_t first_visible,
                        uint32_t position, uint32_t end_pos, uint32_t ring_mask, uint32_t kv_heads) {
    constexpr int HD = 256, PITCH = HD + 8;
    __shared__ __attribute__((aligned(16))) uint16_t tile[32][PITCH];
    const uint32_t kvh = blockIdx.y, v0 = blockIdx.x * 32;
    const size_t row_stride = size_t(kv_heads) * HD;
    for (uint32_t c = threadIdx.x; c < 32 * (HD / 8); c += 256) {
        const uint32_t token = c / (HD / 8), d8 = c % (HD / 8);
        const uint32_t kp = base32 + v0 + token;
        uint4 val = make_uint4(0, 0, 0, 0);
        if (kp >= first_visible && kp < end_pos) {
            const uint16_t* src = kp >= position ? run_v + size_t(kp - position) * row_stride
                                                 : ring_v + size_t(kp & ring_mask) * row_stride;
            val = *reinterpret_cast<const uint4*>(src + kvh * HD + 8 * d8);
        }
        *reinterpret_cast<uint4*>(&tile[token][8 * d8]) = val;
    }
    __syncthreads();
    const uint32_t dim = threadIdx.x;
    uint32_t w[16];
#pragma unroll
    for (int t = 0; t < 16; ++t) w[t] = uint32_t(tile[2 * t][dim]) | (uint32_t(tile[2 * t + 1][dim]) << 16);
    uint4* dst = reinterpret_cast<uint4*>(vt + (size_t(kvh) * HD + dim) * T + v0);
#pragma unroll
    for (int i = 0; i < 4; ++i) dst[i] = make_uint4(w[4 * i], w[4 * i + 1], w[4 * i + 2], w[4 * i + 3]);
}

__device__ __forceinline__ void split_half8(const float (&x)[8], uint4& hi, uint4& lo) {
    uint32_t h[4], l[4];
#pragma unroll
    for (int p = 0; p < 4; ++p) {
        uint32_t hw = 0, lw = 0;
#pragma unroll
        for (int q = 0; q < 2; ++q) {
            const _Float16 a = static_cast<_Float16>(x[2 * p + q]);
            const _Float16 b = static_cast<_Float16>(x[2 * p + q] - static_cast<float>(a));
            hw |= uint32_t(__builtin_bit_cast(uint16_t, a)) << (16 * q);
            lw |= uint32_t(__builtin_bit_cast(uint16_t, b)) << (16 * q);
        }
        h[p] = hw; l[p] = lw;
    }
    hi = make_uint4(h[0], h[1], h[2], h[3]);
    lo = make_uint4(l[0], l[1], l[2], l[3]);
}

// grid (ceil(rows / 16), kv_heads), 4 waves.  A workgroup serves 16 query rows x GROUP heads of one
// KV head.  Each wave walks its own 32-token tiles (tile index = wave mod 4) with its own online
// softmax state and its own output accumulators; the four states are merged at the end.
//   scores   S = Q K^T: queries (scaled, fp16 hi + lo, staged once in LDS in operand order) as A,
//            keys straight from their fp16 rows as B (a lane reads 8 dims of one key per MFMA)
//   values   O += P V: probabilities times 2^10 as fp16 hi + lo through a wave-private LDS
//            transpose as A, V^T rows as B
template <int GROUP>
__global__ void __launch_bounds__(256)
prefill_attention_mfma_kernel(const float* __restrict__ q, const uint16_t* __restrict__ ring_k,
                              const uint16_t* __restrict__ run_k, const uint16_t* __restrict__ vt,
                              float* __restrict__ out, uint32_t rows, uint32_t position, uint32_t window,
                              uint32_t ring_mask, uint32_t q_heads, uint32_t kv_heads, float scale,
                              uint32_t base32, uint32_t T) {
    constexpr int HD = 256, QT = 16;
    constexpr float kProbScale = 1024.0f;
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    // [GROUP][8 k-steps][hi, lo][64 lanes] 16-byte query operands, later the merge buffer
    uint8_t* qa = lds;
    const uint32_t lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t j = lane & 15, lg = lane >> 4;
    float* pt = reinterpret_cast<float*>(lds + GROUP * 16384) + wave * (GROUP * QT * 32);  // [GROUP][16 rows][32 tokens]
    float* ml = reinterpret_cast<float*>(lds + GROUP * 16384 + 4 * GROUP * QT * 32 * 4);     // [GROUP][16][2] for the merge
    const uint32_t kvh = blockIdx.y, r0 = blockIdx.x * QT;
    const size_t row_stride = size_t(kv_heads) * HD;

    for (uint32_t idx = threadIdx.x; idx < GROUP * QT * 32; idx += 256) {
        const uint32_t g = idx / (QT * 32), i = (idx / 32) % QT, c8 = idx % 32;
        const uint32_t row = min(r0 + i, rows - 1);
        const float* src = q + (size_t(row) * q_heads + kvh * GROUP + g) * HD + 8 * c8;
        const float4 a = *reinterpret_cast<const float4*>(src), b = *reinterpret_cast<const float4*>(src + 4);
        const float x[8] = {a.x * scale, a.y * scale, a.z * scale, a.w * scale, b.x * scale, b.y * scale, b.z * scale, b.w * scale};
        uint4 hi, lo;
        split_half8(x, hi, lo);
        uint8_t* dst = qa + ((g * 8 + c8 / 4) * 2) * 1024 + (i + 16 * (c8 % 4)) * 16;
        *reinterpret_cast<uint4*>(dst) = hi;
        *reinterpret_cast<uint4*>(dst + 1024) = lo;
    }
    __syncthreads();

    float m[GROUP][4], l[GROUP][4];
    float4_t O[GROUP][16];
#pragma unroll
    for (int g = 0; g < GROUP; ++g) {
#pragma unroll
        for (int r = 0; r < 4; ++r) { m[g][r] = -INFINITY; l[g][r] = 0.f; }
#pragma unroll
        for (int dt = 0; dt < 16; ++dt) O[g][dt] = float4_t{0.f, 0.f, 0.f, 0.f};
    }
    const uint32_t last_row = min(r0 + QT, rows) - 1;
    const uint32_t hi_pos = position + last_row;
    const uint32_t lo_first = (window && position + r0 + 1 > window) ? position + r0 + 1 - window : 0;
    uint32_t pos_r[4], first_r[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        const uint32_t row = r0 + 4 * lg + r;
        pos_r[r] = row < rows ? position + row : 0u;  // a padding row sees nothing: first > pos
        first_r[r] = row < rows ? ((window && position + row + 1 > window) ? position + row + 1 - window : 0u) : 1u;
    }
    const uint32_t tile_lo = (lo_first - base32) / 32, tile_hi = (hi_pos - base32) / 32;
    for (uint32_t ti = tile_lo + wave; ti <= tile_hi; ti += 4) {
        const uint32_t t0 = base32 + 32 * ti;
        float4_t S[GROUP][2];
#pragma unroll
        for (int c = 0; c < 2; ++c) {
            const uint32_t kp = min(t0 + 16 * c + j, hi_pos);
            const uint16_t* krow = (kp >= position ? run_k + size_t(kp - position) * row_stride
                                                   : ring_k + size_t(kp & ring_mask) * row_stride) + kvh * HD + 8 * lg;
            uint4 kb[8];
#pragma unroll
            for (int ks = 0; ks < 8; ++ks) kb[ks] = *reinterpret_cast<const uint4*>(krow + 32 * ks);
#pragma unroll
            for (int g = 0; g < GROUP; ++g) {
                float4_t acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int ks = 0; ks < 8; ++ks) {
                    const uint8_t* ap = qa + ((g * 8 + ks) * 2) * 1024 + lane * 16;
                    const half8_t kv = __builtin_bit_cast(half8_t, kb[ks]);
                    acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8_t, *reinterpret_cast<const uint4*>(ap)), kv, acc, 0, 0, 0);
                    acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8_t, *reinterpret_cast<const uint4*>(ap + 1024)), kv, acc, 0, 0, 0);
                }
                S[g][c] = acc;
            }
        }
        // online softmax of the lane group's four rows; a row's 32 scores sit in 16 lanes x 2 tiles
#pragma unroll
        for (int g = 0; g < GROUP; ++g) {
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                float sv[2];
#pragma unroll
                for (int c = 0; c < 2; ++c) {
                    const uint32_t kp = t0 + 16 * c + j;
                    const bool visible = kp <= pos_r[r] && kp >= first_r[r] && kp <= hi_pos;
                    sv[c] = visible ? S[g][c][r] : -INFINITY;
                }
                const float tmax = row16_max(fmaxf(sv[0], sv[1]));
                const float new_m = fmaxf(m[g][r], tmax);
                const float resc = new_m == -INFINITY ? 1.f : expf(m[g][r] - new_m);
                const float p0 = sv[0] == -INFINITY ? 0.f : expf(sv[0] - new_m);
                const float p1 = sv[1] == -INFINITY ? 0.f : expf(sv[1] - new_m);
                const float add = row16_sum(p0 + p1);
                l[g][r] = l[g][r] * resc + add;
                m[g][r] = new_m;
#pragma unroll
                for (int dt = 0; dt < 16; ++dt) O[g][dt][r] *= resc;
                pt[(g * QT + 4 * lg + r) * 32 + j] = p0 * kProbScale;
                pt[(g * QT + 4 * lg + r) * 32 + 16 + j] = p1 * kProbScale;
            }
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        half8_t pa_hi[GROUP], pa_lo[GROUP];
#pragma unroll
        for (int g = 0; g < GROUP; ++g) {
            const float* src = pt + (g * QT + j) * 32 + 8 * lg;  // A lane (row j, tokens 8 lg .. 8 lg + 7)
            const float4 a = *reinterpret_cast<const float4*>(src), b = *reinterpret_cast<const float4*>(src + 4);
            const float x[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
            uint4 hi, lo;
            split_half8(x, hi, lo);
            pa_hi[g] = __builtin_bit_cast(half8_t, hi);
            pa_lo[g] = __builtin_bit_cast(half8_t, lo);
        }
        const uint16_t* vcol = vt + (size_t(kvh) * HD + j) * T + (t0 - base32) + 8 * lg;
#pragma unroll
        for (int dt = 0; dt < 16; ++dt) {
            const half8_t vb = __builtin_bit_cast(half8_t, *reinterpret_cast<const uint4*>(vcol + size_t(16 * dt) * T));
#pragma unroll
            for (int g = 0; g < GROUP; ++g) {
                O[g][dt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(pa_hi[g], vb, O[g][dt], 0, 0, 0);
                O[g][dt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(pa_lo[g], vb, O[g][dt], 0, 0, 0);
            }
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    }
    // merge the four waves' states in wave order through LDS (the query operands are dead now)
    float* ob = reinterpret_cast<float*>(qa);  // [(g * 16 + dt) * 4 + r][lane]
    for (uint32_t w = 0; w < 4; ++w) {
        __syncthreads();
        if (wave != w) continue;
#pragma unroll
        for (int g = 0; g < GROUP; ++g)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                float mine = 1.f, theirs = 0.f;
                if (w > 0) {
                    const float mo = ml[(g * QT + 4 * lg + r) * 2], lo_ = ml[(g * QT + 4 * lg + r) * 2 + 1];
                    const float M = fmaxf(m[g][r], mo);
                    mine = m[g][r] == -INFINITY ? 0.f : expf(m[g][r] - M);
                    theirs = mo == -INFINITY ? 0.f : expf(mo - M);
                    l[g][r] = l[g][r] * mine + lo_ * theirs;
                    m[g][r] = M;
                }
#pragma unroll
                for (int dt = 0; dt < 16; ++dt) {
                    float* slot = ob + (((g * 16 + dt) * 4 + r) * 64 + lane);
                    const float v = O[g][dt][r] * mine + (w > 0 ? *slot * theirs : 0.f);
                    *slot = v;
                }
            }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        if (j == 0) {
#pragma unroll
            for (int g = 0; g < GROUP; ++g)
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    ml[(g * QT + 4 * lg + r) * 2] = m[g][r];
                    ml[(g * QT + 4 * lg + r) * 2 + 1] = l[g][r];
                }
        }
    }
    __syncthreads();
    for (uint32_t idx = threadIdx.x; idx < GROUP * QT * HD; idx += 256) {
        const uint32_t g = idx / (QT * HD), i = (idx / HD) % QT, d = idx % HD;
        const uint32_t row = r0 + i;
        if (row >= rows) continue;
        const float v = ob[((g * 16 + d / 16) * 4 + (i & 3)) * 64 + (d & 15) + 16 * (i >> 2)];
        out[(size_t(row) * q_heads + kvh * GROUP + g) * HD + d] = v / (ml[(g * QT + i) * 2 + 1] * kProbScale);
    }
}

// ring[(position + row) & mask] = run[row] for the rows that survive in a ring of this capacity.
// Rows move as 16-byte pieces asked for at 4-byte alignment: a ring may be a view that starts at any word of its
// allocation (the reference's caches are, tests/tensor/gemma3_metal_tests.cpp:765-774).
__global__ void publish_run_kernel(const U4a4* __restrict__ run_k, const U4a4* __restrict__ run_v,
                                   U4a4* __restrict__ ring_k, U4a4* __restrict__ ring_v, uint32_t rows,
                                   uint32_t first_row, uint32_t position, uint32_t ring_mask, uint32_t row_vec) {
    const uint64_t i = uint64_t(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i >= uint64_t(rows - first_row) * row_vec) return;
    const uint32_t row = first_row + static_cast<uint32_t>(i / row_vec), c = static_cast<uint32_t>(i % row_vec);
    const size_t dst = size_t((position + row) & ring_mask) * row_vec + c;
    ring_k[dst] = run_k[size_t(row) * row_vec + c];
    ring_v[dst] = run_v[size_t(row) * row_vec + c];
}

// dst[(position + t) & dst_mask] = src[(position + t) & src_mask], keys and values
__global__ void kv_cache_copy_kernel(const U4a4* __restrict__ src_k, const U4a4* __restrict__ src_v,
                                     U4a4* __restrict__ dst_k, U4a4* __restrict__ dst_v, uint32_t tokens,
                                     uint32_t position, uint32_t src_mask, uint32_t dst_mask, uint32_t row_vec) {
    const uint64_t i = uint64_t(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i >= uint64_t(tokens) * row_vec) return;
    const uint32_t t = static_cast<uint32_t>(i / row_vec), c = static_cast<uint32_t>(i % row_vec);
    const size_t from = size_t((position + t) & src_mask) * row_vec + c, to = size_t((position + t) & dst_mask) * row_vec + c;
    dst_k[to] = src_k[from];
    dst_v[to] = src_v[from];
}

}  // namespace
}  // namespace guffin

using namespace guffin;

extern "C" int guffin_hip_kv_cache_copy(void* stream, const void* src_k, const void* src_v, void* dst_k, void* dst_v,
                                        uint32_t position, uint32_t tokens, uint32_t src_mask, uint32_t dst_mask,
                                        uint32_t row_width) {
    if (!src_k || !src_v || !dst_k || !dst_v) return fail(GUFFIN_E_ARG, "kv_cache_copy: null pointer");
    if (tokens == 0 || row_width == 0 || row_width % 8 != 0) return fail(GUFFIN_E_SHAPE, "kv_cache_copy: row width must be a multiple of 8 halves");
    if ((src_mask & (src_mask + 1)) != 0 || (dst_mask & (dst_mask + 1)) != 0)
        return fail(GUFFIN_E_ARG, "kv_cache_copy: row masks must be a power of two minus one");
    if (tokens > src_mask + 1 || tokens > dst_mask + 1) return fail(GUFFIN_E_CAPACITY, "kv_cache_copy: more tokens than rows on one side");
    if (((reinterpret_cast<uintptr_t>(src_k) | reinterpret_cast<uintptr_t>(src_v) | reinterpret_cast<uintptr_t>(dst_k)
          | reinterpret_cast<uintptr_t>(dst_v)) & 3u) != 0)
        return fail(GUFFIN_E_ALIGN, "kv_cache_copy: rows must be 4-byte aligned");
    const uint64_t n = uint64_t(tokens) * (row_width / 8);
    launch(kv_cache_copy_kernel, dim3(static_cast<uint32_t>((n + 255) / 256)), dim3(256), 0, as_stream(stream),
                       static_cast<const U4a4*>(src_k), static_cast<const U4a4*>(src_v), static_cast<U4a4*>(dst_k),
                       static_cast<U4a4*>(dst_v), tokens, position, src_mask, dst_mask, row_width / 8);
    return check_launch("kv_cache_copy");
}

extern "C" int guffin_hip_publish_run(void* stream, const void* run_k, const void* run_v, void* ring_k, void* ring_v,
                                      uint32_t rows, uint32_t position, uint32_t ring_mask, uint32_t row_width) {
    if (!run_k || !run_v || !ring_k || !ring_v) return fail(GUFFIN_E_ARG, "publish_run: null pointer");
    if (rows == 0 || row_width == 0 || row_width % 8 != 0) return fail(GUFFIN_E_SHAPE, "publish_run: row width must be a multiple of 8 halves");
    if ((ring_mask & (ring_mask + 1)) != 0) return fail(GUFFIN_E_ARG, "publish_run: ring capacity must be a power of two");
    if (((reinterpret_cast<uintptr_t>(run_k) | reinterpret_cast<uintptr_t>(run_v) | reinterpret_cast<uintptr_t>(ring_k)
          | reinterpret_cast<uintptr_t>(ring_v)) & 3u) != 0)
        return fail(GUFFIN_E_ALIGN, "publish_run: rows must be 4-byte aligned");
    const uint32_t first = rows > ring_mask + 1 ? rows - (ring_mask + 1) : 0;  // older rows would be overwritten anyway
    const uint64_t n = uint64_t(rows - first) * (row_width / 8);
    launch(publish_run_kernel, dim3(static_cast<uint32_t>((n + 255) / 256)), dim3(256), 0, as_stream(stream),
                       static_cast<const U4a4*>(run_k), static_cast<const U4a4*>(run_v), static_cast<U4a4*>(ring_k),
                       static_cast<U4a4*>(ring_v), rows, first, position, ring_mask, row_width / 8);
    return check_launch("publish_run");
}

extern "C" uint64_t guffin_hip_prefill_image_bytes(uint32_t M, uint32_t K) {
    if (M == 0 || K == 0 || K % 32 != 0) return 0;
    return image_layout(M, K).bytes;
}

extern "C" int guffin_hip_prefill_pack(void* stream, const float* x, void* image, uint32_t M, uint32_t K) {
    if (!x || !image) return fail(GUFFIN_E_ARG, "prefill_pack: null pointer");
    if (M == 0 || K == 0 || K % 32 != 0) return fail(GUFFIN_E_SHAPE, "prefill_pack: K must be a positive multiple of 32");
    if (reinterpret_cast<uintptr_t>(image) & 255u) return fail(GUFFIN_E_ALIGN, "prefill_pack: the image must be 256-byte aligned");
    const ImageLayout L = image_layout(M, K);
    const uint64_t threads = uint64_t(L.mpad) * (K / 32) * 4;
    launch(prefill_pack_kernel, dim3(static_cast<uint32_t>((threads + 255) / 256)), dim3(256), 0,
                       as_stream(stream), x, static_cast<uint8_t*>(image), M, K);
    return check_launch("prefill_pack");
}

extern "C" int guffin_hip_prefill_gemm(void* stream, int dtype, const void* tiles, const void* image, float* y,
                                       uint32_t M, uint32_t K, uint32_t N) {
    if (!tiles || !image || !y) return fail(GUFFIN_E_ARG, "prefill_gemm: null pointer");
    if (dtype < GUFFIN_Q8_0 || dtype > GUFFIN_Q6_K) return fail(GUFFIN_E_ARG, "prefill_gemm: unknown dtype");
    if (M == 0 || K == 0 || N == 0 || K % block_elems(dtype) != 0 || N % kCols != 0)
        return fail(GUFFIN_E_SHAPE, "prefill_gemm: need K % block == 0 and N % 64 == 0");
    if ((reinterpret_cast<uintptr_t>(tiles) & 15u) || (reinterpret_cast<uintptr_t>(image) & 255u))
        return fail(GUFFIN_E_ALIGN, "prefill_gemm: tiles need 16-byte, the image 256-byte alignment");
    const ImageLayout L = image_layout(M, K);
    // the Q4_K and Q6_K kernels address the image with 32-bit offsets
    if (L.bytes >= (size_t(1) << 31)) return fail(GUFFIN_E_SHAPE, "prefill_gemm: the image of M x K exceeds 2 GiB, split the rows");
    const dim3 grid(N / kCols, L.mpad / kChunkRows), block(256);
    hipStream_t s = as_stream(stream);
    const uint8_t* t = static_cast<const uint8_t*>(tiles);
    const uint8_t* im = static_cast<const uint8_t*>(image);
    if (dtype == GUFFIN_Q4_K)
        launch(prefill_gemm_q4k_kernel, dim3(L.mpad / kWaveRows, (N / kCols + 3) / 4), block, 0, s, t, im, y, M, K, N);
    else if (dtype == GUFFIN_Q6_K)
        launch(prefill_gemm_q6k_kernel, dim3(L.mpad / kWaveRows, (N / kCols + 1) / 2), block, 0, s, t, im, y, M, K, N);
    else launch(prefill_gemm_kernel<GUFFIN_Q8_0>, grid, block, 0, s, t, im, y, M, K, N);
    return check_launch("prefill_gemm");
}

namespace {
struct ValueSpan { uint32_t first_visible, base32, T; };
// virtual tokens whose values a run of `rows` rows at `position` can see, padded to whole 32-token tiles
ValueSpan value_span(uint32_t rows, uint32_t position, uint32_t window) {
    const uint32_t first = (window && position + 1 > window) ? position + 1 - window : 0;
    const uint32_t base32 = first & ~31u;
    return {first, base32, (position + rows - base32 + 31u) & ~31u};
}
}  // namespace

extern "C" uint64_t guffin_hip_prefill_attention_workspace_bytes(uint32_t rows, uint32_t position, uint32_t window,
                                                                 uint32_t kv_heads, uint32_t head_dim) {
    if (rows == 0 || kv_heads == 0 || head_dim != 256) return 0;
    return uint64_t(kv_heads) * head_dim * value_span(rows, position, window).T * 2;
}

extern "C" int guffin_hip_prefill_attention(void* stream, const float* q, const void* ring_k, const void* ring_v,
                                            const void* run_k, const void* run_v, float* out, uint32_t rows,
                                            uint32_t position, uint32_t window, uint32_t ring_mask,
                                            uint32_t q_heads, uint32_t kv_heads, uint32_t head_dim, float scale,
                                            void* workspace) {
    if (!q || !ring_k || !ring_v || !run_k || !run_v || !out) return fail(GUFFIN_E_ARG, "prefill_attention: null pointer");
    if (rows == 0 || head_dim != 256 || kv_heads == 0 || q_heads % kv_heads != 0)
        return fail(GUFFIN_E_SHAPE, "prefill_attention: head_dim must be 256 and q_heads a multiple of kv_heads");
    if ((ring_mask & (ring_mask + 1)) != 0) return fail(GUFFIN_E_ARG, "prefill_attention: ring capacity must be a power of two");
    const uint32_t past = window ? (window - 1 < position ? window - 1 : position) : position;  // ring tokens a row can see
    if (past > ring_mask + 1) return fail(GUFFIN_E_CAPACITY, "prefill_attention: the ring does not hold the visible past");
    if (!(scale > 0.f)) return fail(GUFFIN_E_ARG, "prefill_attention: scale must be positive");
    if (reinterpret_cast<uintptr_t>(workspace) & 15u) return fail(GUFFIN_E_ALIGN, "prefill_attention: workspace must be 16-byte aligned");
    const uint32_t group = q_heads / kv_heads;
    const dim3 grid((rows + 15) / 16, kv_heads), block(256);
    hipStream_t s = as_stream(stream);
    const uint16_t* rk = static_cast<const uint16_t*>(ring_k);
    const uint16_t* rv = static_cast<const uint16_t*>(ring_v);
    const uint16_t* uk = static_cast<const uint16_t*>(run_k);
    const uint16_t* uv = static_cast<const uint16_t*>(run_v);
    if (workspace && group <= 2 && (reinterpret_cast<uintptr_t>(q) & 15u) == 0
        && ((reinterpret_cast<uintptr_t>(ring_k) | reinterpret_cast<uintptr_t>(run_k) | reinterpret_cast<uintptr_t>(ring_v)
             | reinterpret_cast<uintptr_t>(run_v)) & 15u) == 0) {
        // matrix-core path: V^T first, then scores and values as MFMA chains
        const ValueSpan vs = value_span(rows, position, window);
        uint16_t* vt = static_cast<uint16_t*>(workspace);
        launch(transpose_values_kernel, dim3(vs.T / 32, kv_heads), dim3(256), 0, s, rv, uv, vt, vs.base32, vs.T,
                           vs.first_visible, position, position + rows, ring_mask, kv_heads);
        if (int rc = check_launch("transpose_values")) return rc;
        const size_t lds = size_t(group) * 16384 + size_t(4) * group * 16 * 32 * 4 + size_t(group) * 16 * 2 * 4;
        if (group == 1)
            launch(prefill_attention_mfma_kernel<1>, grid, block, lds, s, q, rk, uk, vt, out, rows, position, window,
                               ring_mask, q_heads, kv_heads, scale, vs.base32, vs.T);
        else
            launch(prefill_attention_mfma_kernel<2>, grid, block, lds, s, q, rk, uk, vt, out, rows, position, window,
                               ring_mask, q_heads, kv_heads, scale, vs.base32, vs.T);
        return check_launch("prefill_attention_mfma");
    }
#define GUFFIN_PA(G_) launch(prefill_attention_kernel<G_>, grid, block, 0, s, q, rk, rv, uk, uv, out, rows, \
                                         position, window, ring_mask, q_heads, kv_heads, scale)
    if (group == 1) GUFFIN_PA(1); else if (group == 2) GUFFIN_PA(2); else if (group == 4) GUFFIN_PA(4);
    else return fail(GUFFIN_E_SHAPE, "prefill_attention: q_heads / kv_heads must be 1, 2 or 4");
#undef GUFFIN_PA
    return check_launch("prefill_attention");
}
