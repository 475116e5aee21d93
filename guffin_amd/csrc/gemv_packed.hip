// Wave-tile weight layout and the dequant-GEMV that streams it (gfx950, wavefront 64).
//
// Role in the reference: the Metal backend re-lays K-quant weights once at upload into a
// "columns8" order for its SIMD-group loads and keeps that repack lossless
// (src/tensor/kquant_packing.hpp:9-23, src/tensor/kquant_packing.cpp).  This file is the
// CDNA counterpart: a lossless repack into 64-column wave tiles plus the GEMV kernels
// (replacing src/tensor/backends/metal/metal_kernels.mm:551-750, 788-922, 267-436) that
// consume it.
//
// Tile = 64 adjacent output columns x one block along K, tiles of one column group
// consecutive along K, same byte count as the GGUF stream.  Inside a tile the quant bytes are
// laid out for the matrix core: the wave treats the 64 columns as four groups of 16; lane
// (j = lane % 16, s = lane / 16) holds, for each group, the bytes of elements 8s..8s+7 of every
// 32-element run of column 16*group + j, in 16-byte pieces stored lane-major (piece p of lane l
// at p*1024 + l*16, one coalesced 1 KiB load per piece).  Scales and d/dmin sit behind the
// quant pieces indexed by column (tile_offset below is the exact map; unpack inverts it).
//   Q4_K  9216 B : pieces 0..7 quants, piece 8 = {d, dmin, 12 scale bytes} of column `lane`
//   Q6_K 13440 B : pieces 0..7 ql, 8..11 qh, piece 12 = 16 int8 scales, then 64 x fp16 d
//   Q8_0  2176 B : pieces 0..1 quants, then 64 x fp16 d
//
// GEMV: one v_mfma_f32_16x16x32_f16 per 32 elements and column group.  B = the quants as fp16
// subnormals (an integer n < 1024 in a half is exactly n*2^-24, and the matrix core honours
// subnormal inputs), A = the activation image of the producer's receipt (hi/lo fp16 split of
// x * 2^-E per 32-group, four variants = two rows), so every product is exact and sums are
// fp32.  Block scales are applied to the per-group sums in fp32 by the lane that owns the
// column; the offset terms (-dmin*m for Q4_K, -32 for Q6_K, -128 for the biased Q8_0 bytes)
// use the receipt's 16- / 32-sums.  K is cut into slices: up to 16 slices are the waves of
// one workgroup, combined in wave order through LDS; the remaining S "planes" go to
// [S][rows][N] and are summed in plane order by the consumer (or by reduce_partials below).
// The split depends on the shape only, and a row's arithmetic does not depend on how many
// rows are computed, so results are deterministic and 2-row rows equal 1-row calls bit for bit.
#include "common.hpp"
#include "receipt.hpp"
#include "gemv_tiles.hpp"

namespace guffin {
namespace {

// offset of canonical block byte `o` (even) of lane `l` inside its tile
template <int DTYPE>
__device__ __forceinline__ uint32_t tile_offset(uint32_t o, uint32_t l) {
    if constexpr (DTYPE == GUFFIN_Q4_K) {
        // matrix-core tile: the 16-byte header is piece 8 of lane l; quant byte q = o - 16 belongs
        // to 32-byte chunk ch, k-slice s = (q % 32) / 8; column l = 16*cg + j feeds lane 16*s + j
        // of column group cg, piece 2*cg + ch/2, as bytes (ch % 2)*8 + q % 8
        if (o < 16u) return 8u * 1024u + l * 16u + o;
        const uint32_t q = o - 16u, ch = q >> 5, s = (q & 31u) >> 3, cg = l >> 4, j = l & 15u;
        return (2u * cg + (ch >> 1)) * 1024u + (16u * s + j) * 16u + (ch & 1u) * 8u + (q & 7u);
    } else if constexpr (DTYPE == GUFFIN_Q6_K) {
        // ql byte o: half n = o/64, run m = (o%64)/32, k-slice s = (o%32)/8 -> piece 2*cg + n, lane
        // 16*s + j, byte 8*m + o%8.  qh byte o-128: half n, k-slice s -> piece 8 + cg, byte 8*n + o%8.
        // Scales: piece 12 of the column's lane; d: after the pieces.
        const uint32_t cg = l >> 4, j = l & 15u;
        if (o < 128u) {
            const uint32_t n = o >> 6, m = (o & 63u) >> 5, s = (o & 31u) >> 3;
            return (2u * cg + n) * 1024u + (16u * s + j) * 16u + 8u * m + (o & 7u);
        }
        if (o < 192u) {
            const uint32_t q = o - 128u, n = q >> 5, s = (q & 31u) >> 3;
            return (8u + cg) * 1024u + (16u * s + j) * 16u + 8u * n + (q & 7u);
        }
        return o < 208u ? 12288u + l * 16u + (o - 192u) : 13312u + l * 2u + (o - 208u);
    } else {
        // Q8_0: quant byte q = o - 2, k-slice s = q/8 -> piece cg/2, lane 16*s + j, byte 8*(cg%2) + q%8
        if (o < 2u) return 2048u + l * 2u + o;
        const uint32_t q = o - 2u, cg = l >> 4, j = l & 15u, s = q >> 3;
        return (cg >> 1) * 1024u + (16u * s + j) * 16u + 8u * (cg & 1u) + (q & 7u);
    }
}

// One thread moves one 16-bit word (every field of every block is 2-byte aligned on both sides).
template <int DTYPE, bool TO_TILES>
__global__ void repack_kernel(const uint16_t* __restrict__ src, uint16_t* __restrict__ dst,
                              uint32_t nblk, uint64_t total_words) {
    constexpr uint32_t BB = block_bytes(DTYPE), WPB = BB / 2;
    const uint64_t stride = uint64_t(gridDim.x) * blockDim.x;
    for (uint64_t i = uint64_t(blockIdx.x) * blockDim.x + threadIdx.x; i < total_words; i += stride) {
        // canonical word index -> (column, block, word in block)
        const uint64_t blk = i / WPB;
        const uint32_t wd = static_cast<uint32_t>(i - blk * WPB);
        const uint64_t col = blk / nblk;
        const uint32_t b = static_cast<uint32_t>(blk - col * nblk);
        const uint64_t tile = (col / kTileCols) * nblk + b;
        const uint32_t lane = static_cast<uint32_t>(col % kTileCols);
        const uint64_t t = tile * (uint64_t(kTileCols) * WPB) + tile_offset<DTYPE>(wd * 2u, lane) / 2u;
        if (TO_TILES) dst[t] = src[i];
        else dst[i] = src[t];
    }
}

// One workgroup per row writes the row's activation receipt (sums, multipliers, image).
__global__ void __launch_bounds__(256) group_sums_kernel(const float* __restrict__ x, void* __restrict__ receipt, uint32_t K, uint32_t rows) {
    emit_receipt(x + size_t(blockIdx.x) * K, 0, K, blockIdx.x, rows, K, receipt);
}

__global__ void reduce_partials_kernel(const float* __restrict__ part, float* __restrict__ y, uint32_t S, uint32_t count) {
    for (uint32_t i = blockIdx.x * blockDim.x + threadIdx.x; i < count; i += gridDim.x * blockDim.x) {
        float t = part[i];
        for (uint32_t s = 1; s < S; ++s) t += part[size_t(s) * count + i];
        y[i] = t;
    }
}

// Workgroup = W waves over consecutive k-slices of one column tile; the W per-lane sums are
// combined through LDS in wave order and written as one plane.  grid = (tiles, planes).
struct PackedCfg { uint32_t K, nblk, bps, W; };

template <int R>
__device__ __forceinline__ void finish_tile(float (&acc)[R], float* __restrict__ part, uint32_t N, uint32_t ct,
                                            uint32_t plane, uint32_t W) {
    __shared__ float red[16 * 2 * 64];
    const uint32_t lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
    if (W == 1) {
#pragma unroll
        for (int r = 0; r < R; ++r) part[(size_t(plane) * R + r) * N + ct * kTileCols + lane] = acc[r];
        return;
    }
#pragma unroll
    for (int r = 0; r < R; ++r) red[(wv * R + r) * 64 + lane] = acc[r];
    __syncthreads();
    if (threadIdx.x < R * 64) {
        const uint32_t r = threadIdx.x >> 6;
        float t = red[r * 64 + lane];
        for (uint32_t w = 1; w < W; ++w) t += red[(w * R + r) * 64 + lane];
        part[(size_t(plane) * R + r) * N + ct * kTileCols + lane] = t;
    }
}

// Q6_K tiles need more than the 128 registers a 16-wave workgroup leaves each lane.
constexpr uint32_t max_waves(int dtype) { return dtype == GUFFIN_Q6_K ? 8 : 16; }
constexpr int kMixed = 3;  // Q4_K and Q6_K matrices in one launch

template <int DTYPE, int R>
__global__ void __launch_bounds__(64 * max_waves(DTYPE))
gemv_packed_kernel(const uint8_t* __restrict__ wt, const float* __restrict__ x, const float* __restrict__ xsums,
                   float* __restrict__ part, uint32_t N, PackedCfg c) {
    const uint32_t slice = blockIdx.y * c.W + __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t b0 = min(slice * c.bps, c.nblk), b1 = min(b0 + c.bps, c.nblk);
    float acc[R];
    run_blocks<DTYPE, R>(wt, x, xsums, c.K, c.nblk, blockIdx.x, b0, b1, acc);
    finish_tile<R>(acc, part, N, blockIdx.x, blockIdx.y, c.W);
}

// Q6_K with one block per wave and 16 waves per workgroup (shapes whose split leaves every wave a single block)
template <int R>
__global__ void __launch_bounds__(1024)
gemv_q6k_single_kernel(const uint8_t* __restrict__ wt, const float* __restrict__ x, const float* __restrict__ xsums,
                       float* __restrict__ part, uint32_t N, PackedCfg c) {
    const uint32_t slice = blockIdx.y * c.W + __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t b0 = min(slice, c.nblk), b1 = min(b0 + 1u, c.nblk);
    float acc[R];
    run_blocks<GUFFIN_Q6_K, R, true>(wt, x, xsums, c.K, c.nblk, blockIdx.x, b0, b1, acc);
    finish_tile<R>(acc, part, N, blockIdx.x, blockIdx.y, c.W);
}

// Several matrices that share the activation rows (q/k/v, gate/up) in one launch: the column
// tiles of all matrices sit side by side along grid x.  COUNT also names the instantiation
// so that profiles tell q/k/v (3) from gate/up (2).
struct MultiMeta { uint32_t N[3], dtype[3], tile_end[3]; };

template <int R, int COUNT, int MODE>
__global__ void __launch_bounds__(64 * max_waves(MODE == kMixed ? GUFFIN_Q6_K : MODE))
gemv_packed_multi_kernel(const uint8_t* __restrict__ t0, const uint8_t* __restrict__ t1, const uint8_t* __restrict__ t2,
                         float* __restrict__ p0, float* __restrict__ p1, float* __restrict__ p2,
                         const float* __restrict__ x, const float* __restrict__ xsums, MultiMeta m, PackedCfg c) {
    uint32_t which = 0;
    if (COUNT > 1 && blockIdx.x >= m.tile_end[0]) which = 1;
    if (COUNT > 2 && blockIdx.x >= m.tile_end[1]) which = 2;
    const uint32_t first = which == 0 ? 0 : m.tile_end[which - 1];
    const uint8_t* __restrict__ wt = which == 0 ? t0 : which == 1 ? t1 : t2;
    float* __restrict__ part = which == 0 ? p0 : which == 1 ? p1 : p2;
    const uint32_t ct = blockIdx.x - first, N = m.N[which];
    [[maybe_unused]] const uint32_t dtype = m.dtype[which];
    const uint32_t slice = blockIdx.y * c.W + __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t b0 = min(slice * c.bps, c.nblk), b1 = min(b0 + c.bps, c.nblk);
    float acc[R];
    if constexpr (MODE == kMixed) {
        if (dtype == GUFFIN_Q4_K) run_blocks<GUFFIN_Q4_K, R>(wt, x, xsums, c.K, c.nblk, ct, b0, b1, acc);
        else run_blocks<GUFFIN_Q6_K, R>(wt, x, xsums, c.K, c.nblk, ct, b0, b1, acc);
    } else {
        run_blocks<MODE, R>(wt, x, xsums, c.K, c.nblk, ct, b0, b1, acc);
    }
    finish_tile<R>(acc, part, N, ct, blockIdx.y, c.W);
}

// gate and up projections of one column tile in one workgroup (waves [0, W) gate, [W, 2W) up,
// k-slices combined in wave order), then h = gelu_tanh(gate) * up for the 64 columns and the two
// 32-groups of h's activation receipt: no partial planes and no separate GeGLU launch.
template <int DTYPE, int R>
__global__ void __launch_bounds__(1024)
gateup_geglu_kernel(const uint8_t* __restrict__ gate_tiles, const uint8_t* __restrict__ up_tiles,
                    const float* __restrict__ x, const float* __restrict__ xsums, float* __restrict__ h,
                    void* __restrict__ h_receipt, uint32_t F, PackedCfg c) {
    __shared__ float red[16 * 2 * 64];
    __shared__ float vals[2 * 64];
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
    const bool is_up = wave >= c.W;
    const uint32_t slice = is_up ? wave - c.W : wave;
    const uint32_t b0 = min(slice * c.bps, c.nblk), b1 = min(b0 + c.bps, c.nblk);
    float acc[R];
    run_blocks<DTYPE, R>(is_up ? up_tiles : gate_tiles, x, xsums, c.K, c.nblk, blockIdx.x, b0, b1, acc);
#pragma unroll
    for (int r = 0; r < R; ++r) red[(wave * R + r) * 64 + lane] = acc[r];
    __syncthreads();
    if (threadIdx.x < R * 64) {
        const uint32_t r = threadIdx.x >> 6;
        float g = red[r * 64 + lane], u = red[(c.W * R + r) * 64 + lane];
        for (uint32_t w = 1; w < c.W; ++w) { g += red[(w * R + r) * 64 + lane]; u += red[((c.W + w) * R + r) * 64 + lane]; }
        const float v = geglu_value(g, u);
        h[size_t(r) * F + blockIdx.x * kTileCols + lane] = v;
        vals[r * 64 + lane] = v;
    }
    __syncthreads();
    if (h_receipt) {
#pragma unroll
        for (int r = 0; r < R; ++r) emit_receipt(vals + r * 64, blockIdx.x * kTileCols, kTileCols, r, R, F, h_receipt);
    }
}

int g_cus = 256;

// Scratch of the entry point that allocates nothing (guffin_hip_gemv_packed_static): the partial
// planes of one launch.  Every GPU the library runs on holds its own copy of this array at its own
// address until the process ends; host code reaches it only through the pointer taken at init.
constexpr uint32_t kStaticScratchFloats = 32768;   // 128 KiB: planes * rows * N of the largest supported launch
static __device__ __align__(256) float scratch[kStaticScratchFloats];
constexpr int kMaxDevices = 64;
float* g_scratch_ptr[kMaxDevices] = {};

// Work split of a launch over `tiles` column tiles of `nblk` blocks each: blocks per wave so
// that the chip holds about four waves per SIMD, waves per workgroup (k-slices reduced in LDS,
// at most max_w) and planes (k-slices left to the consumer), preferring one workgroup per CU.
struct Split { uint32_t bps, W, planes; };
Split choose_split(uint32_t nblk, uint32_t tiles, uint32_t max_w, uint32_t waves_per_cu = 0) {
    // a kernel capped at 8 waves per workgroup is register-bound: a CU holds 8 of its waves, not 16
    if (waves_per_cu == 0) waves_per_cu = max_w < 16 ? 8 : 16;
    const uint64_t units = uint64_t(tiles) * nblk, target_waves = uint64_t(g_cus) * waves_per_cu;
    uint32_t bps = static_cast<uint32_t>((units + target_waves - 1) / target_waves);
    if (bps < 1) bps = 1;
    const uint32_t wpt = (nblk + bps - 1) / bps;  // waves per tile
    uint32_t planes = (wpt + max_w - 1) / max_w;
    if (tiles * planes * 4 < uint32_t(g_cus) * 3) {  // fewer workgroups than 3/4 of the CUs: split further
        uint32_t want = (g_cus + tiles - 1) / tiles;
        if (want > 4) want = 4;  // small matrices are latency-bound: more planes only slow their consumers
        if (want > wpt) want = wpt;
        if (want > planes) planes = want;
    }
    uint32_t W = (wpt + planes - 1) / planes;
    planes = (wpt + W - 1) / W;
    return {bps, W, planes};
}

// The split of a single-matrix launch.  A Q6_K shape whose finest split leaves every wave one block runs
// the single-block kernel: without a second tile in registers 16 waves fit a workgroup.
struct PackedPlan { Split sp; bool single; };
PackedPlan packed_plan(int dtype, uint32_t nblk, uint32_t tiles) {
    if (dtype == GUFFIN_Q6_K) {
        const Split wide = choose_split(nblk, tiles, 16, 16);
        if (wide.bps == 1) return {wide, true};
    }
    return {choose_split(nblk, tiles, max_waves(dtype)), false};
}

template <int DTYPE>
int launch_packed(hipStream_t s, const uint8_t* w, const float* x, const float* xsums, float* part,
                  uint32_t rows, uint32_t K, uint32_t N) {
    const uint32_t nblk = K / block_elems(DTYPE);
    const PackedPlan plan = packed_plan(DTYPE, nblk, N / kTileCols);
    const Split sp = plan.sp;
    const PackedCfg c {K, nblk, sp.bps, sp.W};
    const dim3 grid(N / kTileCols, sp.planes), block(sp.W * 64);
    if constexpr (DTYPE == GUFFIN_Q6_K) {
        if (plan.single) {
            if (rows == 2) launch((gemv_q6k_single_kernel<2>), grid, block, 0, s, w, x, xsums, part, N, c);
            else launch((gemv_q6k_single_kernel<1>), grid, block, 0, s, w, x, xsums, part, N, c);
            return check_launch("gemv_packed");
        }
    }
    if (rows == 2) launch((gemv_packed_kernel<DTYPE, 2>), grid, block, 0, s, w, x, xsums, part, N, c);
    else launch((gemv_packed_kernel<DTYPE, 1>), grid, block, 0, s, w, x, xsums, part, N, c);
    return check_launch("gemv_packed");
}

}  // namespace

// Called by guffin_hip_init with `device` current: the split heuristics' CU count and this device's
// address of the static scratch array.
int gemv_packed_init(int device, int cu_count) {
    g_cus = cu_count > 0 ? cu_count : 256;
    if (device < 0 || device >= kMaxDevices) return -1;
    float* ptr = nullptr;
    if (hipGetSymbolAddress(reinterpret_cast<void**>(&ptr), HIP_SYMBOL(scratch)) != hipSuccess || !ptr) return -1;
    g_scratch_ptr[device] = ptr;
    return 0;
}

}  // namespace guffin

using namespace guffin;

static int check_packed_shape(const char* what, int dtype, uint32_t K, uint32_t N) {
    if (dtype < GUFFIN_Q8_0 || dtype > GUFFIN_Q6_K) return fail(GUFFIN_E_ARG, what);
    if (K == 0 || N == 0 || K % block_elems(dtype) != 0 || N % kTileCols != 0) return fail(GUFFIN_E_SHAPE, what);
    return GUFFIN_OK;
}

extern "C" uint64_t guffin_hip_packed_bytes(int dtype, uint32_t K, uint32_t N) {
    if (check_packed_shape("packed_bytes: need K % block == 0 and N % 64 == 0", dtype, K, N)) return 0;
    return uint64_t(N) * (K / block_elems(dtype)) * block_bytes(dtype);
}

static int repack_common(void* stream, int dtype, const void* src, void* dst, uint32_t K, uint32_t N, bool to_tiles) {
    if (!src || !dst) return fail(GUFFIN_E_ARG, "repack: null pointer");
    if (int rc = check_packed_shape("repack: need K % block == 0 and N % 64 == 0", dtype, K, N)) return rc;
    if ((reinterpret_cast<uintptr_t>(to_tiles ? dst : src) & 15u) || (reinterpret_cast<uintptr_t>(to_tiles ? src : dst) & 1u))
        return fail(GUFFIN_E_ALIGN, "repack: tiles must be 16-byte aligned, the canonical stream 2-byte aligned");
    const uint32_t nblk = K / block_elems(dtype);
    const uint64_t words = uint64_t(N) * nblk * block_bytes(dtype) / 2;
    const uint32_t grid = static_cast<uint32_t>(words / 256 < 262144 ? (words + 255) / 256 : 262144);
    const uint16_t* s16 = static_cast<const uint16_t*>(src);
    uint16_t* d16 = static_cast<uint16_t*>(dst);
    hipStream_t s = as_stream(stream);
#define GUFFIN_REPACK(DT)                                                                                   \
    if (to_tiles) launch((repack_kernel<DT, true>), dim3(grid), dim3(256), 0, s, s16, d16, nblk, words); \
    else launch((repack_kernel<DT, false>), dim3(grid), dim3(256), 0, s, s16, d16, nblk, words)
    if (dtype == GUFFIN_Q4_K) { GUFFIN_REPACK(GUFFIN_Q4_K); }
    else if (dtype == GUFFIN_Q6_K) { GUFFIN_REPACK(GUFFIN_Q6_K); }
    else { GUFFIN_REPACK(GUFFIN_Q8_0); }
#undef GUFFIN_REPACK
    return check_launch("repack");
}

extern "C" int guffin_hip_repack(void* stream, int dtype, const void* canonical, void* tiles, uint32_t K, uint32_t N) {
    return repack_common(stream, dtype, canonical, tiles, K, N, true);
}

extern "C" int guffin_hip_unpack(void* stream, int dtype, const void* tiles, void* canonical, uint32_t K, uint32_t N) {
    return repack_common(stream, dtype, tiles, canonical, K, N, false);
}

extern "C" int guffin_hip_group_sums(void* stream, const float* x, float* xsums, uint32_t rows, uint32_t K) {
    if (!x || !xsums) return fail(GUFFIN_E_ARG, "group_sums: null pointer");
    if (rows == 0 || rows > 2 || K == 0 || K % 32 != 0) return fail(GUFFIN_E_SHAPE, "group_sums: K must be a positive multiple of 32, rows 1 or 2");
    if (reinterpret_cast<uintptr_t>(xsums) & 255u) return fail(GUFFIN_E_ALIGN, "group_sums: the receipt must be 256-byte aligned");
    launch(group_sums_kernel, dim3(rows), dim3(256), 0, as_stream(stream), x, xsums, K, rows);
    return check_launch("group_sums");
}

extern "C" uint64_t guffin_hip_receipt_bytes(uint32_t rows, uint32_t K) {
    if (rows == 0 || rows > 2 || K == 0 || K % 32 != 0) return 0;
    return receipt_layout(rows, K).bytes;
}

extern "C" uint32_t guffin_hip_gemv_packed_slices(int dtype, uint32_t K, uint32_t N) {
    if (check_packed_shape("gemv_packed_slices: need K % block == 0 and N % 64 == 0", dtype, K, N)) return 0;
    return packed_plan(dtype, K / block_elems(dtype), N / kTileCols).sp.planes;
}

static int multi_split(const char* what, uint32_t count, const int* dtypes, const uint32_t* N, uint32_t K, Split* out, int* mode) {
    if (!dtypes || !N) return fail(GUFFIN_E_ARG, what);
    if (count == 0 || count > 3) return fail(GUFFIN_E_SHAPE, "gemv_packed_multi: 1 to 3 matrices");
    uint32_t tiles = 0;
    *mode = dtypes[0];
    for (uint32_t i = 0; i < count; ++i) {
        if (int rc = check_packed_shape("gemv_packed_multi: need K % block == 0 and N % 64 == 0", dtypes[i], K, N[i])) return rc;
        if (dtypes[i] != dtypes[0]) *mode = kMixed;
        if (block_elems(dtypes[i]) != block_elems(dtypes[0]))
            return fail(GUFFIN_E_SHAPE, "gemv_packed_multi: matrices of one launch must share the block length");
        tiles += N[i] / kTileCols;
    }
    *out = choose_split(K / block_elems(dtypes[0]), tiles, max_waves(*mode == kMixed ? GUFFIN_Q6_K : *mode));
    return GUFFIN_OK;
}

extern "C" uint32_t guffin_hip_gemv_packed_multi_slices(uint32_t count, const int* dtypes, const uint32_t* N, uint32_t K) {
    Split sp {};
    int mode = 0;
    if (multi_split("gemv_packed_multi_slices: null pointer", count, dtypes, N, K, &sp, &mode)) return 0;
    return sp.planes;
}

extern "C" int guffin_hip_gemv_packed_multi(void* stream, uint32_t count, const int* dtypes, const void* const* tiles,
                                            const uint32_t* N, float* const* partials, const float* x,
                                            const float* xsums, uint32_t rows, uint32_t K) {
    if (!tiles || !partials || !x || !xsums) return fail(GUFFIN_E_ARG, "gemv_packed_multi: null pointer");
    if (rows == 0 || rows > 2) return fail(GUFFIN_E_SHAPE, "gemv_packed_multi: rows must be 1 or 2");
    Split sp {};
    int mode = 0;
    if (int rc = multi_split("gemv_packed_multi: null pointer", count, dtypes, N, K, &sp, &mode)) return rc;
    if (count == 1) {
        if (!tiles[0] || !partials[0]) return fail(GUFFIN_E_ARG, "gemv_packed_multi: null pointer");
        return guffin_hip_gemv_packed(stream, dtypes[0], tiles[0], x, xsums, partials[0], nullptr, rows, K, N[0]);
    }
    MultiMeta m {};
    const uint8_t* t[3] = {nullptr, nullptr, nullptr};
    float* p[3] = {nullptr, nullptr, nullptr};
    uint32_t tile_end = 0;
    for (uint32_t i = 0; i < count; ++i) {
        if (!tiles[i] || !partials[i]) return fail(GUFFIN_E_ARG, "gemv_packed_multi: null pointer");
        if (reinterpret_cast<uintptr_t>(tiles[i]) & 15u) return fail(GUFFIN_E_ALIGN, "gemv_packed_multi: tiles must be 16-byte aligned");
        tile_end += N[i] / kTileCols;
        m.N[i] = N[i]; m.dtype[i] = static_cast<uint32_t>(dtypes[i]); m.tile_end[i] = tile_end;
        t[i] = static_cast<const uint8_t*>(tiles[i]); p[i] = partials[i];
    }
    for (uint32_t i = count; i < 3; ++i) { t[i] = t[0]; p[i] = p[0]; m.tile_end[i] = tile_end; m.N[i] = m.N[0]; m.dtype[i] = m.dtype[0]; }
    const PackedCfg c {K, K / block_elems(dtypes[0]), sp.bps, sp.W};
    const dim3 grid(tile_end, sp.planes), block(sp.W * 64);
    hipStream_t s = as_stream(stream);
#define GUFFIN_MULTI(R_, C_, M_) launch((gemv_packed_multi_kernel<R_, C_, M_>), grid, block, 0, s, t[0], t[1], t[2], p[0], p[1], p[2], x, xsums, m, c)
#define GUFFIN_MULTI_MODE(R_, C_) do { \
        if (mode == GUFFIN_Q4_K) GUFFIN_MULTI(R_, C_, GUFFIN_Q4_K); else if (mode == GUFFIN_Q6_K) GUFFIN_MULTI(R_, C_, GUFFIN_Q6_K); \
        else if (mode == GUFFIN_Q8_0) GUFFIN_MULTI(R_, C_, GUFFIN_Q8_0); else GUFFIN_MULTI(R_, C_, kMixed); } while (0)
    if (rows == 2) { if (count == 3) GUFFIN_MULTI_MODE(2, 3); else GUFFIN_MULTI_MODE(2, 2); }
    else { if (count == 3) GUFFIN_MULTI_MODE(1, 3); else GUFFIN_MULTI_MODE(1, 2); }
#undef GUFFIN_MULTI_MODE
#undef GUFFIN_MULTI
    return check_launch("gemv_packed_multi");
}

extern "C" int guffin_hip_gateup_geglu(void* stream, int dtype, const void* gate_tiles, const void* up_tiles,
                                       const float* x, const float* xsums, float* h, float* h_sums,
                                       uint32_t rows, uint32_t K, uint32_t F) {
    if (!gate_tiles || !up_tiles || !x || !xsums || !h) return fail(GUFFIN_E_ARG, "gateup_geglu: null pointer");
    if (dtype != GUFFIN_Q4_K && dtype != GUFFIN_Q8_0) return fail(GUFFIN_E_SHAPE, "gateup_geglu: Q4_K or Q8_0 pairs only");
    if (rows == 0 || rows > 2) return fail(GUFFIN_E_SHAPE, "gateup_geglu: rows must be 1 or 2");
    if (int rc = check_packed_shape("gateup_geglu: need K % block == 0 and F % 64 == 0", dtype, K, F)) return rc;
    if ((reinterpret_cast<uintptr_t>(gate_tiles) & 15u) || (reinterpret_cast<uintptr_t>(up_tiles) & 15u))
        return fail(GUFFIN_E_ALIGN, "gateup_geglu: tiles must be 16-byte aligned");
    if (reinterpret_cast<uintptr_t>(h_sums) & 255u) return fail(GUFFIN_E_ALIGN, "gateup_geglu: the receipt must be 256-byte aligned");
    const uint32_t nblk = K / block_elems(dtype), tiles = F / kTileCols;
    Split sp = choose_split(nblk, 2 * tiles, 8, 16);  // two matrices of up to 8 waves each in a workgroup
    if (sp.planes > 1) {  // all k-slices of a tile must sit in one workgroup: at most 8 per matrix
        sp.bps = (nblk + 7) / 8;
        sp.W = (nblk + sp.bps - 1) / sp.bps;
    }
    const PackedCfg c {K, nblk, sp.bps, sp.W};
    const dim3 grid(tiles), block(2 * sp.W * 64);
    hipStream_t s = as_stream(stream);
    const uint8_t* g = static_cast<const uint8_t*>(gate_tiles);
    const uint8_t* u = static_cast<const uint8_t*>(up_tiles);
#define GUFFIN_GU(D_, R_) launch((gateup_geglu_kernel<D_, R_>), grid, block, 0, s, g, u, x, xsums, h, h_sums, F, c)
    if (dtype == GUFFIN_Q4_K) { if (rows == 2) GUFFIN_GU(GUFFIN_Q4_K, 2); else GUFFIN_GU(GUFFIN_Q4_K, 1); }
    else { if (rows == 2) GUFFIN_GU(GUFFIN_Q8_0, 2); else GUFFIN_GU(GUFFIN_Q8_0, 1); }
#undef GUFFIN_GU
    return check_launch("gateup_geglu");
}

extern "C" int guffin_hip_gemv_packed(void* stream, int dtype, const void* tiles, const float* x, const float* xsums,
                                      float* partials, float* y, uint32_t rows, uint32_t K, uint32_t N) {
    if (!tiles || !x || !xsums || !partials) return fail(GUFFIN_E_ARG, "gemv_packed: null pointer");
    if (int rc = check_packed_shape("gemv_packed: need K % block == 0 and N % 64 == 0", dtype, K, N)) return rc;
    if (rows == 0 || rows > 2) return fail(GUFFIN_E_SHAPE, "gemv_packed: rows must be 1 or 2");
    if (reinterpret_cast<uintptr_t>(tiles) & 15u) return fail(GUFFIN_E_ALIGN, "gemv_packed: tiles must be 16-byte aligned");
    if ((reinterpret_cast<uintptr_t>(x) & 3u) || (reinterpret_cast<uintptr_t>(xsums) & 3u) || (reinterpret_cast<uintptr_t>(partials) & 3u))
        return fail(GUFFIN_E_ALIGN, "gemv_packed: fp32 pointers must be 4-byte aligned");
    const uint32_t S = packed_plan(dtype, K / block_elems(dtype), N / kTileCols).sp.planes;
    const uint8_t* w = static_cast<const uint8_t*>(tiles);
    hipStream_t s = as_stream(stream);
    float* out = (y && S == 1) ? y : partials;  // a single plane is the result: no second launch
    int rc;
    if (dtype == GUFFIN_Q4_K) rc = launch_packed<GUFFIN_Q4_K>(s, w, x, xsums, out, rows, K, N);
    else if (dtype == GUFFIN_Q6_K) rc = launch_packed<GUFFIN_Q6_K>(s, w, x, xsums, out, rows, K, N);
    else rc = launch_packed<GUFFIN_Q8_0>(s, w, x, xsums, out, rows, K, N);
    if (rc || !y || S == 1) return rc;
    const uint32_t count = rows * N;
    launch(reduce_partials_kernel, dim3((count + 255) / 256), dim3(256), 0, s, partials, y, S, count);
    return check_launch("reduce_partials");
}

extern "C" uint64_t guffin_hip_gemv_packed_static_limit(void) { return kStaticScratchFloats; }

extern "C" int guffin_hip_gemv_packed_static(void* stream, int dtype, const void* tiles, const float* x, const float* xsums,
                                             float* y, uint32_t rows, uint32_t K, uint32_t N) {
    if (!tiles || !x || !xsums || !y) return fail(GUFFIN_E_ARG, "gemv_packed_static: null pointer");
    if (int rc = check_packed_shape("gemv_packed_static: need K % block == 0 and N % 64 == 0", dtype, K, N)) return rc;
    if (rows == 0 || rows > 2) return fail(GUFFIN_E_SHAPE, "gemv_packed_static: rows must be 1 or 2");
    const uint32_t S = packed_plan(dtype, K / block_elems(dtype), N / kTileCols).sp.planes;
    if (S > 1 && uint64_t(S) * rows * N > kStaticScratchFloats)
        return fail(GUFFIN_E_CAPACITY, "gemv_packed_static: planes * rows * N exceeds the static scratch of 32768 floats");
    int device = -1;
    if (hipGetDevice(&device) != hipSuccess || device < 0 || device >= kMaxDevices || !g_scratch_ptr[device])
        return fail(GUFFIN_E_STATE, "gemv_packed_static: guffin_hip_init has not run for the current device");
    // the kernels write every plane element they later read, so nothing needs clearing between calls
    return guffin_hip_gemv_packed(stream, dtype, tiles, x, xsums, g_scratch_ptr[device], y, rows, K, N);
}
