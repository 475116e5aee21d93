// The block graph of a decode / verify pass as one launch per group of blocks whose workgroups stay
// resident on the chip: one workgroup per CU, the 32 workgroups of an XCD (one L2) own one KV head.
//
// Operator order and arithmetic per block are those of encode_gemma_target_blocks
// (src/engine/gemma_target_runtime.cpp:13-221) and of the drafter's forward
// (src/engine/gemma3_draft.mm:888-972), as in the launch-per-operator path of plan.hip; what changes
// is where a block's data moves.  The work is cut the way a tensor-parallel deployment cuts it, with
// an XCD in the place of a GPU:
//   q/k/v columns of KV head h, attention of head h, o-projection over head h's slice of K  -> XCD h
//   gate/up columns and the down projection over the same slice of the FFN width             -> XCD h
// so that everything between two projections stays inside one L2 and only the two reductions of a
// block (after the o-projection and after the down projection) cross XCDs.  Inside an XCD workgroups
// hand data over through that L2: plain stores, a counter in the L2 (atomics execute there), and reads of
// addresses this CU has not read before in the launch (a set of exchange buffers per block, so that no line
// of the L1 can be stale).  Across XCDs the partial planes are written through (sc1 stores)
// and read with sc1 loads after a two-level barrier (XCD counter, then one device counter).
// A model with one KV head (the drafter) runs on the 32 CUs of XCD 0; the others leave at once.
//
// Every wait is bounded: a workgroup that gives up raises GUFFIN_STATUS_SYNC, stops waiting for the
// rest of the launch and still runs to the end, so the grid always drains.  Placement (workgroup i
// on XCD i % 8, one workgroup per CU) is what the hardware's dispatcher does for a 256-workgroup
// launch on an idle device; each workgroup reads its XCD from the hardware register, and a launch
// whose XCDs do not each receive 32 workgroups ends in that same bounded give-up.
#include "common.hpp"
#include "receipt.hpp"
#include "gemv_tiles.hpp"

#include <algorithm>
#include <cstring>

namespace guffin {
namespace {

constexpr uint32_t kGroups = 32;        // workgroups per XCD
constexpr uint32_t kWaves = 8;          // waves per workgroup: two per SIMD, 256 registers each
constexpr uint32_t kThreads = 512;
constexpr uint32_t kGrid = 256;
constexpr uint32_t kRowThreads = 256;   // threads that hold one row of the residual stream (two runs of 8 columns each)
constexpr uint32_t kRowItems = 2;       // runs of 8 columns per thread: run i of thread t covers columns 8 * (t + 256 i) ..
constexpr uint32_t kHd = 256;
constexpr uint32_t kSyncWords = 64 * (2 * 8 + 2);   // per launch: 8 counter lines, 8 flag lines, device counter, spare

struct RLayer {
    const uint8_t* tiles[7];     // q k v o gate up down (wave tiles)
    const float* norm[6];        // attn_norm (unused here), q_norm, k_norm, post_attention_norm, ffn_norm, post_ffw_norm
    const float* gamma_next;     // the norm that follows this block's second residual add
    const uint16_t* ring_k; const uint16_t* ring_v;
    const float2* rope;          // [rows][128] (cos, sin)
    const uint32_t* schedule;    // [rows][4]
    uint16_t* priv_k; uint16_t* priv_v;   // this block's private rows [rows][kv_heads * 256]
    uint32_t ring_mask, dtype_bits;       // dtype of matrix m in bits 4m .. 4m+3
};

struct RArgs {
    RLayer layer[kResidentLayers];
    uint32_t layers, H, F, kv_heads;
    float eps, scale;
    float* qkv_part;     // [X][PA][R][(G+2)*256]
    float* attn_out;     // [X][32][NQ][256]
    float* attn_ml;      // [X][32][NQ][2]
    float* o_planes;     // [X*kparts_o][R][H]
    float* d_planes;     // [X*kparts_d][R][H]
    float* vec;          // [X][R][H]
    void* h_receipt;     // receipt of the FFN activation, layout (R, F)
    uint32_t* sync;      // this launch's kSyncWords words, zero at launch
    const float* x_in; const void* u_receipt_in;
    float* x_out; float* u_out; void* u_receipt_out;   // written by one workgroup after the last block
    const uint32_t* ancestors;
    uint32_t* status;
    uint32_t spin_limit, opnd_bytes;
    uint32_t set_floats, vec_floats;   // floats between the exchange buffers of consecutive blocks; floats of one `vec`
    unsigned long long* stamps;   // profiling aid: 8 clock readings per block from workgroup 0, or null
};

__device__ __forceinline__ uint32_t xcc_id() {
    uint32_t v;
    asm volatile("s_getreg_b32 %0, hwreg(HW_REG_XCC_ID)" : "=s"(v));
    return v & 0xFu;
}

// ---- loads of data another workgroup wrote during this launch ----------------------------------
// Plain vector loads: every call site indexes by thread, so none is served by the scalar cache, and the
// barrier before them ends in an asm statement that clobbers memory, so none moves above it.  (A volatile
// load would be a system-scope access that the compiler waits for one by one.)
typedef float f4_t __attribute__((ext_vector_type(4)));
__device__ __forceinline__ float xld(const float* p) { return *p; }
__device__ __forceinline__ f4_t xld4(const float* p) { return *reinterpret_cast<const f4_t*>(p); }
__device__ __forceinline__ uint4_t xld16(const void* p) { return *reinterpret_cast<const uint4_t*>(p); }
__device__ __forceinline__ float ld_dev(const float* p) { return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
__device__ __forceinline__ void st_dev(float* p, float v) { __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
__device__ __forceinline__ uint32_t ld_dev(const uint32_t* p) { return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }

struct Shared {
    float red[kWaves * 2 * 64];      // per-wave column sums of a projection
    float vals[2 * 64];
    float rowsum[kWaves];
    float q_s[8 * kHd];              // prepared queries [NQ][256]
    uint16_t k_s[2][kHd], v_s[2][kHd];
    float s_max[8], s_sum[8], wgt[8 * kGroups], den[8];
    uint32_t dead, xcd, slot;
};

struct Ctx {
    Shared* sh;
    uint8_t* dyn;         // dynamic LDS: operand receipt, or attention scratch
    uint32_t x, slot;     // XCD (= KV head) and workgroup slot inside it
    uint32_t lgen, ggen;  // barrier generations
    uint32_t X;
    const RArgs* a;
    uint32_t tid;         // the thread index
    // this block's exchange buffers
    float *qkv_part, *attn_out, *attn_ml, *o_planes, *d_planes, *vec;
    uint8_t* h_receipt;
};

// clock reading `phase` of block `layer` (first workgroup of XCD 0 only; 100 MHz constant clock)
__device__ __forceinline__ void stamp(const Ctx& c, uint32_t layer, uint32_t phase) {
    if (c.a->stamps && c.x == 0 && c.slot == 0 && c.tid == 0) c.a->stamps[layer * 16 + phase] = wall_clock64();
}

__device__ __forceinline__ void give_up(Ctx& c) {
    c.sh->dead = 1u;
    atomicOr(c.a->status, GUFFIN_STATUS_SYNC);
}

// Barrier of the 32 workgroups of this XCD.  Stores issued before it are in the L2 when it opens
// (the wait for the memory counters precedes the arrival).  Nothing invalidates this CU's L1 here: a
// device-scope invalidate also sweeps the XCD's L2 (14 us per barrier, measured), and one of workgroup scope
// does nothing for data from other CUs.  Instead no address of the exchange buffers is read twice during a
// launch -- every block of a launch has its own set of them (RArgs::set_floats), the two norm joints of a block
// their own slice buffers -- so a line in the L1 is never older than the data it stands for; the L1 starts
// every launch empty.  (With one set for all blocks a small model, whose weight stream does not sweep the L1
// between blocks, read rows of the block before: the reference's six-block fixture caught that.)
// drained: the caller has already waited for its stores (and then asked for data it does not need before
// the barrier opens: such loads stay in flight across the wait).
__device__ __forceinline__ void xcd_barrier(Ctx& c, bool drained = false) {
    if (!drained) __builtin_amdgcn_s_waitcnt(0);
    __syncthreads();
    c.lgen += 1;
    if (c.tid == 0 && !c.sh->dead) {
        uint32_t* ctr = c.a->sync + 64 * c.x;
        __hip_atomic_fetch_add(ctr, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
        const uint32_t target = kGroups * c.lgen;
        uint32_t spins = 0;
        while (ld_dev(ctr) < target) {
            if (++spins > c.a->spin_limit) { give_up(c); break; }
        }
    }
    __syncthreads();
    asm volatile("" ::: "memory");
}

// Barrier of all participating workgroups: arrival at the XCD's counter, the last arrival of an XCD
// joins the device counter and waits for every XCD, then releases its own XCD through a flag.
__device__ __forceinline__ void device_barrier(Ctx& c, bool drained = false) {
    if (!drained) __builtin_amdgcn_s_waitcnt(0);
    __syncthreads();
    c.lgen += 1;
    c.ggen += 1;
    if (c.tid == 0 && !c.sh->dead) {
        uint32_t* ctr = c.a->sync + 64 * c.x;
        uint32_t* flag = c.a->sync + 64 * (8 + c.x);
        uint32_t* gctr = c.a->sync + 64 * 16;
        uint32_t spins = 0;
        const uint32_t prev = __hip_atomic_fetch_add(ctr, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
        if (prev + 1 == kGroups * c.lgen) {
            __hip_atomic_fetch_add(gctr, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            const uint32_t target = c.X * c.ggen;
            bool ok = true;
            while (ld_dev(gctr) < target) {
                if (++spins > c.a->spin_limit) { ok = false; break; }
            }
            if (!ok) give_up(c);
            // the flag opens the XCD in either case: its workgroups then go on (a give-up is in the status word)
            __hip_atomic_fetch_max(flag, c.ggen, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
        } else {
            while (ld_dev(flag) < c.ggen) {
                if (++spins > c.a->spin_limit) { give_up(c); break; }
            }
        }
    }
    __syncthreads();
    asm volatile("" ::: "memory");
}

// sum over one row's threads (waves 8r .. 8r+7), the same order for every row index
__device__ __forceinline__ float row_sum(Ctx& c, float v) {
    v = wave_sum(v);
    const uint32_t lane = c.tid & 63, wv = __builtin_amdgcn_readfirstlane(c.tid >> 6);
    __syncthreads();
    if (lane == 0) c.sh->rowsum[wv] = v;
    __syncthreads();
    const uint32_t base = (c.tid / kRowThreads) * (kRowThreads / 64);
    float t = 0.f;
#pragma unroll
    for (uint32_t i = 0; i < kRowThreads / 64; ++i) t += c.sh->rowsum[base + i];
    return t;
}

__device__ __forceinline__ uint32_t dtype_of(const RLayer& L, int m) { return (L.dtype_bits >> (4 * m)) & 15u; }
__device__ __forceinline__ uint32_t tile_bytes(uint32_t dtype) { return kTileCols * block_bytes(static_cast<int>(dtype)); }

// One wave's run of blocks against the operand receipt at the start of the dynamic LDS.
// KQ: 256-element formats (Q4_K or Q6_K by the matrix's dtype), else Q8_0.
template <bool KQ, int R, bool AHEAD = false>
__device__ __forceinline__ void wave_blocks(const Ctx& c, uint32_t dtype, const uint8_t* tiles, uint32_t K, uint32_t ob0,
                                            uint32_t count, float (&acc)[R], const Q8Ahead& ahead = Q8Ahead{}) {
    const uint32_t lane = c.tid & 63;
    extern __shared__ __attribute__((aligned(256))) uint8_t dyn[];
    const float* opnd = reinterpret_cast<const float*>(dyn);
    if constexpr (!KQ && AHEAD) {
        run_blocks_ahead<R>(ahead, tiles, opnd, K, ob0, count, acc, lane);
        return;
    }
    if constexpr (KQ) {
        if (dtype == GUFFIN_Q4_K) {
            run_blocks_at<GUFFIN_Q4_K, R>(tiles, opnd, K, ob0, count, acc, lane);
        } else {
            run_blocks_at<GUFFIN_Q6_K, R, true>(tiles, opnd, K, ob0, count, acc, lane);
        }
    } else {
        run_blocks_at<GUFFIN_Q8_0, R>(tiles, opnd, K, ob0, count, acc, lane);
    }
}

// Copies the part [k0, k0 + count) of a receipt laid out for (R, K) in global memory into a receipt laid
// out for (R, count) in LDS.  k0 and count are multiples of 32.
template <int R>
__device__ __forceinline__ void copy_receipt(const Ctx& c, const void* src, uint32_t K, uint32_t k0, uint32_t count, uint8_t* dst) {
    const ReceiptLayout LS = receipt_layout(R, K), LD = receipt_layout(R, count);
    const uint8_t* s8 = static_cast<const uint8_t*>(src);
    const float* ssum = static_cast<const float*>(src);
    const float* smul = reinterpret_cast<const float*>(s8 + LS.mult_off);
    float* dsum = reinterpret_cast<float*>(dst);
    float* dmul = reinterpret_cast<float*>(dst + LD.mult_off);
    const uint32_t n16 = count / 16, n32 = count / 32, per_s = K / 16 + K / 32, per_d = n16 + n32;
    for (uint32_t i = c.tid; i < uint32_t(R) * per_d; i += kThreads) {
        const uint32_t r = i / per_d, j = i % per_d;
        const float v = j < n16 ? xld(ssum + r * per_s + k0 / 16 + j) : xld(ssum + r * per_s + K / 16 + k0 / 32 + (j - n16));
        dsum[i] = v;
    }
    for (uint32_t i = c.tid; i < uint32_t(R) * n32; i += kThreads) {
        const uint32_t r = i / n32, j = i % n32;
        dmul[i] = xld(smul + r * (K / 32) + k0 / 32 + j);
    }
    const uint8_t* simg = s8 + LS.image_off + size_t(k0 / 32) * 256;
    uint8_t* dimg = dst + LD.image_off;
    for (uint32_t i = c.tid; i < n32 * 16; i += kThreads)
        *reinterpret_cast<uint4_t*>(dimg + i * 16) = xld16(simg + i * 16);
}

// How the projections whose K is cut across XCDs (o and down) are laid over an XCD's 32 workgroups:
// `kparts` parts of the XCD's K range, `groups` workgroups per part, each with `tpw` column tiles.
struct KSplit { uint32_t kparts, groups, tpw, bpp; };
__host__ __device__ inline KSplit ksplit_of(uint32_t tiles, uint32_t nbx) {
    uint32_t kparts = tiles >= kGroups ? 1u : kGroups / tiles;
    if (kparts > nbx) kparts = nbx;
    if (kparts < 1) kparts = 1;
    uint32_t groups = kGroups / kparts;
    if (groups > tiles) groups = tiles;
    uint32_t tpw = (tiles + groups - 1) / groups;
    // a workgroup's waves are dealt evenly to its tiles: a power of two, at most the wave count
    uint32_t p2 = 1;
    while (p2 < tpw) p2 <<= 1;
    return {kparts, groups, p2, (nbx + kparts - 1) / kparts};
}

// The slice of the FFN width an XCD owns, in column tiles of 64: whole down-projection blocks, dealt evenly.
struct FSlice { uint32_t tile0, tiles; };
__host__ __device__ inline FSlice fslice_of(uint32_t F, uint32_t block, uint32_t X, uint32_t x) {
    const uint32_t unit = block > 64 ? block / 64 : 1u;     // tiles per indivisible unit
    const uint32_t units = F / 64 / unit, base = units / X, rem = units % X;
    const uint32_t u0 = x * base + (x < rem ? x : rem), n = base + (x < rem ? 1u : 0u);
    return {u0 * unit, n * unit};
}

// This wave's run of blocks in a K-split projection: column tile, first block (relative to the part), count.
struct WaveRun { uint32_t tile, wb0, cnt; };
__device__ __forceinline__ WaveRun ksplit_wave(const Ctx& c, const KSplit ks, uint32_t tg, uint32_t ntiles, uint32_t nbp, bool active) {
    const uint32_t wave = __builtin_amdgcn_readfirstlane(c.tid >> 6);
    const uint32_t wpt = kWaves / ks.tpw;                 // waves per tile
    const uint32_t ti = wave / wpt, wl = wave % wpt;
    const uint32_t tile = tg + ti * ks.groups;
    const uint32_t bpw = (nbp + wpt - 1) / wpt;
    const uint32_t wb0 = min(wl * bpw, nbp);
    const uint32_t cnt = active && tile < ntiles ? min(bpw, nbp - wb0) : 0u;
    return {tile, wb0, cnt};
}

// The first tiles of this wave's run in a K-split projection, requested ahead of the wait before it.
__device__ __forceinline__ void ksplit_ahead(const Ctx& c, Q8Ahead& ahead, const uint8_t* tiles, uint32_t dtype, uint32_t ntiles,
                                             uint32_t nblk_total, uint32_t first_block, uint32_t nbp, const KSplit ks,
                                             uint32_t tg, bool active) {
    const WaveRun wr = ksplit_wave(c, ks, tg, ntiles, nbp, active);
    const uint8_t* tp = tiles + (size_t(wr.cnt ? wr.tile : 0u) * nblk_total + first_block + wr.wb0) * tile_bytes(dtype);
    load_ahead(ahead, tp, wr.cnt, c.tid & 63);
}

// Projection of the LDS operand (R rows of `count` inputs, blocks relative to the part) with the part's
// column tiles; partial plane `plane` of `out` ([planes][R][N]) receives the sums.
template <bool KQ, int R, bool AHEAD = false>
__device__ __forceinline__ void ksplit_project(Ctx& c, const uint8_t* tiles, uint32_t dtype, uint32_t ntiles,
                                               uint32_t nblk_total, uint32_t first_block, uint32_t nbp, uint32_t Kp,
                                               const KSplit ks, uint32_t tg, bool active, float* out, uint32_t plane,
                                               uint32_t N, const Q8Ahead& ahead = Q8Ahead{}) {
    const uint32_t wave = __builtin_amdgcn_readfirstlane(c.tid >> 6), lane = c.tid & 63;
    const uint32_t wpt = kWaves / ks.tpw;
    const WaveRun wr = ksplit_wave(c, ks, tg, ntiles, nbp, active);
    const uint32_t tile = wr.tile, wb0 = wr.wb0, cnt = wr.cnt;
    float acc[R];
    if (cnt > 0) {
        const uint8_t* tp = tiles + (size_t(tile) * nblk_total + first_block + wb0) * tile_bytes(dtype);
        wave_blocks<KQ, R, AHEAD>(c, dtype, tp, Kp, wb0, cnt, acc, ahead);
    } else {
#pragma unroll
        for (int r = 0; r < R; ++r) acc[r] = 0.f;
    }
#pragma unroll
    for (int r = 0; r < R; ++r) c.sh->red[(wave * R + r) * 64 + lane] = acc[r];
    __syncthreads();
    if (active) {
        for (uint32_t i = c.tid; i < ks.tpw * R * 64; i += kThreads) {
            const uint32_t t = i / (R * 64), r = (i / 64) % R, l = i % 64;
            const uint32_t tl = tg + t * ks.groups;
            if (tl >= ntiles) continue;
            float s = c.sh->red[((t * wpt) * R + r) * 64 + l];
            for (uint32_t w = 1; w < wpt; ++w) s += c.sh->red[((t * wpt + w) * R + r) * 64 + l];
            float* dst = out + (size_t(plane) * R + r) * N + tl * 64 + l;
            if (c.X > 1) st_dev(dst, s); else *dst = s;
        }
    }
    __syncthreads();
}

// out_residual = residual + rms(sum of planes, gamma_post); u = rms(out_residual, gamma_next) as the operand
// receipt in LDS.  Every workgroup does the whole vector; the residual lives in the threads' registers.
template <int R>
__device__ __forceinline__ void norm_pair(Ctx& c, const float* planes, uint32_t P, const float* gamma_post,
                                          const float* gamma_next, float (&xr)[kRowItems][8], bool last, bool drained,
                                          float* vec, uint32_t stamp_layer = 0, uint32_t stamp_base = 0) {
    const RArgs& a = *c.a;
    const uint32_t H = a.H, r = c.tid / kRowThreads, t0 = c.tid % kRowThreads;
    bool on[kRowItems];
    size_t col[kRowItems];
    // the norms' weights do not depend on this launch's data: requested before the wait
    f4_t gp4[kRowItems][2], gn4[kRowItems][2];
#pragma unroll
    for (uint32_t k = 0; k < kRowItems; ++k) {
        const uint32_t item = t0 + kRowThreads * k;
        on[k] = r < uint32_t(R) && item < H / 8;
        col[k] = on[k] ? item * 8u : 0u;
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            gp4[k][h] = on[k] ? *reinterpret_cast<const f4_t*>(gamma_post + col[k] + 4 * h) : f4_t{0, 0, 0, 0};
            gn4[k][h] = on[k] ? *reinterpret_cast<const f4_t*>(gamma_next + col[k] + 4 * h) : f4_t{0, 0, 0, 0};
        }
    }
    float v[kRowItems][8];
#pragma unroll
    for (uint32_t k = 0; k < kRowItems; ++k)
#pragma unroll
        for (int i = 0; i < 8; ++i) v[k][i] = 0.f;
    if (c.X > 1) {
        device_barrier(c, drained);
        if (stamp_base) stamp(c, stamp_layer, stamp_base);
        // this workgroup's slice of the columns: the planes of all XCDs summed in plane order
        const uint32_t cw = H / kGroups;
        if (c.tid < uint32_t(R) * cw) {
            const uint32_t rr = c.tid / cw, cc = c.slot * cw + c.tid % cw;
            // all planes requested before the first sum (batches of eight), summed in plane order
            float s = 0.f;
            for (uint32_t p0 = 0; p0 < P; p0 += 8) {
                float t[8];
#pragma unroll
                for (uint32_t i = 0; i < 8; ++i) t[i] = p0 + i < P ? ld_dev(planes + (size_t(p0 + i) * R + rr) * H + cc) : 0.f;
#pragma unroll
                for (uint32_t i = 0; i < 8; ++i) if (p0 + i < P) s = p0 + i == 0 ? t[i] : s + t[i];
            }
            vec[(size_t(c.x) * R + rr) * H + cc] = s;
        }
        if (stamp_base) stamp(c, stamp_layer, stamp_base + 1);
        xcd_barrier(c);
        if (stamp_base) stamp(c, stamp_layer, stamp_base + 2);
#pragma unroll
        for (uint32_t k = 0; k < kRowItems; ++k) {
            if (on[k]) {
                const float* src = vec + (size_t(c.x) * R + r) * H + col[k];
                const f4_t lo = xld4(src), hi = xld4(src + 4);
                v[k][0] = lo.x; v[k][1] = lo.y; v[k][2] = lo.z; v[k][3] = lo.w;
                v[k][4] = hi.x; v[k][5] = hi.y; v[k][6] = hi.z; v[k][7] = hi.w;
            }
        }
    } else {
        xcd_barrier(c, drained);
#pragma unroll
        for (uint32_t k = 0; k < kRowItems; ++k) {
            if (on[k]) {
                for (uint32_t p = 0; p < P; ++p) {
                    const float* src = planes + (size_t(p) * R + r) * H + col[k];
                    const f4_t lo = xld4(src), hi = xld4(src + 4);
                    v[k][0] += lo.x; v[k][1] += lo.y; v[k][2] += lo.z; v[k][3] += lo.w;
                    v[k][4] += hi.x; v[k][5] += hi.y; v[k][6] += hi.z; v[k][7] += hi.w;
                }
            }
        }
    }
    float ss = 0.f;
#pragma unroll
    for (uint32_t k = 0; k < kRowItems; ++k)
#pragma unroll
        for (int i = 0; i < 8; ++i) ss = fmaf(v[k][i], v[k][i], ss);
    float total = row_sum(c, ss);
    if (stamp_base) stamp(c, stamp_layer, stamp_base + 3);
    float inv = 1.0f / sqrtf(total / static_cast<float>(H) + a.eps);
    bool bad = false;
    ss = 0.f;
#pragma unroll
    for (uint32_t k = 0; k < kRowItems; ++k) {
        const float gp[8] = {gp4[k][0].x, gp4[k][0].y, gp4[k][0].z, gp4[k][0].w, gp4[k][1].x, gp4[k][1].y, gp4[k][1].z, gp4[k][1].w};
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const float t = on[k] ? v[k][i] * inv * gp[i] + xr[k][i] : 0.f;
            bad |= !isfinite(t);
            xr[k][i] = t;
            ss = fmaf(t, t, ss);
        }
    }
    total = row_sum(c, ss);
    inv = 1.0f / sqrtf(total / static_cast<float>(H) + a.eps);
    const bool writer = last && c.x == 0 && c.slot == 0;
#pragma unroll
    for (uint32_t k = 0; k < kRowItems; ++k) {
        const float gn[8] = {gn4[k][0].x, gn4[k][0].y, gn4[k][0].z, gn4[k][0].w, gn4[k][1].x, gn4[k][1].y, gn4[k][1].z, gn4[k][1].w};
        float y[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) y[i] = xr[k][i] * inv * gn[i];
        const uint32_t item = t0 + kRowThreads * k;
        if (on[k]) emit_receipt_values(y, 0, item, r, R, H, c.dyn);
        if (writer && on[k]) {
            // the pass's output, or the state the next launch starts from
            float* xo = a.x_out + size_t(r) * H + col[k];
            float* uo = a.u_out + size_t(r) * H + col[k];
            *reinterpret_cast<f4_t*>(xo) = f4_t{xr[k][0], xr[k][1], xr[k][2], xr[k][3]};
            *reinterpret_cast<f4_t*>(xo + 4) = f4_t{xr[k][4], xr[k][5], xr[k][6], xr[k][7]};
            *reinterpret_cast<f4_t*>(uo) = f4_t{y[0], y[1], y[2], y[3]};
            *reinterpret_cast<f4_t*>(uo + 4) = f4_t{y[4], y[5], y[6], y[7]};
            if (a.u_receipt_out) emit_receipt_values(y, 0, item, r, R, H, a.u_receipt_out);
        }
    }
    if (bad) atomicOr(a.status, GUFFIN_STATUS_NONFINITE);
    __syncthreads();   // the operand is complete
}

// ---- attention of this XCD's KV head over partition `slot` of the token list ---------------------
// The merged token list of a block's rows (union of the rows' ring ranges, then the private rows) and this
// workgroup's part of it.
struct TokenList { uint32_t u_first, n_ring, n_total, tp, t0, t1; };
template <int R>
__device__ __forceinline__ TokenList token_list(const RLayer& L, uint32_t slot) {
    uint32_t u_first = 0xFFFFFFFFu, u_end = 0;
#pragma unroll
    for (int r = 0; r < R; ++r) {
        const uint32_t* s = L.schedule + 4 * r;
        if (s[1]) { u_first = min(u_first, s[0]); u_end = max(u_end, s[0] + s[1]); }
    }
    if (u_end == 0) u_first = 0;
    TokenList t;
    t.u_first = u_first; t.n_ring = u_end - u_first; t.n_total = t.n_ring + R;
    t.tp = (t.n_total + kGroups - 1) / kGroups;
    t.t0 = min(slot * t.tp, t.n_total); t.t1 = min(t.t0 + t.tp, t.n_total);
    return t;
}

struct HeadVals { float v[4]; float gm[4]; float2 rp[2]; };

template <int R, int G>
__device__ __forceinline__ void attention_partition(Ctx& c, const RLayer& L, uint32_t PA) {
    constexpr int NQ = R * G;
    constexpr uint32_t CW = (G + 2) * kHd;
    const RArgs& a = *c.a;
    Shared& sh = *c.sh;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(c.tid >> 6), lane = c.tid & 63;
    const uint32_t row_stride = a.kv_heads * kHd;   // halves between ring rows
    const float* part = c.qkv_part + size_t(c.x) * PA * R * CW;   // [PA][R][CW]
    const size_t pstride = size_t(R) * CW;

    // token list: union of the rows' ring ranges, then the private rows
    uint32_t bfirst[R], bend[R], amask[R];
#pragma unroll
    for (int r = 0; r < R; ++r) {
        const uint32_t* s = L.schedule + 4 * r;
        bfirst[r] = s[0]; bend[r] = s[0] + s[1]; amask[r] = 0;
        for (uint32_t i = 0; i < s[3]; ++i) amask[r] |= 1u << a.ancestors[s[2] + i];
    }
    const TokenList tl = token_list<R>(L, c.slot);
    const uint32_t u_first = tl.u_first, n_ring = tl.n_ring, tp = tl.tp, t0 = tl.t0, t1 = tl.t1;

    const uint32_t half = lane >> 5, l32 = lane & 31;            // token slot of the wave's round, 8-dim segment
    constexpr int U = 4;                                         // rounds of loads in flight
    // ring rows of this wave's first rounds: their addresses need the schedule only, so the keys travel while
    // the queries are prepared and the values while the softmax runs (private rows come from LDS at use)
    const uint32_t tb_first = t0 + wave * 2 + half;
    auto load_ring = [&](const uint16_t* ring, uint32_t tb, uint4 (&dst)[U]) {
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const uint32_t t = tb + 2 * kWaves * u;
            dst[u] = make_uint4(0, 0, 0, 0);
            if (t < t1 && t < n_ring)
                dst[u] = *reinterpret_cast<const uint4*>(ring + size_t((u_first + t) & L.ring_mask) * row_stride + c.x * kHd + l32 * 8);
        }
    };
    uint4 kk[U], vv[U];
    load_ring(L.ring_k, tb_first, kk);

    // item n < NQ is query row n; items NQ .. NQ + 2R - 1 are the private rows' key and value, prepared when
    // this partition holds them (head norm, rotation, fp16 rounding after rotation); a wave takes items
    // wave, wave + 8, ..
    for (uint32_t it = wave; it < uint32_t(NQ + 2 * R); it += kWaves) {
        const bool is_q = it < uint32_t(NQ);
        const uint32_t i = it - NQ, pr = i >> 1;
        const bool is_key = (i & 1u) == 0;
        const bool mine_kv = !is_q && n_ring + pr >= t0 && n_ring + pr < t1;
        if (is_q || mine_kv) {
            const uint32_t r = is_q ? it / G : pr;
            const uint32_t colbase = is_q ? (it % G) * kHd : (is_key ? G * kHd : (G + 1) * kHd);
            const float* gamma = is_q ? L.norm[1] : (is_key ? L.norm[2] : nullptr);
            const bool rotate = is_q || is_key;
            HeadVals h;
#pragma unroll
            for (int k = 0; k < 4; ++k) h.gm[k] = gamma ? gamma[lane + 64 * k] : 1.f;
            h.rp[0] = rotate ? L.rope[size_t(r) * (kHd / 2) + lane] : make_float2(1.f, 0.f);
            h.rp[1] = rotate ? L.rope[size_t(r) * (kHd / 2) + lane + 64] : make_float2(1.f, 0.f);
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const float* src = part + size_t(r) * CW + colbase + lane + 64 * k;
                float s = xld(src);
                for (uint32_t p = 1; p < PA; ++p) s += xld(src + p * pstride);
                h.v[k] = s;
            }
            if (gamma) {
                float ss = 0.f;
#pragma unroll
                for (int k = 0; k < 4; ++k) ss = fmaf(h.v[k], h.v[k], ss);
                ss = wave_sum(ss);
                const float inv = 1.0f / sqrtf(ss / 256.0f + a.eps);
#pragma unroll
                for (int k = 0; k < 4; ++k) h.v[k] = h.v[k] * inv * h.gm[k];
            }
            if (rotate) {
#pragma unroll
                for (int k = 0; k < 2; ++k) {
                    const float first = h.v[k], second = h.v[k + 2];
                    h.v[k] = __fsub_rn(__fmul_rn(first, h.rp[k].x), __fmul_rn(second, h.rp[k].y));
                    h.v[k + 2] = __fadd_rn(__fmul_rn(first, h.rp[k].y), __fmul_rn(second, h.rp[k].x));
                }
            }
            if (is_q) {
#pragma unroll
                for (int k = 0; k < 4; ++k) sh.q_s[it * kHd + lane + 64 * k] = h.v[k] * a.scale;
            } else {
                bool bad = false;
                const size_t kv_off = (size_t(pr) * a.kv_heads + c.x) * kHd;
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    const _Float16 hv = static_cast<_Float16>(h.v[k]);
                    bad |= !isfinite(static_cast<float>(hv));
                    const uint16_t bits = __builtin_bit_cast(uint16_t, hv);
                    (is_key ? sh.k_s : sh.v_s)[pr][lane + 64 * k] = bits;
                    (is_key ? L.priv_k : L.priv_v)[kv_off + lane + 64 * k] = bits;
                }
                if (bad) atomicOr(a.status, GUFFIN_STATUS_KV_NONFINITE);
            }
        }
    }
    __syncthreads();

    float* sc = reinterpret_cast<float*>(c.dyn);                 // [NQ][tp] scores, then probabilities
    float* merge = sc + ((size_t(NQ) * tp + 63) & ~size_t{63});  // [waves][NQ][256]
    // ---- scores: a half wave per token, 8 dims per lane -----------------------------------------
    {
        float qv[NQ][8];
#pragma unroll
        for (int n = 0; n < NQ; ++n)
#pragma unroll
            for (int i = 0; i < 8; ++i) qv[n][i] = sh.q_s[n * kHd + l32 * 8 + i];
        for (uint32_t tb = tb_first; tb < t1; tb += 2 * kWaves * U) {
            if (tb != tb_first) load_ring(L.ring_k, tb, kk);
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const uint32_t t = tb + 2 * kWaves * u;
                if (t < t1 && t >= n_ring) kk[u] = *reinterpret_cast<const uint4*>(&sh.k_s[t - n_ring][l32 * 8]);
            }
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const uint32_t t = tb + 2 * kWaves * u;
                if (t >= t1) break;
                const uint32_t kw[4] = {kk[u].x, kk[u].y, kk[u].z, kk[u].w};
                float s[NQ];
#pragma unroll
                for (int n = 0; n < NQ; ++n) {
                    s[n] = 0.f;
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        const half2_t h2 = __builtin_bit_cast(half2_t, kw[i]);
                        s[n] = fmaf(static_cast<float>(h2.x), qv[n][2 * i], s[n]);
                        s[n] = fmaf(static_cast<float>(h2.y), qv[n][2 * i + 1], s[n]);
                    }
                    s[n] = row16_sum(s[n]);
                    s[n] += __shfl_xor(s[n], 16, kWave);
                }
                if (l32 == 0) {
                    const bool is_priv = t >= n_ring;
                    const uint32_t pos = u_first + t, prow = t - n_ring;
#pragma unroll
                    for (int n = 0; n < NQ; ++n) {
                        const uint32_t r = n / G;
                        const bool valid = is_priv ? ((amask[r] >> prow) & 1u) != 0 : (pos >= bfirst[r] && pos < bend[r]);
                        sc[n * tp + (t - t0)] = valid ? s[n] : -INFINITY;
                    }
                }
            }
        }
    }
    load_ring(L.ring_v, tb_first, vv);
    __syncthreads();
    // ---- softmax over the partition, one wave per query ------------------------------------------
    const uint32_t np = t1 - t0;
    for (uint32_t n = wave; n < uint32_t(NQ); n += kWaves) {
        float m = -INFINITY;
        for (uint32_t i = lane; i < np; i += 64) m = fmaxf(m, sc[n * tp + i]);
        m = wave_max(m);
        float l = 0.f;
        for (uint32_t i = lane; i < np; i += 64) {
            const float v = sc[n * tp + i];
            const float p = v == -INFINITY ? 0.f : expf(v - m);
            sc[n * tp + i] = p;
            l += p;
        }
        l = wave_sum(l);
        if (lane == 0) { sh.s_max[n] = m; sh.s_sum[n] = l; }
    }
    __syncthreads();
    // ---- values: the same lane layout; halves by a lane exchange, waves through LDS ----------------
    {
        float acc[NQ][8];
#pragma unroll
        for (int n = 0; n < NQ; ++n)
#pragma unroll
            for (int i = 0; i < 8; ++i) acc[n][i] = 0.f;
        for (uint32_t tb = tb_first; tb < t1; tb += 2 * kWaves * U) {
            if (tb != tb_first) load_ring(L.ring_v, tb, vv);
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const uint32_t t = tb + 2 * kWaves * u;
                if (t < t1 && t >= n_ring) vv[u] = *reinterpret_cast<const uint4*>(&sh.v_s[t - n_ring][l32 * 8]);
            }
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const uint32_t t = tb + 2 * kWaves * u;
                if (t >= t1) break;
                const uint32_t w4[4] = {vv[u].x, vv[u].y, vv[u].z, vv[u].w};
#pragma unroll
                for (int n = 0; n < NQ; ++n) {
                    const float p = sc[n * tp + (t - t0)];
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        const half2_t h2 = __builtin_bit_cast(half2_t, w4[i]);
                        acc[n][2 * i] = fmaf(static_cast<float>(h2.x), p, acc[n][2 * i]);
                        acc[n][2 * i + 1] = fmaf(static_cast<float>(h2.y), p, acc[n][2 * i + 1]);
                    }
                }
            }
        }
#pragma unroll
        for (int n = 0; n < NQ; ++n) {
#pragma unroll
            for (int i = 0; i < 8; ++i) acc[n][i] += __shfl_xor(acc[n][i], 32, kWave);
            if (half == 0) {
                float* mp = merge + (size_t(wave) * NQ + n) * kHd + l32 * 8;
                *reinterpret_cast<f4_t*>(mp) = f4_t{acc[n][0], acc[n][1], acc[n][2], acc[n][3]};
                *reinterpret_cast<f4_t*>(mp + 4) = f4_t{acc[n][4], acc[n][5], acc[n][6], acc[n][7]};
            }
        }
    }
    __syncthreads();
    // waves that had no token hold zeros: every wave's slot is summed, in wave order
    float* po = c.attn_out + (size_t(c.x) * kGroups + c.slot) * NQ * kHd;
    float* pml = c.attn_ml + (size_t(c.x) * kGroups + c.slot) * NQ * 2;
    for (uint32_t i = c.tid; i < uint32_t(NQ) * kHd; i += kThreads) {
        const uint32_t n = i / kHd, d = i % kHd;
        float v = merge[(0 * NQ + n) * kHd + d];
#pragma unroll
        for (uint32_t w = 1; w < kWaves; ++w) v += merge[(size_t(w) * NQ + n) * kHd + d];
        po[i] = v;
        if (d == 0) { pml[2 * n] = sh.s_max[n]; pml[2 * n + 1] = sh.s_sum[n]; }
    }
}

// Merges the partitions' results for the elements [e0, e0 + count) of this XCD's attention output
// (element = head-in-group * 256 + dim) into LDS values and their operand receipt.
template <int R, int G>
__device__ __forceinline__ void merge_attention(Ctx& c, uint32_t e0, uint32_t count, float* vals) {
    constexpr int NQ = R * G;
    const RArgs& a = *c.a;
    Shared& sh = *c.sh;
    const float* pml = c.attn_ml + size_t(c.x) * kGroups * NQ * 2;
    const float* po = c.attn_out + size_t(c.x) * kGroups * NQ * kHd;
    // weights of the 32 partitions per query: half a wave per query.  The two reductions stay xor butterflies
    // (not the quad-and-mirror tree of row16_sum): a row's tokens sit one partition further along as the second
    // row of a two-row pass than when the row is decoded alone, and the butterfly's pairing keeps the sum's bits
    // under that shift where the tree does not (the width-two verify pass must reproduce the one-row bits).
    if (c.tid < uint32_t(NQ) * kGroups) {
        const uint32_t n = c.tid / kGroups, p = c.tid % kGroups;
        const float m = xld(pml + (size_t(p) * NQ + n) * 2), l = xld(pml + (size_t(p) * NQ + n) * 2 + 1);
        float M = l > 0.f ? m : -INFINITY;
#pragma unroll
        for (int s = 16; s > 0; s >>= 1) M = fmaxf(M, __shfl_xor(M, s, kWave));
        const float w = l > 0.f ? expf(m - M) : 0.f;
        float dn = w * l;
#pragma unroll
        for (int s = 16; s > 0; s >>= 1) dn += __shfl_xor(dn, s, kWave);
        sh.wgt[n * kGroups + p] = w;
        if (p == 0) sh.den[n] = dn;
    }
    __syncthreads();
    bool bad = false;
    for (uint32_t i = c.tid; i < uint32_t(R) * count; i += kThreads) {
        const uint32_t r = i / count, e = e0 + i % count;
        const uint32_t n = r * G + e / kHd, d = e % kHd;
        float pv[kGroups];
#pragma unroll
        for (uint32_t p = 0; p < kGroups; ++p) pv[p] = xld(po + (size_t(p) * NQ + n) * kHd + d);
        float acc = 0.f;
#pragma unroll
        for (uint32_t p = 0; p < kGroups; ++p) acc = fmaf(sh.wgt[n * kGroups + p], pv[p], acc);
        const float v = acc / sh.den[n];
        bad |= !isfinite(v);
        vals[i] = v;
    }
    if (bad) atomicOr(a.status, GUFFIN_STATUS_NONFINITE);
    __syncthreads();
}

template <int R, int G, bool KQ>
__global__ void __launch_bounds__(kThreads) resident_blocks_kernel(const RArgs a) {
    extern __shared__ __attribute__((aligned(256))) uint8_t dyn[];
    __shared__ Shared sh;
    constexpr uint32_t BE = KQ ? 256u : 32u;
    constexpr uint32_t CW = (G + 2) * kHd;
    if (threadIdx.x == 0) {
        sh.dead = 0;
        sh.xcd = xcc_id();
        // the slot inside the XCD: the dispatcher deals workgroups to XCDs in turn
        sh.slot = blockIdx.x / 8;
    }
    __syncthreads();
    Ctx c {&sh, dyn, sh.xcd, sh.slot, 0, 0, a.kv_heads, &a, threadIdx.x, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr};
    if (c.x >= c.X) return;            // a model with fewer KV heads than XCDs leaves the others idle
    if (c.slot >= kGroups) return;
    const uint32_t H = a.H, F = a.F, nbH = H / BE;

    // the state this launch starts from: the residual rows in registers, the normalised rows' receipt in LDS
    float xr[kRowItems][8];
    {
        const uint32_t r = threadIdx.x / kRowThreads;
#pragma unroll
        for (uint32_t k = 0; k < kRowItems; ++k) {
            const uint32_t item = threadIdx.x % kRowThreads + kRowThreads * k;
            const bool on = r < uint32_t(R) && item < H / 8;
#pragma unroll
            for (int i = 0; i < 8; ++i) xr[k][i] = on ? a.x_in[size_t(r) * H + item * 8 + i] : 0.f;
        }
        const uint32_t bytes = static_cast<uint32_t>(receipt_layout(R, H).bytes);
        const uint8_t* src = static_cast<const uint8_t*>(a.u_receipt_in);
        for (uint32_t i = threadIdx.x; i < bytes / 16; i += kThreads)
            *reinterpret_cast<uint4_t*>(dyn + i * 16) = *reinterpret_cast<const uint4_t*>(src + i * 16);
    }
    __syncthreads();

    // projections with all of K in one XCD (q/k/v): workgroups per column tile and their share of K
    constexpr uint32_t TA = 4 * G + 8;
    constexpr uint32_t PA = kGroups / TA >= 1 ? kGroups / TA : 1;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(c.tid >> 6), lane = c.tid & 63;

    // ---- this workgroup's share of every projection (the same for every block) --------------------
    // q/k/v: column tile qt (matrix qm, tile qct of it), blocks [qb0, qb0 + qcnt) of K
    const uint32_t qt = c.slot / PA, qkp = c.slot % PA;
    const bool q_active = qt < TA;
    const uint32_t qper = (nbH + PA - 1) / PA, qb0 = min(qkp * qper, nbH), qcnt = q_active ? min(qper, nbH - qb0) : 0u;
    const int qm = qt < 4 * G ? 0 : (qt < 4 * G + 4 ? 1 : 2);
    const uint32_t qct = qm == 0 ? c.x * 4 * G + qt : c.x * 4 + (qt - 4 * G - (qm == 2 ? 4 : 0));
    // o-projection: part okp of this KV head's slice of K, column tiles otg, otg + groups, ..
    const uint32_t o_nbx = G * kHd / BE;
    const KSplit oks = ksplit_of(H / 64, o_nbx);
    const uint32_t okp = c.slot / oks.groups, otg = c.slot % oks.groups;
    const bool o_active = okp < oks.kparts;
    const uint32_t opb0 = min(okp * oks.bpp, o_nbx), onbp = o_active ? min(oks.bpp, o_nbx - opb0) : 0u;
    const uint32_t o_nblk = (a.kv_heads * G * kHd) / BE, o_first = c.x * o_nbx + opb0;
    // gate / up: column tiles of this XCD's slice of the FFN width; down: the same slice as its K range
    const FSlice fs = fslice_of(F, BE, c.X, c.x);
    const uint32_t d_nbx = fs.tiles * 64 / BE;
    KSplit dks = ksplit_of(H / 64, fslice_of(F, BE, c.X, 0).tiles * 64 / BE);   // the widest slice's split: every XCD
    const uint32_t d_planes_per_xcd = dks.kparts;                               // writes the same number of planes
    dks.bpp = (d_nbx + dks.kparts - 1) / dks.kparts;
    const uint32_t dkp = c.slot / dks.groups, dtg = c.slot % dks.groups;
    const bool d_active = dkp < dks.kparts;
    const uint32_t dpb0 = min(dkp * dks.bpp, d_nbx), dnbp = d_active ? min(dks.bpp, d_nbx - dpb0) : 0u;
    const uint32_t d_nblk = F / BE, d_first = fs.tile0 * 64 / BE + dpb0;

    // A wave's runs of blocks in the four projections (the same for every block)
    const uint32_t q_bpw = (qcnt + kWaves - 1) / kWaves, q_wb0 = min(wave * q_bpw, qcnt), q_cnt = min(q_bpw, qcnt - q_wb0);
    constexpr uint32_t HW = kWaves / 2;   // waves per matrix in the gate / up phase
    const bool g_is_up = wave >= HW;
    const uint32_t g_bps = (nbH + HW - 1) / HW, g_wb0 = min((wave % HW) * g_bps, nbH);
    const uint32_t g_cnt = c.slot < fs.tiles ? min(g_bps, nbH - g_wb0) : 0u;
    auto q_tiles = [&](const RLayer& LL) { return LL.tiles[qm] + (size_t(qct) * nbH + qb0 + q_wb0) * tile_bytes(dtype_of(LL, qm)); };
    auto g_tiles = [&](const RLayer& LL, uint32_t ct) {
        const int m = g_is_up ? 5 : 4;
        return LL.tiles[m] + (size_t(ct) * nbH + g_wb0) * tile_bytes(dtype_of(LL, m));
    };

    // Q8_0 models: the first two tiles of a wave's next run of blocks are requested before the wait that
    // precedes the run (the weights do not depend on the pass) and held in registers across it, so that the
    // trip to memory overlaps the hand-over instead of following it.  The 256-element formats' tiles are
    // too large to hold across the norms.
    Q8Ahead ahead = {};
    if constexpr (!KQ) load_ahead(ahead, q_tiles(a.layer[0]), q_cnt, lane);

    for (uint32_t l = 0; l < a.layers; ++l) {
        const RLayer& L = a.layer[l];
        {
            const size_t at = size_t(l) * a.set_floats;
            c.qkv_part = a.qkv_part + at; c.attn_out = a.attn_out + at; c.attn_ml = a.attn_ml + at;
            c.o_planes = a.o_planes + at; c.d_planes = a.d_planes + at; c.vec = a.vec + at;
            c.h_receipt = static_cast<uint8_t*>(a.h_receipt) + at * 4;
        }
        stamp(c, l, 0);
        // ---- q, k, v columns of this XCD's KV head -------------------------------------------------
        {
            const uint32_t dtype = dtype_of(L, qm);
            float acc[R];
            if (q_cnt > 0) {
                wave_blocks<KQ, R, !KQ>(c, dtype, q_tiles(L), H, qb0 + q_wb0, q_cnt, acc, ahead);
            } else {
#pragma unroll
                for (int r = 0; r < R; ++r) acc[r] = 0.f;
            }
#pragma unroll
            for (int r = 0; r < R; ++r) sh.red[(wave * R + r) * 64 + lane] = acc[r];
            __syncthreads();
            if (q_active && c.tid < R * 64) {
                const uint32_t r = c.tid >> 6;
                float s = sh.red[r * 64 + lane];
                for (uint32_t w = 1; w < kWaves; ++w) s += sh.red[(w * R + r) * 64 + lane];
                c.qkv_part[((size_t(c.x) * PA + qkp) * R + r) * CW + qt * 64 + lane] = s;
            }
        }
        if constexpr (!KQ) {   // the o-projection's tiles travel while attention runs
            __builtin_amdgcn_s_waitcnt(0);
            ksplit_ahead(c, ahead, L.tiles[3], dtype_of(L, 3), H / 64, o_nblk, o_first, onbp, oks, otg, o_active);
            xcd_barrier(c, true);
        } else {
            xcd_barrier(c);
        }
        stamp(c, l, 1);
        // ---- attention over this workgroup's partition of the tokens ------------------------------
        attention_partition<R, G>(c, L, PA);
        xcd_barrier(c);
        stamp(c, l, 2);
        // ---- merge of the partitions, o-projection over this KV head's slice of K ---------------------
        {
            const uint32_t Kp = max(onbp, 1u) * BE;
            float* vals = reinterpret_cast<float*>(dyn + a.opnd_bytes);   // [R][Kp], behind the operand
            if (o_active) {
                merge_attention<R, G>(c, opb0 * BE, onbp * BE, vals);
#pragma unroll
                for (int r = 0; r < R; ++r) emit_receipt(vals + size_t(r) * onbp * BE, 0, onbp * BE, r, R, Kp, dyn, c.tid, kThreads);
            }
            __syncthreads();
            ksplit_project<KQ, R, !KQ>(c, L.tiles[3], dtype_of(L, 3), H / 64, o_nblk, o_first, onbp, Kp, oks, otg, o_active,
                                       c.o_planes, c.x * oks.kparts + okp, H, ahead);
        }
        stamp(c, l, 3);
        if constexpr (!KQ) {   // this workgroup's first gate / up tiles
            __builtin_amdgcn_s_waitcnt(0);
            load_ahead(ahead, g_tiles(L, fs.tile0 + (c.slot < fs.tiles ? c.slot : 0u)), g_cnt, lane);
        }
        // ---- x1 = x + rms(o, post_attention_norm); u = rms(x1, ffn_norm) -------------------------------
        norm_pair<R>(c, c.o_planes, c.X * oks.kparts, L.norm[3], L.norm[4], xr, false, !KQ, c.vec, l, 8);
        stamp(c, l, 4);
        // ---- gate and up columns of this XCD's slice of the FFN width, GeGLU, its receipt --------------
        for (uint32_t pair = c.slot; pair < fs.tiles; pair += kGroups) {
            const uint32_t ct = fs.tile0 + pair;
            const uint32_t dtype = dtype_of(L, g_is_up ? 5 : 4);
            float acc[R];
            if (g_cnt > 0) {
                if (!KQ && pair == c.slot) wave_blocks<KQ, R, !KQ>(c, dtype, g_tiles(L, ct), H, g_wb0, g_cnt, acc, ahead);
                else wave_blocks<KQ, R>(c, dtype, g_tiles(L, ct), H, g_wb0, g_cnt, acc);
            } else {
#pragma unroll
                for (int r = 0; r < R; ++r) acc[r] = 0.f;
            }
#pragma unroll
            for (int r = 0; r < R; ++r) sh.red[(wave * R + r) * 64 + lane] = acc[r];
            __syncthreads();
            if (c.tid < R * 64) {
                const uint32_t r = c.tid >> 6;
                float g = sh.red[r * 64 + lane], u = sh.red[(HW * R + r) * 64 + lane];
                for (uint32_t w = 1; w < HW; ++w) { g += sh.red[(w * R + r) * 64 + lane]; u += sh.red[((HW + w) * R + r) * 64 + lane]; }
                sh.vals[r * 64 + lane] = geglu_value(g, u);
            }
            __syncthreads();
#pragma unroll
            for (int r = 0; r < R; ++r) emit_receipt(sh.vals + r * 64, ct * kTileCols, kTileCols, r, R, F, c.h_receipt, c.tid, kThreads);
        }
        if constexpr (!KQ) {   // the down projection's first tiles
            __builtin_amdgcn_s_waitcnt(0);
            ksplit_ahead(c, ahead, L.tiles[6], dtype_of(L, 6), H / 64, d_nblk, d_first, dnbp, dks, dtg, d_active);
            xcd_barrier(c, true);
        } else {
            xcd_barrier(c);
        }
        stamp(c, l, 5);
        // ---- down projection over this XCD's slice of the FFN width -----------------------------------
        {
            const uint32_t Kp = max(dnbp, 1u) * BE;
            if (d_active && dnbp) copy_receipt<R>(c, c.h_receipt, F, fs.tile0 * 64 + dpb0 * BE, dnbp * BE, dyn);
            __syncthreads();
            ksplit_project<KQ, R, !KQ>(c, L.tiles[6], dtype_of(L, 6), H / 64, d_nblk, d_first, dnbp, Kp, dks, dtg, d_active,
                                       c.d_planes, c.x * d_planes_per_xcd + dkp, H, ahead);
        }
        stamp(c, l, 6);
        const bool more = l + 1 < a.layers;
        if constexpr (!KQ) {   // the next block's q / k / v tiles
            __builtin_amdgcn_s_waitcnt(0);
            if (more) load_ahead(ahead, q_tiles(a.layer[l + 1]), q_cnt, lane);
        }
        // ---- x = x1 + rms(down, post_ffw_norm); u = rms(x, next block's attn_norm or the output norm) ----
        norm_pair<R>(c, c.d_planes, c.X * d_planes_per_xcd, L.norm[5], L.gamma_next, xr, !more, !KQ, c.vec + a.vec_floats);
        stamp(c, l, 7);
    }
}

}  // namespace

uint32_t g_spin_limit = 1u << 20;
unsigned long long* g_resident_stamps = nullptr;
int g_forward_mode = 0;   // 0: resident where the model fits, 1: one launch per operator, 2: resident or an error
namespace {
int g_device_cus = 0;          // CU count of the device guffin_hip_init saw (0: not initialised yet)
bool g_resident_off = false;   // a pass gave up a wait: the automatic mode uses one launch per operator from then on
}  // namespace

int resident_init(int cu_count) {
    g_device_cus = cu_count;
    return 0;
}

void resident_note_status(uint32_t status_word) {
    if (status_word & GUFFIN_STATUS_SYNC) g_resident_off = true;
}

bool resident_chosen(const guffin_model_desc& m, uint32_t rows) {
    if (!resident_fits(m, rows)) return false;
    return g_forward_mode == 2 || (g_forward_mode == 0 && m.kv_heads == 1 && !g_resident_off);
}

}  // namespace guffin

using namespace guffin;

namespace guffin {

uint32_t resident_lds_bytes(const guffin_model_desc& m, uint32_t rows, uint32_t max_ring_tokens);

// Whether the resident kernel covers this model: one KV head per XCD (1 or 8 heads of 256), rows of the
// residual in 512 threads, formats of one block length per model.
bool resident_fits(const guffin_model_desc& m, uint32_t rows) {
    // the placement the pass relies on (256 workgroups, one per CU, dealt to 8 XCDs of 32 CUs in turn) is this part's:
    // on a device with another CU count the per-operator path runs
    if (g_device_cus != 0 && g_device_cus != static_cast<int>(kGrid)) return false;
    if (rows < 1 || rows > 2 || m.head_dim != 256) return false;
    if (m.kv_heads != 1 && m.kv_heads != 8) return false;
    const uint32_t G = m.q_heads / m.kv_heads;
    if (m.q_heads % m.kv_heads || (G != 1 && G != 2 && G != 4)) return false;
    if (m.hidden % 64 || m.hidden > 4096 || m.hidden / 8 > kRowThreads * kRowItems) return false;
    bool kq = false, q8 = false;
    for (uint32_t l = 0; l < m.layer_count; ++l)
        for (int i = 0; i < 7; ++i) (m.layers[l].dtype[i] == GUFFIN_Q8_0 ? q8 : kq) = true;
    if (kq == q8) return false;
    const uint32_t BE = kq ? 256u : 32u;
    if (m.hidden % BE || (m.q_heads * m.head_dim) % BE) return false;
    if (m.ffn % 256 || m.ffn / std::max(BE, 64u) < m.kv_heads) return false;
    // the operand of the widest K part and the attention scratch must fit the CU's LDS beside the static part
    return resident_lds_bytes(m, rows, m.ring_global) <= 140u * 1024u;
}

struct ResidentSizes { uint64_t qkv, attn_out, attn_ml, o_planes, d_planes, vec, h_receipt, set, sync, total; uint32_t opnd, lds; };

static ResidentSizes resident_sizes(const guffin_model_desc& m, uint32_t rows, uint32_t max_ring_tokens) {
    ResidentSizes s {};
    const uint32_t X = m.kv_heads, G = m.q_heads / m.kv_heads, NQ = rows * G, H = m.hidden, F = m.ffn;
    const bool kq = m.layers[0].dtype[0] != GUFFIN_Q8_0;
    const uint32_t BE = kq ? 256u : 32u;
    const uint32_t TA = 4 * G + 8, PA = std::max(1u, kGroups / TA);
    auto al = [](uint64_t b) { return (b + 255) & ~uint64_t{255}; };
    s.qkv = al(uint64_t(X) * PA * rows * (G + 2) * kHd * 4);
    s.attn_out = al(uint64_t(X) * kGroups * NQ * kHd * 4);
    s.attn_ml = al(uint64_t(X) * kGroups * NQ * 2 * 4);
    const KSplit ko = ksplit_of(H / 64, G * kHd / BE);
    const FSlice f0 = fslice_of(F, BE, X, 0);
    const KSplit kd = ksplit_of(H / 64, f0.tiles * 64 / BE);
    s.o_planes = al(uint64_t(X) * ko.kparts * rows * H * 4);
    s.d_planes = al(uint64_t(X) * kd.kparts * rows * H * 4);
    s.vec = al(uint64_t(X) * rows * H * 4);
    s.h_receipt = al(receipt_layout(rows, F).bytes);
    const uint32_t launches = (m.layer_count + kResidentLayers - 1) / kResidentLayers;
    s.sync = al(uint64_t(launches) * kSyncWords * 4);
    // one set of exchange buffers per block of a launch (two `vec`: one per norm joint): no address is read twice
    s.set = s.qkv + s.attn_out + s.attn_ml + s.o_planes + s.d_planes + 2 * s.vec + s.h_receipt;
    s.total = s.set * kResidentLayers + s.sync;
    // LDS: the operand receipt of the widest K a workgroup sees (the hidden width, or a K part of o / down),
    // then that part's fp32 values (the merged attention rows); or the attention scratch
    const uint32_t kp_o = ko.bpp * BE, kp_d = kd.bpp * BE;
    const uint32_t kmax = std::max({H, kp_o, kp_d});
    s.opnd = static_cast<uint32_t>(al(receipt_layout(rows, kmax).bytes));
    const uint32_t vals = rows * kp_o * 4;
    const uint32_t tp = (max_ring_tokens + rows + kGroups - 1) / kGroups;
    const uint32_t attn = ((NQ * tp + 63) & ~63u) * 4 + kWaves * NQ * kHd * 4;
    s.lds = std::max(s.opnd + vals, attn);
    return s;
}

// Where the regions of one block's set start: q/k/v parts, attention outputs, attention (maximum, denominator)
// pairs, o planes, down planes, the two norm joints' vectors, the GeGLU receipt.  Regions are handed over in
// different phases, between CUs whose L1 nothing invalidates: each starts on a 256-byte boundary of the set
// (two cache lines), so no line holds words of two regions.
struct ResidentLayout { uint64_t offset[8], bytes[8]; };

static ResidentLayout resident_layout(const ResidentSizes& s) {
    ResidentLayout at {};
    const uint64_t sizes[8] = {s.qkv, s.attn_out, s.attn_ml, s.o_planes, s.d_planes, s.vec, s.vec, s.h_receipt};
    uint64_t p = 0;
    for (int i = 0; i < 8; ++i) {
        at.offset[i] = p;
        at.bytes[i] = sizes[i];
        p += sizes[i];
    }
    return at;
}

uint32_t resident_lds_bytes(const guffin_model_desc& m, uint32_t rows, uint32_t max_ring_tokens) {
    return resident_sizes(m, rows, max_ring_tokens).lds;
}

uint64_t resident_scratch_bytes(const guffin_model_desc& m, uint32_t rows) {
    return resident_sizes(m, rows, m.ring_global).total;
}

uint32_t resident_sync_words(const guffin_model_desc& m) {
    return ((m.layer_count + kResidentLayers - 1) / kResidentLayers) * kSyncWords;
}

template <int R, int G, bool KQ>
static int launch_resident(hipStream_t stream, const RArgs& args, uint32_t lds) {
    static bool raised = false;
    auto* kernel = resident_blocks_kernel<R, G, KQ>;
    if (!raised) {
        if (hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, 140 * 1024) != hipSuccess)
            return fail(GUFFIN_E_HIP, "resident forward: could not raise the dynamic LDS limit");
        raised = true;
    }
    launch(kernel, dim3(kGrid), dim3(kThreads), lds, stream, args);
    return check_launch("resident_blocks");
}

// Runs blocks [first, first + count) of the model (count <= kResidentLayers) from the state in x / u_receipt.
int resident_launch(hipStream_t stream, const guffin_model_desc& m, uint32_t rows, uint32_t first, uint32_t count,
                    uint8_t* exchange, uint32_t* sync_words, const float* rope_local, const float* rope_global,
                    const uint32_t* schedule, const uint32_t* ancestors, void* priv_k, void* priv_v, const float* x_in,
                    const void* u_receipt_in, float* x_out, float* u_out, void* u_receipt_out, uint32_t max_ring_tokens,
                    uint32_t* status) {
    const ResidentSizes s = resident_sizes(m, rows, max_ring_tokens);
    RArgs a {};
    const uint32_t KW = m.kv_heads * m.head_dim;
    for (uint32_t i = 0; i < count; ++i) {
        const uint32_t l = first + i;
        const guffin_layer_desc& L = m.layers[l];
        RLayer& rl = a.layer[i];
        rl.dtype_bits = 0;
        for (int k = 0; k < 7; ++k) {
            rl.tiles[k] = static_cast<const uint8_t*>(L.tiles[k]);
            rl.dtype_bits |= uint32_t(L.dtype[k]) << (4 * k);
        }
        for (int k = 0; k < 6; ++k) rl.norm[k] = L.norm[k];
        rl.gamma_next = l + 1 == m.layer_count ? m.out_norm : m.layers[l + 1].norm[0];
        rl.ring_k = static_cast<const uint16_t*>(L.ring_k);
        rl.ring_v = static_cast<const uint16_t*>(L.ring_v);
        const bool local = layer_is_local(m.global_period, l);
        rl.rope = reinterpret_cast<const float2*>(local ? rope_local : rope_global);
        rl.schedule = schedule + size_t(l) * rows * 4;
        rl.priv_k = static_cast<uint16_t*>(priv_k) + size_t(l) * rows * KW;
        rl.priv_v = static_cast<uint16_t*>(priv_v) + size_t(l) * rows * KW;
        rl.ring_mask = (local ? m.ring_local : m.ring_global) - 1;
    }
    a.layers = count; a.H = m.hidden; a.F = m.ffn; a.kv_heads = m.kv_heads;
    a.eps = m.eps; a.scale = 1.0f / std::sqrt(static_cast<float>(m.head_dim));
    const ResidentLayout at = resident_layout(s);
    a.qkv_part = reinterpret_cast<float*>(exchange + at.offset[0]);
    a.attn_out = reinterpret_cast<float*>(exchange + at.offset[1]);
    a.attn_ml = reinterpret_cast<float*>(exchange + at.offset[2]);
    a.o_planes = reinterpret_cast<float*>(exchange + at.offset[3]);
    a.d_planes = reinterpret_cast<float*>(exchange + at.offset[4]);
    a.vec = reinterpret_cast<float*>(exchange + at.offset[5]);     // the second joint's follows at vec_floats
    a.h_receipt = exchange + at.offset[7];
    a.sync = sync_words;
    a.x_in = x_in; a.u_receipt_in = u_receipt_in; a.x_out = x_out; a.u_out = u_out; a.u_receipt_out = u_receipt_out;
    a.ancestors = ancestors; a.status = status;
    a.spin_limit = g_spin_limit; a.opnd_bytes = s.opnd;
    a.set_floats = static_cast<uint32_t>(s.set / 4); a.vec_floats = static_cast<uint32_t>(s.vec / 4);
    a.stamps = g_resident_stamps ? g_resident_stamps + size_t(first) * 16 : nullptr;
    const uint32_t G = m.q_heads / m.kv_heads;
    const bool kq = m.layers[0].dtype[0] != GUFFIN_Q8_0;
#define GUFFIN_RES(R_, G_) (kq ? launch_resident<R_, G_, true>(stream, a, s.lds) : launch_resident<R_, G_, false>(stream, a, s.lds))
    switch (rows * 10 + G) {
        case 11: return GUFFIN_RES(1, 1);
        case 12: return GUFFIN_RES(1, 2);
        case 14: return GUFFIN_RES(1, 4);
        case 21: return GUFFIN_RES(2, 1);
        case 22: return GUFFIN_RES(2, 2);
        case 24: return GUFFIN_RES(2, 4);
    }
#undef GUFFIN_RES
    return fail(GUFFIN_E_SHAPE, "resident forward: unsupported head grouping");
}

}  // namespace guffin

extern "C" int guffin_hip_set_forward_mode(int mode) {
    if (mode < 0 || mode > 2) return fail(GUFFIN_E_ARG, "set_forward_mode: 0 (automatic), 1 (one launch per operator) or 2 (resident only)");
    g_forward_mode = mode;
    g_resident_off = false;   // the caller chose again: an earlier give-up no longer decides
    return GUFFIN_OK;
}

extern "C" int guffin_hip_resident_enabled(void) { return g_resident_off ? 0 : 1; }

extern "C" int guffin_hip_resident_layout(const guffin_model_desc* model, uint32_t rows, uint64_t* offsets, uint64_t* bytes,
                                          uint64_t* set_bytes, uint32_t* sets, uint64_t* total_bytes) {
    if (!model || !model->layers || !offsets || !bytes || !set_bytes || !sets || !total_bytes || rows < 1 || rows > 2)
        return fail(GUFFIN_E_ARG, "resident_layout: null pointer or rows outside [1, 2]");
    if (model->kv_heads == 0 || model->q_heads % model->kv_heads != 0 || model->hidden % 64 != 0)
        return fail(GUFFIN_E_SHAPE, "resident_layout: not a shape the resident pass is laid out for");
    const ResidentSizes s = resident_sizes(*model, rows, model->ring_global);
    const ResidentLayout at = resident_layout(s);
    for (int i = 0; i < 8; ++i) { offsets[i] = at.offset[i]; bytes[i] = at.bytes[i]; }
    *set_bytes = s.set;
    *sets = kResidentLayers;
    *total_bytes = s.total;
    return GUFFIN_OK;
}

extern "C" int guffin_hip_set_spin_limit(uint32_t polls) {
    g_spin_limit = polls;
    return GUFFIN_OK;
}

extern "C" int guffin_hip_set_resident_stamps(void* device_words) {
    g_resident_stamps = static_cast<unsigned long long*>(device_words);
    return GUFFIN_OK;
}
