/*
 * guffin_hip.h — C ABI of the MI355X (gfx950) backend for Guffin's H1 speculative
 * decode step.  One entry point per `encode_*` operation of the reference's kernel
 * boundary (src/tensor/backends/metal/metal_command_context.hpp:54-369): plain
 * pointers and sizes, caller-owned device memory, work enqueued on the caller's HIP
 * stream (`stream` is a hipStream_t passed as void*, NULL = default stream).
 *
 * Return value of every function: 0 on success, a negative GUFFIN_E_* code when the
 * arguments are rejected before anything is enqueued (the reference throws
 * std::invalid_argument there), or GUFFIN_E_HIP when the HIP runtime refuses a
 * launch.  Numerical faults never fail a call: kernels OR bits into a caller-provided
 * device status word (reference: metal_command_context.hpp:16-17), which the host
 * reads after completion.  guffin_hip_last_error() describes the last failure of the
 * calling thread.  Nothing here allocates device memory.
 *
 * Weight matrices are GGUF block streams of a [K inputs, N output columns] matrix in
 * which output column n owns the K/block consecutive blocks starting at block
 * n*(K/block) (reference: src/tensor/backends/cpu_backend.cpp:43-53).
 */
#ifndef GUFFIN_HIP_H
#define GUFFIN_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define GUFFIN_OK 0
#define GUFFIN_E_ARG (-1)       /* null pointer, zero size, unsupported value */
#define GUFFIN_E_SHAPE (-2)     /* K not a multiple of the block size, rows out of range ... */
#define GUFFIN_E_ALIGN (-3)     /* pointer alignment below what the block stream guarantees */
#define GUFFIN_E_CAPACITY (-4)  /* exceeds a fixed capacity (LDS, candidate count ...) */
#define GUFFIN_E_HIP (-5)       /* HIP runtime error, see guffin_hip_last_error() */

/* reference: include/local_gguf_engine/tensor/dtype.hpp:9-15 (block layouts 34/144/210 B) */
#define GUFFIN_Q8_0 0
#define GUFFIN_Q4_K 1
#define GUFFIN_Q6_K 2

/* device status bits (reference: metal_command_context.hpp:16-17, gemma3_draft.mm status codes) */
#define GUFFIN_STATUS_BAD_TOKEN 1u       /* token id outside the vocabulary */
#define GUFFIN_STATUS_NONFINITE 2u       /* non-finite activation or logit */
#define GUFFIN_STATUS_KV_NONFINITE 8u    /* non-finite value narrowed into the fp16 KV rows */
#define GUFFIN_STATUS_LAW_INVALID 16u    /* proposal / target law could not be built */

const char* guffin_hip_last_error(void);
/* Binds the calling thread to `device`, checks that it is a gfx950 and raises the
 * kernels' dynamic LDS limits.  Must be called once per device before any other call. */
int guffin_hip_init(int device);
/* Name of the architecture the loaded code object was built for ("gfx950"). */
const char* guffin_hip_arch(void);

/* ---- block decode ---------------------------------------------------------------
 * out[b*elems + i] = value of element i of block b, bit-exact with the reference's
 * block views: Q8_0 d*q (src/tensor/quantization.cpp:457-459), Q4_K (d*sc)*q - dmin*m
 * (:517-521), Q6_K (d*scale)*q (:590-593). */
int guffin_hip_dequant(void* stream, int dtype, const void* blocks, uint64_t n_blocks, float* out);

/* ---- dequant-GEMV: y[r,n] = sum_k x[r,k] * W[k,n], fp32 accumulate ------------------
 * Replaces MetalCommandContext::encode_verifier_matmul (metal_command_context.hpp:94),
 * encode_target_head_rows (:103) and the drafter's `linear` (src/engine/gemma3_draft.mm:826-838);
 * CPU definition src/tensor/backends/cpu_backend.cpp:301-323.
 * x is [rows, K] fp32 row-major, y is [rows, N] fp32 row-major, rows in [1, 8].
 * Each output row is computed by the same instruction sequence whatever `rows` is, so a
 * row of a 2-row call is bit-equal to the 1-row call on that row. */
int guffin_hip_gemv(void* stream, int dtype, const void* w, const float* x, float* y,
                    uint32_t rows, uint32_t K, uint32_t N);
int guffin_hip_gemv_q4k(void* stream, const void* w, const float* x, float* y,
                        uint32_t rows, uint32_t K, uint32_t N);
int guffin_hip_gemv_q6k(void* stream, const void* w, const float* x, float* y,
                        uint32_t rows, uint32_t K, uint32_t N);
int guffin_hip_gemv_q80(void* stream, const void* w, const float* x, float* y,
                        uint32_t rows, uint32_t K, uint32_t N);

/* ---- wave-tile weights (lossless repack) and the GEMV that streams them ------------------
 * The reference re-lays K-quant weights at upload into a layout its GPU loads coalesce on
 * and keeps the repack lossless (src/tensor/kquant_packing.hpp:9-23; round trip pinned in
 * tests/tensor/tensor_tests.cpp:3193-3283).  This is the gfx950 counterpart: tiles of 64
 * adjacent output columns x one block, every 16-byte piece stored lane-major.  Same byte
 * count as the canonical stream; N must be a multiple of 64. */
uint64_t guffin_hip_packed_bytes(int dtype, uint32_t K, uint32_t N);
int guffin_hip_repack(void* stream, int dtype, const void* canonical, void* tiles, uint32_t K, uint32_t N);
int guffin_hip_unpack(void* stream, int dtype, const void* tiles, void* canonical, uint32_t K, uint32_t N);

/* Per-row sums of 16 and of 32 consecutive activations: xsums is [rows][K/16 + K/32]
 * (16-sums first).  The reference's producers emit the same kind of receipt for its Q4_K
 * kernels (src/tensor/backends/metal/metal_kernels.mm:16-27, "Q4 sums"). */
int guffin_hip_group_sums(void* stream, const float* x, float* xsums, uint32_t rows, uint32_t K);

/* Number of k-slices S the packed GEMV cuts this shape into (size of the partials buffer). */
uint32_t guffin_hip_gemv_packed_slices(int dtype, uint32_t K, uint32_t N);
/* Same operator as guffin_hip_gemv on repacked weights.  rows in {1, 2}.  Slice partials are
 * written to partials[S][rows][N]; if y is non-null they are summed in slice order into
 * y[rows][N] by a second small launch, otherwise the consumer does that sum. */
int guffin_hip_gemv_packed(void* stream, int dtype, const void* tiles, const float* x, const float* xsums,
                           float* partials, float* y, uint32_t rows, uint32_t K, uint32_t N);

#ifdef __cplusplus
}
#endif
#endif /* GUFFIN_HIP_H */
