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
#define GUFFIN_E_STATE (-6)     /* call out of order for the session's state, or the session is poisoned */
#define GUFFIN_E_NUMERIC (-7)   /* a verify pass raised its device status word (guffin_hip_ticket_complete) */

/* reference: include/local_gguf_engine/tensor/dtype.hpp:9-15 (block layouts 34/144/210 B) */
#define GUFFIN_Q8_0 0
#define GUFFIN_Q4_K 1
#define GUFFIN_Q6_K 2

/* device status bits (reference: metal_command_context.hpp:16-17, gemma3_draft.mm status codes) */
#define GUFFIN_STATUS_BAD_TOKEN 1u       /* token id outside the vocabulary */
#define GUFFIN_STATUS_NONFINITE 2u       /* non-finite activation or logit */
#define GUFFIN_STATUS_KV_NONFINITE 8u    /* non-finite value narrowed into the fp16 KV rows */
#define GUFFIN_STATUS_LAW_INVALID 16u    /* proposal / target law could not be built */
#define GUFFIN_STATUS_SYNC 64u           /* a workgroup of the resident forward pass gave up a bounded wait */

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

/* Activation receipt of rows x K activations (K % 32 == 0, rows 1 or 2): one 256-byte aligned
 * blob of guffin_hip_receipt_bytes(rows, K) bytes holding
 *   float sums[rows][K/16 + K/32]   sums of 16 and of 32 consecutive activations (16-sums first);
 *                                   the reference's producers emit the same kind of receipt for its
 *                                   Q4_K kernels (src/tensor/backends/metal/metal_kernels.mm:16-27)
 *   float mult[rows][K/32]          at the next 256-byte boundary: 2^(E+24) per 32-group
 *   half  image[K/32][4][32]        at the next 256-byte boundary: variants {row0 hi, row0 lo,
 *                                   row1 hi, row1 lo} of x * 2^-E (hi + lo exact to 22 bits), the
 *                                   matrix-core operand of the packed Q4_K GEMV; inside a group the
 *                                   halves of elements 8s..8s+7 sit at 8s + {0,2,1,3,4,6,5,7}
 * Every operator below that has an `*_sums` output writes this whole blob. */
uint64_t guffin_hip_receipt_bytes(uint32_t rows, uint32_t K);
int guffin_hip_group_sums(void* stream, const float* x, float* xsums, uint32_t rows, uint32_t K);

/* Number of k-slices S the packed GEMV cuts this shape into (size of the partials buffer). */
uint32_t guffin_hip_gemv_packed_slices(int dtype, uint32_t K, uint32_t N);
/* Same operator as guffin_hip_gemv on repacked weights.  rows in {1, 2}.  Slice partials are
 * written to partials[S][rows][N]; if y is non-null they are summed in slice order into
 * y[rows][N] by a second small launch (with S == 1 the kernel writes y directly and leaves
 * partials untouched), otherwise the consumer does that sum. */
int guffin_hip_gemv_packed(void* stream, int dtype, const void* tiles, const float* x, const float* xsums,
                           float* partials, float* y, uint32_t rows, uint32_t K, uint32_t N);

/* guffin_hip_gemv_packed for callers that cannot allocate device memory or carry a workspace (code under
 * HIP graph capture, tight serving loops, harnesses that forbid hipMalloc): the partial planes live in a
 * static device array of the library (128 KiB per GPU, held until the process ends) instead of `partials`.
 * No counterpart in the reference.  Refuses launches whose planes * rows * N exceed
 * guffin_hip_gemv_packed_static_limit() floats (GUFFIN_E_CAPACITY) and devices guffin_hip_init has not
 * seen (GUFFIN_E_STATE).  Calls no allocator.  All calls on one GPU share that GPU's array: calls that
 * overlap on one GPU (two streams) race; calls on one stream do not. */
uint64_t guffin_hip_gemv_packed_static_limit(void);
int guffin_hip_gemv_packed_static(void* stream, int dtype, const void* tiles, const float* x, const float* xsums,
                                  float* y, uint32_t rows, uint32_t K, uint32_t N);

/* Up to three matrices that share the activation rows (q/k/v, gate/up) in one launch.  Each
 * matrix i writes partials[i] as [S][rows][N_i] with the one S = guffin_hip_gemv_packed_multi_slices
 * of the launch.  All matrices must share the block length (Q4_K and Q6_K mix, Q8_0 does not). */
uint32_t guffin_hip_gemv_packed_multi_slices(uint32_t count, const int* dtypes, const uint32_t* N, uint32_t K);
int guffin_hip_gemv_packed_multi(void* stream, uint32_t count, const int* dtypes, const void* const* tiles,
                                 const uint32_t* N, float* const* partials, const float* x,
                                 const float* xsums, uint32_t rows, uint32_t K);

/* h = gelu_tanh(x W_gate) * (x W_up) with its activation receipt in one launch (gate and up of
 * the same dtype, Q4_K or Q8_0): guffin_hip_gemv_packed_multi + guffin_hip_geglu without the
 * partial planes in between (reference: two encode_verifier_matmul and encode_gelu_tanh_multiply,
 * src/engine/gemma_target_runtime.cpp:176-199).  h [rows][F]; h_sums may be NULL. */
int guffin_hip_gateup_geglu(void* stream, int dtype, const void* gate_tiles, const void* up_tiles,
                            const float* x, const float* xsums, float* h, float* h_sums,
                            uint32_t rows, uint32_t K, uint32_t F);

/* ---- per-layer operators -----------------------------------------------------------------
 * Inputs produced by a packed GEMV may be given as `planes` k-slice partial planes
 * (`plane_stride` floats apart) that the operator sums in slice order while loading; plain
 * tensors pass planes = 1.  Outputs that feed a packed GEMV can also emit their group sums
 * (`*_sums`, layout of guffin_hip_group_sums; pass NULL to skip). */

/* y = x * rsqrt(mean(x^2) + eps) * gamma (+ residual if non-null).  Replaces encode_rms_norm
 * (metal_command_context.hpp:128) and encode_rms_norm_add (:137); CPU definition
 * src/tensor/ops/normalization.cpp:70-99.  status: GUFFIN_STATUS_NONFINITE on a non-finite output. */
int guffin_hip_rms_norm(void* stream, const float* x, uint32_t planes, uint64_t plane_stride,
                        const float* gamma, const float* residual, float* y, float* y_sums,
                        uint32_t rows, uint32_t width, float eps, uint32_t* status);
/* out_residual = residual + rms(x, gamma_post); out_norm = rms(out_residual, gamma_next): the
 * encode_rms_norm_add + encode_rms_norm pair at the joints of a block
 * (src/engine/gemma_target_runtime.cpp:156-173, 201-213 then :60-66 of the next block). */
int guffin_hip_rms_norm_add_norm(void* stream, const float* x, uint32_t planes, uint64_t plane_stride,
                                 const float* gamma_post, const float* residual, float* out_residual,
                                 const float* gamma_next, float* out_norm, float* out_sums,
                                 uint32_t rows, uint32_t width, float eps, uint32_t* status);
/* Per-head RMS norm over head_dim, in place allowed.  Replaces encode_head_rms_norm (:119). */
int guffin_hip_head_rms_norm(void* stream, const float* x, const float* gamma, float* y,
                             uint32_t rows, uint32_t heads, uint32_t head_dim, float eps);
/* Split-half (NeoX) RoPE with one absolute position per row: theta = pos / base^(2i/rope_dim) * scale.
 * Replaces encode_verifier_rope (:239); CPU definition src/tensor/ops/rope.cpp:242-283. */
int guffin_hip_rope_neox(void* stream, const float* in, const uint32_t* positions, float* out,
                         uint32_t rows, uint32_t heads, uint32_t head_dim, uint32_t rope_dim,
                         float freq_base, float freq_scale);
/* K = f16(rope(raw_k)), V = f16(raw_v), round-to-nearest-even after rotation, into private
 * rows [rows][heads*head_dim].  Replaces encode_verifier_kv_store (:250; bit contract
 * tests/tensor/gemma3_metal_tests.cpp:87-128).  status: GUFFIN_STATUS_KV_NONFINITE. */
int guffin_hip_kv_store_f16(void* stream, const float* raw_k, const float* raw_v, const uint32_t* positions,
                            void* out_k, void* out_v, uint32_t rows, uint32_t heads, uint32_t head_dim,
                            uint32_t rope_dim, float freq_base, float freq_scale, uint32_t* status);
/* cos and sin of every (row, pair) angle, table[rows][rope_dim/2][2] = {cos, sin}, formed in
 * double exactly as guffin_hip_rope_neox forms them (src/tensor/ops/rope.cpp:109-117); a
 * forward pass fills one table per frequency base and hands it to every block's qkv_post. */
int guffin_hip_rope_table(void* stream, const uint32_t* positions, float* table, uint32_t rows,
                          uint32_t rope_dim, float freq_base, float freq_scale);
/* The three steps between the QKV GEMVs and attention in one launch: q/k head norms
 * (NULL gamma skips), RoPE on q and k, fp16 narrowing of k and v
 * (src/engine/gemma_target_runtime.cpp:92-124).  rope_table (optional) replaces positions,
 * freq_base and freq_scale by a table from guffin_hip_rope_table. */
int guffin_hip_qkv_post(void* stream, const float* q_raw, const float* k_raw, const float* v_raw,
                        uint32_t q_planes, uint32_t k_planes, uint32_t v_planes,
                        uint64_t q_plane_stride, uint64_t k_plane_stride,
                        uint64_t v_plane_stride, const float* q_norm, const float* k_norm,
                        const uint32_t* positions, float* q_out, void* k_out, void* v_out,
                        uint32_t rows, uint32_t q_heads, uint32_t kv_heads, uint32_t head_dim,
                        uint32_t rope_dim, float freq_base, float freq_scale, float eps,
                        const float* rope_table, uint32_t* status);
/* out = 0.5 g (1 + tanh(0.7978845608 (g + 0.044715 g^3))) * up.  Replaces
 * encode_gelu_tanh_multiply (:313); CPU definition src/tensor/ops/elementwise.cpp:79-94, 50-63. */
int guffin_hip_geglu(void* stream, const float* gate, const float* up, uint32_t planes, uint64_t plane_stride,
                     float* out, float* out_sums, uint32_t rows, uint32_t width);
/* out[r,:] = dequant(row tokens[r] of the [vocab x width] canonical block stream) * scale.
 * Replaces encode_embedding (:75) and the drafter's gd_embed (src/engine/gemma3_draft.mm:61-71).
 * A token >= vocab sets GUFFIN_STATUS_BAD_TOKEN and reads row 0. */
int guffin_hip_embed(void* stream, int dtype, const void* w, const uint32_t* tokens, float* out,
                     uint32_t rows, uint32_t width, float scale, uint32_t vocab, uint32_t* status);
/* ring[(position + i) & ring_mask] = private[selected[i]] for K and V (fp16 rows of row_width
 * elements).  Replaces encode_verifier_kv_scatter (:290). */
int guffin_hip_kv_scatter(void* stream, const void* priv_k, const void* priv_v, const uint32_t* selected,
                          void* ring_k, void* ring_v, uint32_t position, uint32_t rows,
                          uint32_t row_width, uint32_t ring_mask);

/* ---- GQA decode / verify attention over the fp16 KV cache -----------------------------------
 * Replaces encode_verifier_attention (:267) and its partition reducer; CPU definition
 * src/tensor/ops/attention.cpp:482-618 + softmax.cpp:42-71 (no logit softcap: Gemma 3).
 * schedule: 4 u32 per row {base_first_position, base_token_count, ancestor_offset, ancestor_count}
 * (metal_kernels.mm:129-134); row r attends ring slots (base_first+t)&ring_mask for t<base_count,
 * then private rows ancestors[ancestor_offset + i].  rows in {1,2}; head_dim 256;
 * q_heads/kv_heads in {1,2,4}.  max_tokens >= (union of the rows' ring ranges) + private_rows.
 * partial_out holds rows*q_heads*P*head_dim floats and partial_ml rows*q_heads*P*2 floats with
 * P = guffin_hip_attention_partitions(max_tokens, kv_heads). */
uint32_t guffin_hip_attention_partitions(uint32_t max_tokens, uint32_t kv_heads);
int guffin_hip_attention_decode(void* stream, const float* q, const void* ring_k, const void* ring_v,
                                const void* priv_k, const void* priv_v, const uint32_t* schedule,
                                const uint32_t* ancestors, float* out, float* out_sums,
                                float* partial_out, float* partial_ml, uint32_t rows,
                                uint32_t private_rows, uint32_t max_tokens, uint32_t ring_mask,
                                uint32_t q_heads, uint32_t kv_heads, uint32_t head_dim, float scale,
                                uint32_t* status);
/* encode_head_rms_norm + encode_verifier_rope + encode_verifier_kv_store + encode_verifier_attention
 * (metal_command_context.hpp:119, 239, 250, 267) in one pass over the projections' partial planes
 * ([planes][rows][heads * head_dim], summed in plane order): every attention workgroup prepares the
 * query heads it serves, and the partition that holds a private row prepares that row's key and
 * value, uses them and writes them to priv_k / priv_v as fp16 (one private row per query row, full
 * rotation from rope_table: [rows][head_dim / 2] (cos, sin) pairs, guffin_hip_rope_table).
 * q_norm / k_norm may be NULL (no head norm). */
int guffin_hip_qkv_attention(void* stream, const float* q_raw, const float* k_raw, const float* v_raw,
                             uint32_t planes, uint64_t q_plane_stride, uint64_t k_plane_stride,
                             uint64_t v_plane_stride, const float* q_norm, const float* k_norm,
                             const float* rope_table, float eps, const void* ring_k, const void* ring_v,
                             void* priv_k, void* priv_v, const uint32_t* schedule,
                             const uint32_t* ancestors, float* out, float* out_sums, float* partial_out,
                             float* partial_ml, uint32_t rows, uint32_t max_tokens, uint32_t ring_mask,
                             uint32_t q_heads, uint32_t kv_heads, uint32_t head_dim, float scale,
                             uint32_t* status);

/* ---- output-head selection ---------------------------------------------------------------
 * Per row the best `retain` (= top_k + history count, the reference's base_candidate_count)
 * logits by (logit desc, token asc), then the logits of the row's history tokens.  Replaces
 * encode_token_candidates[_width_two] / encode_target_token_candidates (:326-345) and
 * read_token_candidates; order src/engine/sampling.cpp:25-30.
 * result: per row { u32 count; u32 status; {u32 token; f32 logit} values[384]; }
 * (CompactTokenCandidates, include/local_gguf_engine/engine/sampling.hpp:57-61, plus the status).
 * history: [rows][64] token ids with history_count[rows] (both NULL for none).
 * status: one u32 per row; GUFFIN_STATUS_NONFINITE if the row holds a non-finite logit,
 * GUFFIN_STATUS_BAD_TOKEN for a history token outside the vocabulary. */
uint64_t guffin_hip_select_workspace_bytes(uint32_t rows, uint32_t vocab, uint32_t retain);
int guffin_hip_select_candidates(void* stream, const float* logits, uint32_t rows, uint32_t vocab,
                                 uint32_t retain, const uint32_t* history, const uint32_t* history_count,
                                 void* workspace, void* result, uint32_t* status);
/* The token ids a verify pass reads on the device against the ids the host planned: a row whose id is
 * outside the vocabulary or differs sets GUFFIN_STATUS_BAD_TOKEN in the one status word.  Replaces
 * encode_verifier_input_validation (metal_command_context.hpp:221; verifier_input_validate_u32_kernel,
 * src/tensor/backends/metal/metal_kernels.mm:2323-2334, which sets the same bit 1). */
int guffin_hip_input_validation(void* stream, const uint32_t* actual, const uint32_t* expected, uint32_t rows,
                                uint32_t vocab, uint32_t* status);
/* Selection requests of a verify pass, resolved on the device: per row the raw sampler history (a ring
 * of history_window_limit slots with the oldest token at history_head) and the suffix of tokens observed
 * before that row become the window after the appends, without later duplicates, and
 * base_candidate_count = top_k + its length.  Replaces verifier_selection_request_resolve_kernel
 * (src/tensor/backends/metal/metal_kernels.mm:2336-2404); on the host the reference computes the same
 * with make_token_selection_request (src/engine/sampling.cpp:352-392).
 * raw:      rows x guffin_selection_row  (VerifierDeviceSelectionRow,
 *           include/local_gguf_engine/engine/target_verifier.hpp:114-121), device
 * resolved: rows x guffin_resolved_row   (VerifierResolvedSelectionRow, metal_kernels.mm:91-97), device
 * histories: rows x 64 token ids (the lists again, as the candidate kernels of the reference read them), or NULL
 * status:   ONE word with the reference's bits, not the GUFFIN_STATUS_* of the other entry points:
 *           GUFFIN_REQUEST_MALFORMED (window > 64, length > window, suffix > 23, a head outside the
 *           window: the row resolves to top_k with no history) and GUFFIN_REQUEST_BAD_TOKEN (a history
 *           or suffix token >= vocab: it is left out of the list).
 * repetition_enabled == 0 (a penalty of exactly 1): rows resolve to top_k with no history. */
#define GUFFIN_REQUEST_MALFORMED 2u
#define GUFFIN_REQUEST_BAD_TOKEN 4u
typedef struct {
    uint32_t history_token_ids[64]; uint32_t suffix_token_ids[23];
    uint32_t history_head, history_length, history_window_limit, suffix_count;
} guffin_selection_row;
typedef struct {
    uint32_t top_k, base_candidate_count, history_count, reserved; uint32_t history_token_ids[64];
} guffin_resolved_row;
int guffin_hip_selection_requests(void* stream, const void* raw, uint32_t rows, uint32_t vocab, uint32_t top_k,
                                  uint32_t repetition_enabled, void* resolved, uint32_t* histories,
                                  uint32_t* status);
/* guffin_hip_select_candidates on resolved requests: row r keeps its base_candidate_count best logits
 * (at most retain_capacity, which sizes the workspace: guffin_hip_select_workspace_bytes(rows, vocab,
 * retain_capacity)) and then the logits of its history_token_ids. */
int guffin_hip_select_candidates_resolved(void* stream, const float* logits, uint32_t rows, uint32_t vocab,
                                          uint32_t retain_capacity, const void* resolved, void* workspace,
                                          void* result, uint32_t* status);
/* Greedy token per row, strict '>' so the lowest id wins ties (src/tensor/ops/reduction.cpp:93-117).
 * workspace: rows * 256 * 8 bytes.  logit may be NULL. */
int guffin_hip_argmax(void* stream, const float* logits, uint32_t rows, uint32_t vocab, void* workspace,
                      uint32_t* token, float* logit, uint32_t* status);

/* ---- proposal law and lossless acceptance ---------------------------------------------------
 * options: { f32 temperature; u32 top_k; f32 top_p; f32 min_p; f32 repetition_penalty; }
 * draws:   { u32 word; u32 pad; f64 u_accept; f64 u_residual; f64 u_next; } — when the injected
 *          pointer is NULL the kernels derive them from Philox4x32-10 with key = seed and
 *          counters (step, 0) -> {word, u_accept}, (step, 1) -> {u_residual, u_next}, 53-bit
 *          uniforms in [0,1).  The reference draws from mt19937_64 streams
 *          (src/engine/sampling.cpp:45-60); the consumption pattern is kept (:896-934).
 *
 * guffin_hip_draft_law builds the drafter's compact proposal law from full-vocabulary logits:
 * score = logit / T, support = every token scoring >= the top_k-th best (<= 256 entries, else
 * status bit 32 is raised), descending-tail top-p / min-p, f32 prefix / total * 2^32 -> u64 bins
 * in ascending token id (src/engine/gemma3_draft.mm:191-294), and selects the proposal with
 * the step's 32-bit word.  law: { u32 count; u32 pad; u32 ids[256]; u64 cdf[257]; }. */
uint64_t guffin_hip_draft_law_workspace_bytes(uint32_t vocab);
int guffin_hip_draft_law(void* stream, const float* logits, uint32_t vocab, const void* options,
                         uint64_t seed, uint64_t step, const void* injected_draws, void* workspace,
                         void* law, uint32_t* proposal, uint32_t* status);
/* scores[i] = logits[i] with the repetition penalty on the tokens of the sampler history (divided
 * when >= 0, multiplied when negative): what the drafter's gd_process does before its law is built
 * (src/engine/gemma3_draft.mm:186-204); the law entry points then take `scores` for logits.
 * history: at most 64 device words; scores may not alias logits. */
int guffin_hip_draft_process(void* stream, const float* logits, uint32_t vocab, const uint32_t* history,
                             uint32_t history_count, float repetition_penalty, float* scores);

/* The drafter's law by whichever path the options and the logits need, as the reference's
 * `sample` encodes it (src/engine/gemma3_draft.mm:995-1166): the compact law when temperature > 0
 * and top_k <= 64, followed by the full-vocabulary kernels (:295-395), which run only when more
 * than 256 tokens tie into the compact support; the full-vocabulary kernels alone otherwise
 * (top_k > 64, or temperature == 0: all mass on the lowest-id argmax).  A law held as the full
 * table is marked by law.count == 0xFFFFFFFF and lives in full_cdf: u64[vocab + 1], bin of token
 * i = [full_cdf[i], full_cdf[i+1]), last entry 2^32.  vocab must be a multiple of 256 (the
 * reference's tile of sequential f32 sums). */
uint64_t guffin_hip_draft_law_any_workspace_bytes(uint32_t vocab);
int guffin_hip_draft_law_any(void* stream, const float* logits, uint32_t vocab, const void* options,
                             uint64_t seed, uint64_t step, const void* injected_draws, void* workspace,
                             void* law, uint64_t* full_cdf, uint32_t* proposal, uint32_t* status);
/* One accept / residual decision (src/engine/sampling.cpp:394-499, 561-656):
 * target law p from row 0 of target_candidates (two rows of the select result), q gathered
 * from `law` on p's support, accept iff u_accept < min(1, p(x)/q(x)), else inverse-CDF draw
 * from norm(max(p-q, 0)) with u_residual; on acceptance the next root is drawn from row 1's
 * law with u_next (src/engine/chain_chat.mm:524-533).
 * result: { u32 accepted, token, next_root, status; f64 acceptance_probability,
 *           residual_total; u32 residual_count, proposal; }; status != 0 mirrors the reference's
 * throws and also sets GUFFIN_STATUS_LAW_INVALID in *status. */
int guffin_hip_spec_accept(void* stream, const void* target_candidates, const void* law,
                           const uint32_t* proposal, const void* options, uint64_t seed, uint64_t step,
                           const void* injected_draws, void* result, uint32_t* status);
/* The same decision when the law may be a full table (guffin_hip_draft_law_any): q is then
 * gathered as full_cdf[token + 1] - full_cdf[token] (src/engine/gemma3_draft.mm:1528-1581). */
int guffin_hip_spec_accept_law(void* stream, const void* target_candidates, const void* law,
                               const uint64_t* full_cdf, uint32_t vocab, const uint32_t* proposal,
                               const void* options, uint64_t seed, uint64_t step,
                               const void* injected_draws, void* result, uint32_t* status);
/* The same decision with the sampler history of each row (SamplerHistorySnapshot of the reference:
 * the tokens the repetition penalty of `options` applies to, src/engine/sampling.cpp:430-446):
 * history [2][64] token ids, history_count [2], both on the device; the candidate rows must carry
 * the history tokens' logits (guffin_hip_select_candidates with the same history). */
int guffin_hip_spec_accept_history(void* stream, const void* target_candidates, const void* law,
                                   const uint64_t* full_cdf, uint32_t vocab, const uint32_t* history,
                                   const uint32_t* history_count, const uint32_t* proposal,
                                   const void* options, uint64_t seed, uint64_t step,
                                   const void* injected_draws, void* result, uint32_t* status);

/* The drafter's vocabulary map (the reference's TLI map, src/engine/gemma3_draft.mm:648-675):
 * draft_to_target[d] = the target's id of draft token d, or -1 for a draft token the target does not
 * have; injective.  target_to_draft is its inverse over the target's vocabulary (-1 where no draft
 * token maps).  guffin_hip_draft_law_mapped is gd_process -> compact law -> gd_compact_sample with the
 * map: scores (scratch, [vocab] floats) = logits with the repetition penalty of `options` on the
 * history's tokens and -inf for unmapped draft tokens (their raw logits are validated all the same:
 * GUFFIN_STATUS_NONFINITE), the law in draft ids, the proposal in both id spaces.  workspace as for
 * guffin_hip_draft_law.  guffin_hip_spec_accept_mapped is guffin_hip_spec_accept_history with the
 * candidates and the proposal in target ids and masses gathered through target_to_draft
 * (Gemma3DraftPlan::gather, :1528-1581); NULL maps mean one shared vocabulary. */
/* Host only, no GPU call: checks a vocabulary map as the reference's drafter does when it is built
 * (src/engine/gemma3_draft.mm:655-675) and writes its inverse.  draft_to_target: draft_vocab host words;
 * target_to_draft: target_vocab host words, out.  GUFFIN_E_ARG with the reference's reasons: a target id
 * below -1 or at or beyond target_vocab ("out of bounds"), two draft tokens on one target token ("not
 * injective"), no mapped token at all ("intersection is empty"); mapped_count (may be NULL) receives the
 * number of mapped tokens. */
int guffin_vocab_map_invert(const int32_t* draft_to_target, uint32_t draft_vocab, uint32_t target_vocab,
                            int32_t* target_to_draft, uint32_t* mapped_count);
int guffin_hip_draft_law_mapped(void* stream, const float* logits, uint32_t vocab, const int32_t* draft_to_target,
                                const uint32_t* history, uint32_t history_count, const void* options,
                                uint64_t seed, uint64_t step, const void* injected_draws, void* workspace,
                                float* scores, void* law, uint32_t* draft_proposal, uint32_t* target_proposal,
                                uint32_t* status);
/* guffin_hip_draft_law_mapped by whichever path the options and the scores need (guffin_hip_draft_law_any on the
 * processed scores): the full-vocabulary kernels keep suppressed tokens (-inf) out of every sum, so a token without
 * a target id has an empty bin.  workspace: guffin_hip_draft_law_any_workspace_bytes(vocab). */
int guffin_hip_draft_law_any_mapped(void* stream, const float* logits, uint32_t vocab, const int32_t* draft_to_target,
                                    const uint32_t* history, uint32_t history_count, const void* options,
                                    uint64_t seed, uint64_t step, const void* injected_draws, void* workspace,
                                    float* scores, void* law, uint64_t* full_cdf, uint32_t* draft_proposal,
                                    uint32_t* target_proposal, uint32_t* status);
int guffin_hip_spec_accept_mapped(void* stream, const void* target_candidates, const void* law,
                                  const uint64_t* full_cdf, uint32_t vocab, const int32_t* target_to_draft,
                                  const uint32_t* history, const uint32_t* history_count,
                                  const uint32_t* proposal, const void* options, uint64_t seed, uint64_t step,
                                  const void* injected_draws, void* result, uint32_t* status);
/* Host evaluation of the draw schedule above (out: the draws struct). */
int guffin_hip_step_draws(uint64_t seed, uint64_t step, void* out_draws_host);

/* ---- block graph and one H1 cycle ---------------------------------------------------------
 * Descriptors of a Gemma-3 shaped decoder whose projection weights are wave tiles
 * (guffin_hip_repack).  All pointers are device pointers except `layers`, a host array.
 * The layer policy follows src/engine/model.cpp:607-619: layer l is local (sliding window,
 * local_base, scale 1) iff l % global_period != global_period - 1, else global. */
typedef struct guffin_layer_desc {
    int32_t dtype[7];          /* q, k, v, o, gate, up, down */
    const void* tiles[7];
    const float* norm[6];      /* attn_norm, q_norm, k_norm, post_attention_norm, ffn_norm, post_ffw_norm */
    void* ring_k; void* ring_v; /* fp16 [ring capacity][kv_heads * head_dim] */
} guffin_layer_desc;

typedef struct guffin_model_desc {
    uint32_t hidden, ffn, q_heads, kv_heads, head_dim, layer_count, vocab, sliding_window, global_period;
    float local_base, global_base, global_scale, eps;
    uint32_t ring_local, ring_global;         /* ring capacities, powers of two */
    int32_t embed_dtype; const void* embed_rows;   /* canonical [vocab] rows of `hidden` weights */
    int32_t head_dtype; const void* head_tiles;    /* the same (tied) matrix as wave tiles, may be NULL */
    const float* out_norm;
    const guffin_layer_desc* layers;
} guffin_model_desc;

/* Runs `rows` (1 or 2) contiguous tokens at absolute `position` through every block:
 * embedding * sqrt(hidden), per block the operator order of encode_gemma_target_blocks
 * (src/engine/gemma_target_runtime.cpp:13-221; drafter: src/engine/gemma3_draft.mm:888-972),
 * attention schedule of stage_contiguous_rows (:238-271), final output norm.  New K/V stay in
 * the private rows priv_k / priv_v [layer][row][kv_heads*head_dim] fp16; the rings are only read.
 * out_hidden [rows][hidden]; out_hidden_sums (group sums for the head GEMV) may be NULL. */
uint64_t guffin_hip_forward_scratch_bytes(const guffin_model_desc* model, uint32_t rows, uint32_t position);
int guffin_hip_forward_rows(void* stream, const guffin_model_desc* model, const uint32_t* tokens,
                            uint32_t rows, uint32_t position, void* scratch, uint64_t scratch_bytes,
                            void* priv_k, void* priv_v, float* out_hidden, float* out_hidden_sums,
                            uint32_t* status);
/* One pass of 1 or 2 rows of a verify tree (rows whose parent is any earlier row, siblings included): row r sits
 * at cache position base_position + depths[r] and attends the rings below base_position (through the layer's
 * window) and then the private rows its ancestor list names, its own slot last (the list of row r has depths[r] + 1
 * entries; the lists are concatenated in ancestor_lists, host memory like depths and ancestor_counts).  The rows'
 * K/V go to slots first_slot.. of priv_k / priv_v, laid out [layer][slot_count][kv_heads*head_dim] (slot_count <= 8);
 * slots written by earlier passes of the same tree are read where a list names them.  Operator order of
 * guffin_hip_forward_rows with encode_verifier_kv_store and encode_verifier_attention as separate steps
 * (metal_command_context.hpp:250, 267: the general `ancestors` form).  scratch: guffin_hip_forward_scratch_bytes(model,
 * rows, base_position + slot_count) bytes. */
int guffin_hip_forward_tree_rows(void* stream, const guffin_model_desc* model, const uint32_t* tokens, uint32_t rows,
                                 uint32_t base_position, const uint32_t* depths, const uint32_t* ancestor_lists,
                                 const uint32_t* ancestor_counts, uint32_t first_slot, uint32_t slot_count,
                                 void* scratch, uint64_t scratch_bytes, void* priv_k, void* priv_v,
                                 float* out_hidden, float* out_hidden_sums, uint32_t* status);
/* How guffin_hip_forward_rows (and so guffin_hip_h1_step, the sessions and the tickets) runs the blocks:
 * 0 (default) the resident pass for models with one KV head that fit it (measured faster there), else one
 * launch per operator; 1 always one launch per operator; 2 the resident pass for every model it covers
 * (1 or 8 KV heads of 256, hidden width <= 4096, one block length per model), else GUFFIN_E_SHAPE.  The resident pass keeps one workgroup per CU for a
 * group of blocks, gives each of the 8 XCDs one KV head (models with 8 KV heads; one XCD for a single KV
 * head) and moves a block's intermediate rows through that XCD's L2; only the two reductions of a block
 * cross XCDs.  Every wait in it is bounded by the spin limit (polls of a counter): a workgroup that gives up
 * raises GUFFIN_STATUS_SYNC in the status word and the launch still ends.  Same results as the
 * per-operator path up to fp32 summation order; a row's arithmetic does not depend on the row count in
 * the projections.  No counterpart in the reference (its command buffers are per operator).
 * The resident pass assumes this part's placement (256 CUs; a device with another CU count always runs one launch
 * per operator).  When host code of this library reads a status word with GUFFIN_STATUS_SYNC up (a session or
 * ticket completing, a drafter plan's pass), the automatic mode stops choosing the resident pass for the rest of the
 * process -- guffin_hip_resident_enabled() then returns 0 -- until guffin_hip_set_forward_mode is called again; a
 * drafter plan, whose calls are host-synchronous, also runs the pass that gave up once more, per operator. */
int guffin_hip_set_forward_mode(int mode);
int guffin_hip_resident_enabled(void);
/* Host only: where the resident pass puts the eight exchange regions of one block inside its scratch (q/k/v
 * parts, attention outputs, attention maxima and denominators, o planes, down planes, the two norm joints'
 * vectors, the GeGLU receipt), how long one block's set is, how many sets a launch has (one per block it runs,
 * so that no address is read twice in a launch) and the whole scratch.  Regions are handed over between CUs in
 * different phases, so each starts on a 256-byte boundary; tests hold the layout to that. */
int guffin_hip_resident_layout(const guffin_model_desc* model, uint32_t rows, uint64_t* offsets /* [8] */, uint64_t* bytes /* [8] */,
                               uint64_t* set_bytes, uint32_t* sets, uint64_t* total_bytes);
int guffin_hip_set_spin_limit(uint32_t polls);
/* Profiling aid: with a device buffer of 16 * blocks u64 words set, workgroup 0 of the resident pass stores the
 * 100 MHz clock at the start of each block's q/k/v projection, attention, o-projection, first norm pair,
 * gate/up, down projection, second norm pair, and at the block's end (words 0-7 of the block), and inside the
 * first norm pair after the device-wide wait, the slice sums, the XCD-wide wait and the first row sum (words
 * 8-11).  NULL (default) switches it off. */
int guffin_hip_set_resident_stamps(void* device_words);

/* Publishes private rows into the rings of every layer at slot (position + row) & mask: all
 * `rows` when accepted is NULL, else row 0 and, if *accepted != 0, row 1 (provisional commit,
 * src/engine/chain_chat.mm:473-479).  ring_k_table / ring_v_table: device arrays of the
 * per-layer ring pointers. */
int guffin_hip_commit_rows(void* stream, const guffin_model_desc* model, const void* priv_k,
                           const void* priv_v, void* const* ring_k_table, void* const* ring_v_table,
                           const uint32_t* accepted, uint32_t position, uint32_t rows);

/* ---- chunked prefill ------------------------------------------------------------------------
 * Replaces the reference's prefill matrix path (encode_verifier_matmul with allow_prefill_matrix,
 * src/tensor/backends/metal/metal_command_context.mm:384-401, kernels metal_kernels.mm:1031-1199)
 * and encode_f16_prefill_attention (metal_command_context.hpp:185, metal_kernels.mm:2593-2800).
 *
 * guffin_hip_prefill_pack turns x [M][K] fp32 into the matrix-core operand of M rows (fp16 hi/lo
 * image, per-(row, 32-group) multipliers and sums; guffin_hip_prefill_image_bytes bytes, 256-byte
 * aligned); guffin_hip_prefill_gemm multiplies it with a repacked weight matrix, y [M][N] fp32,
 * exact products and fp32 sums like the packed GEMV. */
uint64_t guffin_hip_prefill_image_bytes(uint32_t M, uint32_t K);
int guffin_hip_prefill_pack(void* stream, const float* x, void* image, uint32_t M, uint32_t K);
int guffin_hip_prefill_gemm(void* stream, int dtype, const void* tiles, const void* image, float* y,
                            uint32_t M, uint32_t K, uint32_t N);
/* Causal GQA attention of `rows` consecutive positions starting at `position`: row r sees the
 * ring for positions below `position` and rows 0..r of the run's own fp16 K/V rows
 * run_k / run_v [rows][kv_heads*head_dim]; window = 0 for global layers, else the sliding
 * window (the last `window` positions including the row's own).  q, out: [rows][q_heads*256].
 * workspace: guffin_hip_prefill_attention_workspace_bytes bytes (16-byte aligned) for the
 * transposed values of the matrix-core path (q_heads / kv_heads <= 2); NULL selects the
 * vector-unit kernel, which needs none. */
uint64_t guffin_hip_prefill_attention_workspace_bytes(uint32_t rows, uint32_t position, uint32_t window,
                                                      uint32_t kv_heads, uint32_t head_dim);
int guffin_hip_prefill_attention(void* stream, const float* q, const void* ring_k, const void* ring_v,
                                 const void* run_k, const void* run_v, float* out, uint32_t rows,
                                 uint32_t position, uint32_t window, uint32_t ring_mask,
                                 uint32_t q_heads, uint32_t kv_heads, uint32_t head_dim, float scale,
                                 void* workspace);
/* ring[(position + row) & ring_mask] = run[row] for every row of the run that a ring of this
 * capacity keeps (encode_gemma2_kv_cache_copy, metal_command_context.hpp:170). */
int guffin_hip_publish_run(void* stream, const void* run_k, const void* run_v, void* ring_k, void* ring_v,
                           uint32_t rows, uint32_t position, uint32_t ring_mask, uint32_t row_width);
/* dst[(position + t) & dst_mask] = src[(position + t) & src_mask] for t < tokens, keys and values:
 * encode_gemma2_kv_cache_copy (metal_command_context.hpp:170) with both row masks.  A mask is the
 * side's row capacity minus one (a power of two minus one; 0 = a single row).  With it a host that
 * keeps the reference's provisional protocol backs the ring rows of a verify pass up
 * (src/engine/gemma_target_runtime.cpp:473-479) and restores a rejected suffix
 * (src/engine/gemma2_runtime.cpp:756-765); guffin_hip_h1_step needs neither, it publishes after the
 * decision. */
int guffin_hip_kv_cache_copy(void* stream, const void* src_k, const void* src_v, void* dst_k, void* dst_v,
                             uint32_t position, uint32_t tokens, uint32_t src_mask, uint32_t dst_mask,
                             uint32_t row_width);
/* The block graph of guffin_hip_forward_rows for any number of rows (prompt ingestion): same
 * operator order, matrix-core GEMMs, the run's K/V published to the rings layer by layer.
 * out_hidden [rows][hidden] holds the output-normed rows. */
uint64_t guffin_hip_prefill_scratch_bytes(const guffin_model_desc* model, uint32_t rows);
int guffin_hip_prefill_rows(void* stream, const guffin_model_desc* model, const uint32_t* tokens,
                            uint32_t rows, uint32_t position, void* scratch, uint64_t scratch_bytes,
                            float* out_hidden, uint32_t* status);

/* One H1 cycle (src/engine/standalone_chat.cpp:508-615, src/engine/chain_chat.mm:245-543):
 * the drafter ingests the pending root at drafter_position, projects through its tied head,
 * builds its proposal law and picks x with the step's word; the target evaluates rows
 * [root, x] at target_position, the head produces both rows' logits, the best top_k of each
 * row are selected and row 0 decides accept / residual; the verified rows are published.
 * result: the guffin_hip_spec_accept result.  The ring tables may be NULL to skip publication. */
typedef struct guffin_h1_desc {
    const guffin_model_desc* target;
    const guffin_model_desc* drafter;
    uint32_t target_position, drafter_position;
    float temperature; uint32_t top_k; float top_p, min_p;
    uint64_t seed, step;
    void* const* target_ring_k; void* const* target_ring_v;
    void* const* drafter_ring_k; void* const* drafter_ring_v;
    uint32_t full_law;  /* != 0: encode the full-vocabulary law too (overflow fallback, top_k > 64, greedy) */
    uint32_t drafter_rows;          /* 2: the drafter first ingests *pending_token (the proposal the target
                                       accepted last cycle, src/engine/gemma3_draft.mm:1430-1449), then the root */
    const uint32_t* pending_token;  /* device; read only when drafter_rows == 2 */
    /* sampler history of the verify pass: the last <= 64 confirmed tokens, the root last (device).
     * Row 0 is sampled with the repetition penalty on these, row 1 on these plus the proposal
     * (src/engine/sampling.cpp:430-446).  NULL / 0: no penalty.  The drafter penalises the same tokens
     * before it builds its law (src/engine/gemma3_draft.mm:186-204). */
    const uint32_t* history; uint32_t history_count; float repetition_penalty;
    /* The drafter's vocabulary map and its inverse (device; see guffin_hip_draft_law_mapped): both or
     * neither.  With them the root, the pending token and the history reach the drafter in its own ids,
     * its law lives in its ids, and the proposal enters the verify pass in the target's (with either law). */
    const int32_t* draft_to_target; const int32_t* target_to_draft;
} guffin_h1_desc;
uint64_t guffin_hip_h1_scratch_bytes(const guffin_h1_desc* desc);
int guffin_hip_h1_step(void* stream, const guffin_h1_desc* desc, const uint32_t* root_token, void* scratch,
                       uint64_t scratch_bytes, void* drafter_priv_k, void* drafter_priv_v,
                       void* target_priv_k, void* target_priv_v, void* result, uint32_t* status);
/* Addresses, inside `scratch`, of the step's intermediate results (for tests and diagnostics). */
int guffin_hip_h1_buffers(const guffin_h1_desc* desc, void* scratch, float** drafter_hidden,
                          float** target_hidden, float** q_logits, float** p_logits, void** law,
                          void** candidates, uint32_t** tokens);
/* The full-vocabulary table of the last step (desc->full_law != 0), else NULL. */
int guffin_hip_h1_full_cdf(const guffin_h1_desc* desc, void* scratch, uint64_t** full_cdf);

/* ---- drafter lifecycle --------------------------------------------------------------------
 * The state machine of Gemma3DraftPlan (include/local_gguf_engine/engine/gemma3_draft.hpp:56-82;
 * lifecycle cases tests/engine/gemma3_draft_tests.cpp:206-277) over guffin_hip_forward_rows and the model's
 * rings: a prefix of `position` tokens of which `materialized` have K/V rows (a pending token, the drafter's
 * last emission or one restored by the caller, is run only when the next input needs it), and transactions
 * whose rows can be taken back.  Each call below names the method it replaces.  A transaction's rows go to
 * the rings at once; the ring rows they overwrite are saved per position and copied back by abort, truncate
 * and a commit of a shorter prefix, and the final normalised row of every position a transaction runs is kept
 * (the reference's private_norm, src/engine/gemma3_draft.mm:966-968, 984-992), so logits can be read and
 * proposals drafted at a frontier that a truncate or a shorter commit went back to.  transaction_rows is the
 * reference's constructor argument of that name (:648-657): how many positions one transaction may write, at
 * least the largest horizon + 2 = 25 and, rounded up to a power of two, at most the smallest ring; 0 = 32.
 * Tokens run through the decode path one row per pass, so a token's rows and logits do not
 * depend on how appends were grouped and a commit equals a replay bit for bit.  Every call returns when its device work is done; errors: GUFFIN_E_STATE for a call
 * the state does not admit (nested transaction, truncation of published rows, a second pending token, a
 * poisoned plan), GUFFIN_E_CAPACITY / GUFFIN_E_ARG raised before any state changes, GUFFIN_E_NUMERIC when a pass
 * raises the device status (the plan is then poisoned until reset).  The struct is caller-owned; the fields
 * after `workspace_bytes` belong to the library. */
typedef struct guffin_draft_plan {
    const guffin_model_desc* model;   /* the drafter, with head_tiles and every layer's rings */
    void* workspace; uint64_t workspace_bytes;   /* device, guffin_hip_draft_plan_bytes(model, transaction_rows), 256-byte aligned */
    uint32_t position, materialized, pending_token, has_pending, transaction_active, poisoned;
    uint32_t checkpoint_position, checkpoint_materialized, checkpoint_pending, checkpoint_has_pending;
    uint32_t backup_end, last_rows, logits_valid, hidden_valid, checkpoint_hidden_valid, checkpoint_last_rows;
    uint32_t transaction_rows, transaction_arena;
} guffin_draft_plan;
uint64_t guffin_hip_draft_plan_bytes(const guffin_model_desc* model, uint32_t transaction_rows);   /* 0: not a model or a capacity a plan can have */
int guffin_hip_draft_plan_init(void* stream, guffin_draft_plan* plan, const guffin_model_desc* model, void* workspace,
                               uint64_t workspace_bytes, uint32_t transaction_rows);
int guffin_hip_draft_plan_reset(void* stream, guffin_draft_plan* plan);                        /* reset() */
int guffin_hip_draft_plan_begin_transaction(void* stream, guffin_draft_plan* plan);                        /* begin_transaction() */
int guffin_hip_draft_plan_commit_prefix(void* stream, guffin_draft_plan* plan, uint32_t position);   /* commit_prefix() */
int guffin_hip_draft_plan_abort_transaction(void* stream, guffin_draft_plan* plan);            /* abort_transaction() */
int guffin_hip_draft_plan_can_truncate(const guffin_draft_plan* plan, uint32_t position);      /* can_truncate(): 1 or 0 */
int guffin_hip_draft_plan_truncate(void* stream, guffin_draft_plan* plan, uint32_t position);  /* truncate() */
int guffin_hip_draft_plan_append(void* stream, guffin_draft_plan* plan, const uint32_t* tokens_host, uint32_t count);  /* append() */
int guffin_hip_draft_plan_restore_pending_token(guffin_draft_plan* plan, uint32_t token);     /* restore_pending_token() */
/* propose(): `horizon` (1..23) tokens from the given 32-bit words inside the open transaction; all but the last
 * are run, the last stays pending.  options: the sampler options struct; history (host, <= 64 tokens, may be
 * NULL) feeds the repetition penalty and grows by the drafted tokens.  drafted: host, `horizon` tokens. */
int guffin_hip_draft_plan_propose(void* stream, guffin_draft_plan* plan, const uint32_t* words_host, uint32_t horizon,
                                  const void* options, const uint32_t* history_host, uint32_t history_count,
                                  uint32_t* drafted_host);
int guffin_hip_draft_plan_read_logits(void* stream, guffin_draft_plan* plan, float* logits_host);   /* read_logits() */
/* read_cache(): fp16 rows of `count` materialized positions of one layer, in position order. */
int guffin_hip_draft_plan_read_cache(void* stream, const guffin_draft_plan* plan, uint32_t layer, uint32_t first_position,
                                     uint32_t count, void* keys_host, void* values_host);

/* ---- GGUF container reader (host only) ---------------------------------------------------
 * The validating reader of src/model_format/gguf_reader.cpp (types in
 * include/local_gguf_engine/model_format/gguf_{header,metadata,tensor,reader}.hpp): one pass over
 * the caller's bytes up to `stage` — the depths the reference exposes as read_gguf_header,
 * read_gguf_metadata_section, read_gguf_tensor_directory and read_gguf_model_view.  The handle
 * keeps keys, names and scalar values; tensor payloads are (file_offset, byte_count) views into
 * the caller's bytes, which must outlive the handle.  guffin_gguf_open returns 0, a GUFFIN_E_*
 * argument error, or one of the reader's error codes below (GGUFReadErrorCode, same order), with
 * the reference's expected / actual counts and the offending magic from guffin_gguf_last_failure
 * (per thread).  Tensor types: 0 F32, 1 F16, 8 Q8_0, 12 Q4_K, 14 Q6_K; names up to 64 bytes, up to
 * 4 dimensions, general.alignment a non-zero uint32 multiple of 8 (default 32), zero padding. */
#define GUFFIN_GGUF_TRUNCATED_HEADER (-100)
#define GUFFIN_GGUF_INVALID_MAGIC (-101)
#define GUFFIN_GGUF_TRUNCATED_METADATA (-102)
#define GUFFIN_GGUF_INVALID_METADATA_VALUE_TYPE (-103)
#define GUFFIN_GGUF_INVALID_METADATA_VALUE (-104)
#define GUFFIN_GGUF_UNSUPPORTED_METADATA_VALUE_TYPE (-105)
#define GUFFIN_GGUF_TRUNCATED_TENSOR_DIRECTORY (-106)
#define GUFFIN_GGUF_INVALID_TENSOR_DIMENSION_COUNT (-107)
#define GUFFIN_GGUF_INVALID_TENSOR_NAME (-108)
#define GUFFIN_GGUF_INVALID_ALIGNMENT (-109)
#define GUFFIN_GGUF_INVALID_TENSOR_OFFSET (-110)
#define GUFFIN_GGUF_INVALID_TENSOR_PADDING (-111)
#define GUFFIN_GGUF_TRUNCATED_TENSOR_PAYLOAD (-112)
#define GUFFIN_GGUF_UNSUPPORTED_TENSOR_TYPE (-113)
#define GUFFIN_GGUF_INVALID_TENSOR_SIZE (-114)
#define GUFFIN_GGUF_STAGE_HEADER 0
#define GUFFIN_GGUF_STAGE_METADATA 1
#define GUFFIN_GGUF_STAGE_DIRECTORY 2
#define GUFFIN_GGUF_STAGE_MODEL 3
typedef struct guffin_gguf guffin_gguf;
typedef struct guffin_gguf_info {
    uint32_t version, alignment;
    uint64_t tensor_count, metadata_kv_count;   /* as the header states them */
    uint64_t metadata_end_offset, tensor_infos_end_offset, padding_byte_count, tensor_data_start_offset;
    uint64_t parsed_entries, parsed_tensors;    /* what this handle holds for its stage */
} guffin_gguf_info;
typedef struct guffin_gguf_entry_info {
    const char* key;
    uint32_t type, element_type;   /* GGUFMetadataValueType; element_type for arrays (type 9) */
    uint64_t bits;                 /* scalars: the little-endian value (floats by bit pattern, bool 0 / 1) */
    const char* text; uint64_t text_bytes;   /* strings (type 8) */
    uint64_t count;                /* arrays: number of elements */
} guffin_gguf_entry_info;
typedef struct guffin_gguf_tensor_info {
    const char* name;
    uint32_t n_dims, type_id;
    uint64_t dims[4];
    uint64_t offset, file_offset, byte_count;   /* byte_count is set from GUFFIN_GGUF_STAGE_MODEL on */
} guffin_gguf_tensor_info;
int guffin_gguf_open(const void* bytes, uint64_t size, int stage, guffin_gguf** out);
void guffin_gguf_close(guffin_gguf* gguf);
void guffin_gguf_last_failure(uint64_t* expected, uint64_t* actual, uint8_t magic[4]);
int guffin_gguf_summary(const guffin_gguf* gguf, guffin_gguf_info* out);
int guffin_gguf_entry(const guffin_gguf* gguf, uint64_t index, guffin_gguf_entry_info* out);
int guffin_gguf_entry_element(const guffin_gguf* gguf, uint64_t index, uint64_t element, uint64_t* bits,
                              const char** text, uint64_t* text_bytes);
int guffin_gguf_find_entry(const guffin_gguf* gguf, const char* key, uint64_t* index);
int guffin_gguf_tensor(const guffin_gguf* gguf, uint64_t index, guffin_gguf_tensor_info* out);
int guffin_gguf_find_tensor(const guffin_gguf* gguf, const char* name, uint64_t* index);

/* Weight binding of a Gemma 3 shaped file: bind_gemma_model_weights + validate_gemma3_model_weights
 * (src/engine/gemma_model.cpp:72-177).  Every tensor the block graph needs is looked up by its GGUF name
 * (token_embd, output_norm, output or the tied embedding, per block the 7 matrices and 6 norms) and checked
 * against the configuration: norms F32 of the right width, matrices native block formats of shape
 * [input, output] with input a whole number of blocks.  As in the reference every name is looked up before
 * anything is validated (blocks first, in the order of its initialisers), so a missing tensor is reported
 * whatever else is wrong; validation then follows the reference's order (configuration, token_embd, output,
 * output_norm, blocks).  uses_tied_output_weight is what the reference's loader sets when the file has no
 * output.weight (src/engine/model.cpp:328).  target_geometry is the caller's statement of what the file is:
 * != 0 adds the target's rules (:120-124, :150-158): 256-wide heads, two query heads per KV head, at most 64 blocks, Q4_K / Q6_K matrices, a Q6_K head;
 * without it the drafter's geometry and Q8_0 blocks are admitted (one block length per block).  Returns 0 and the
 * tensor indices (for guffin_gguf_tensor), GUFFIN_BIND_MISSING_TENSOR (EngineModelErrorCode::missing_tensor) or
 * GUFFIN_BIND_INVALID_TENSOR (::invalid_tensor) with the reference's detail string from guffin_gguf_bind_detail
 * (per thread).  `blocks`: caller array of block_count records. */
#define GUFFIN_BIND_MISSING_TENSOR (-120)
#define GUFFIN_BIND_INVALID_TENSOR (-121)
typedef struct guffin_gemma3_config {   /* the GemmaModelConfig fields the validation reads */
    uint32_t block_count, embedding_length, feed_forward_length, vocab_size;
    uint32_t attention_head_count, attention_head_count_kv, attention_key_length, attention_value_length;
    uint32_t sliding_window, context_length, attention_global_layer_period;
    uint32_t uses_qk_norm, uses_tied_output_weight, target_geometry;
    float rms_norm_epsilon, attention_logit_softcap, final_logit_softcap;
    float rope_freq_base, local_rope_freq_base, rope_freq_scale;
} guffin_gemma3_config;
typedef struct guffin_gemma3_block {
    uint64_t matrix[7];    /* q, k, v, o, gate, up, down */
    uint64_t norm[6];      /* attn_norm, attn_q_norm, attn_k_norm, post_attention_norm, ffn_norm, post_ffw_norm */
    uint32_t type_id[7]; uint32_t pad;
} guffin_gemma3_block;
typedef struct guffin_gemma3_binding { uint64_t token_embedding, output_norm, output; uint32_t tied_output, pad; } guffin_gemma3_binding;
int guffin_gguf_bind_gemma3(const guffin_gguf* gguf, const guffin_gemma3_config* config, guffin_gemma3_binding* binding,
                            guffin_gemma3_block* blocks);
const char* guffin_gguf_bind_detail(void);

/* ---- consecutive cycles ---------------------------------------------------------------------
 * Host-side lifecycle around guffin_hip_h1_step for generation over many cycles.  It keeps what
 * the reference keeps between cycles: the verify pass's transaction state (VerifierTransactionState,
 * include/local_gguf_engine/engine/gemma2_metal_plan.hpp:208-215: idle -> submitted -> idle, or
 * poisoned for good once the device status word is raised), the positions of both caches, and the
 * drafter's pending token (include/local_gguf_engine/engine/gemma3_draft.hpp:61-63,
 * src/engine/gemma3_draft.mm:1430-1486): the proposal of a cycle is not in the drafter's cache; if
 * the target accepted it, the next cycle's drafter pass ingests it together with the new root.
 *
 * The caller fills desc (models, sampler, seed, the four ring tables, full_law) and every device
 * pointer below, then calls start once and submit / complete per cycle.  complete blocks on the
 * stream, reads 20 bytes back and reports the tokens the cycle confirmed: {proposal, next root} on
 * acceptance, {residual token} on rejection; the last one is the next cycle's root. */
#define GUFFIN_TXN_IDLE 0u
#define GUFFIN_TXN_SUBMITTED 2u
#define GUFFIN_TXN_POISONED 5u
typedef struct guffin_h1_session {
    guffin_h1_desc desc;
    void* scratch; uint64_t scratch_bytes;   /* device arena, >= guffin_hip_session_scratch_bytes */
    void* drafter_priv_k; void* drafter_priv_v;   /* device, [blocks][2][kv width] fp16 each */
    void* target_priv_k; void* target_priv_v;
    uint32_t* tokens;                        /* device u32[2]: root, pending */
    void* result;                            /* device, one result record (guffin_hip_spec_accept) */
    uint32_t* status;                        /* device status word */
    uint32_t state;                          /* GUFFIN_TXN_* */
    uint32_t root, pending, has_pending;
    uint64_t cycles, accepted;
} guffin_h1_session;
/* Arena size that covers every cycle up to the given cache positions. */
uint64_t guffin_hip_session_scratch_bytes(const guffin_h1_session* session, uint32_t last_target_position,
                                          uint32_t last_drafter_position);
int guffin_hip_session_start(guffin_h1_session* session, uint32_t root_token, uint32_t target_position,
                             uint32_t drafter_position);
int guffin_hip_session_submit(void* stream, guffin_h1_session* session);
int guffin_hip_session_complete(void* stream, guffin_h1_session* session, uint32_t* emitted /* [2] */,
                                uint32_t* emitted_count);

/* ---- the verify pass as a transaction ---------------------------------------------------------
 * The reference's TargetVerificationTicket (include/local_gguf_engine/engine/target_verifier.hpp:
 * 366-412) with its free functions (src/engine/target_verifier_runtime.cpp): encode :349-445,
 * submit :447-463, complete :465-533, provisionally_commit :535-609, finalize :611-673, discard
 * :675-688, and the destructor's rules :315-335 as release.  States are VerifierTransactionState
 * (include/local_gguf_engine/engine/gemma2_metal_plan.hpp:208-215):
 *
 *   idle -encode-> encoded -submit-> submitted -complete-> completed -provisional_commit->
 *   provisional -finalize-> idle;   discard: encoded / completed -> idle, provisional -> finalize(0)
 *
 * A pass runs 1 or 2 contiguous rows (row r's parent is row r - 1) through the target, its head and
 * the candidate selection; its K/V stay in the private rows.  provisional_commit(path) backs the ring
 * rows at position .. position + count - 1 of every layer up into the backup rows and publishes the
 * selected private rows there; finalize(retained) keeps the first `retained` of them and restores
 * the others.  The only causal paths of a chain are {0} and {0, 1}.  Errors follow the reference:
 * a call out of order returns GUFFIN_E_STATE and changes nothing (std::logic_error there); a bad
 * path or row count GUFFIN_E_ARG (std::invalid_argument); a raised device status word drops the
 * transaction (idle again, the caches untouched) and returns GUFFIN_E_NUMERIC; a failed wait, or a
 * failure after the first ring row was written, poisons the ticket for good.
 *
 * The caller fills the first block of fields once (state = GUFFIN_TXN_IDLE); the library keeps the
 * second.  After complete, `candidates` holds one record per row (guffin_hip_select_candidates). */
#define GUFFIN_TXN_ENCODED 1u
#define GUFFIN_TXN_COMPLETED 3u
#define GUFFIN_TXN_PROVISIONAL 4u
#define GUFFIN_TICKET_MAX_ROWS 4u
typedef struct guffin_verify_ticket {
    const guffin_model_desc* target;         /* with head_tiles */
    void* scratch; uint64_t scratch_bytes;   /* device arena, >= guffin_hip_ticket_scratch_bytes */
    void* priv_k; void* priv_v;              /* device, [blocks][rows][kv width] fp16: the pass's own rows */
    void* backup_k; void* backup_v;          /* device, [blocks][4][kv width] fp16: ring rows a commit overwrites */
    uint32_t* tokens;                        /* device u32[4]: the rows' tokens */
    uint32_t* selected;                      /* device u32[4]: the selected path */
    void* candidates;                        /* device, 4 candidate records */
    uint32_t* status;                        /* device u32[5]: the pass's status word, one selection status per row */
    uint32_t retain;                         /* candidates kept per row (top_k), 1..320 */
    uint32_t state;                          /* GUFFIN_TXN_* */
    uint32_t rows, position, provisional_count;
    uint32_t provisional_path[GUFFIN_TICKET_MAX_ROWS];
    uint32_t row_tokens[GUFFIN_TICKET_MAX_ROWS];
    uint32_t parents[GUFFIN_TICKET_MAX_ROWS];   /* row r's parent row (row 0: GUFFIN_TICKET_ROOT); a chain has r - 1 */
    uint32_t depths[GUFFIN_TICKET_MAX_ROWS];    /* row r sits at cache position `position` + depths[r] */
} guffin_verify_ticket;
#define GUFFIN_TICKET_ROOT 0xFFFFFFFFu
/* Arena size that covers every pass up to the given cache position. */
uint64_t guffin_hip_ticket_scratch_bytes(const guffin_verify_ticket* ticket, uint32_t last_position);
/* Host only: validates and records the pass (row tokens are host memory).  A chain of 1 or 2 rows. */
int guffin_hip_ticket_encode(guffin_verify_ticket* ticket, const uint32_t* row_tokens, uint32_t rows, uint32_t position);
/* The same for a tree of up to 4 rows in topological order (VerifierTopologyDescriptor,
 * include/local_gguf_engine/engine/target_verifier.hpp): parents[0] = GUFFIN_TICKET_ROOT, parents[r] < r.  Row r is
 * verified at cache position `position` + its depth and attends the ring and its ancestors among the rows.  A chain
 * of 1 or 2 rows runs as guffin_hip_ticket_encode runs it (one pass); any other tree runs in passes of 2 rows
 * through guffin_hip_forward_tree_rows.  guffin_hip_ticket_provisional_commit then takes any root-to-node path. */
int guffin_hip_ticket_encode_tree(guffin_verify_ticket* ticket, const uint32_t* row_tokens, const uint32_t* parents,
                                  uint32_t rows, uint32_t position);
int guffin_hip_ticket_submit(void* stream, guffin_verify_ticket* ticket);
/* Blocks on the stream.  device_status (may be NULL) receives the OR of the status words. */
int guffin_hip_ticket_complete(void* stream, guffin_verify_ticket* ticket, uint32_t* device_status);
int guffin_hip_ticket_provisional_commit(void* stream, guffin_verify_ticket* ticket, const uint32_t* path, uint32_t count);
int guffin_hip_ticket_finalize(void* stream, guffin_verify_ticket* ticket, uint32_t retained);
int guffin_hip_ticket_discard(void* stream, guffin_verify_ticket* ticket);
/* What the reference's destructor does: encoded / completed are dropped, a provisional commit is
 * rolled back, a submitted pass poisons the ticket.  Never fails. */
int guffin_hip_ticket_release(void* stream, guffin_verify_ticket* ticket);

/* ---- recorded launch chains ---------------------------------------------------------------------------------
 * The command buffer of the reference: MetalCommandContext encodes a whole pass and commits it once
 * (src/tensor/backends/metal/metal_command_context.hpp:346-353, commit / wait_until_completed / commit_and_wait).
 * Between guffin_hip_chain_begin(stream, ..) and guffin_hip_chain_end every kernel this library would enqueue on
 * `stream` is recorded instead of run (guffin_hip_h1_step, guffin_hip_forward_rows, .. are called as usual; calls
 * that copy or synchronise are not recordable); guffin_hip_chain_launch replays the recorded launches as AQL dispatch
 * packets on a hardware queue of the library's own and returns at once, guffin_hip_chain_wait blocks until every
 * replay has completed.  Buffers and arguments are the recorded ones: a replay reads its inputs (root token, step
 * draws) from device memory.  Every packet carries the barrier bit and agent-scope fences, the last one a
 * system-scope release: the order and visibility of a stream, and the results of the same calls made directly, bit
 * for bit.  guffin_hip_chain_launch first waits for the work already enqueued on `stream`; work enqueued on any HIP
 * stream afterwards is not ordered after the replay: call guffin_hip_chain_wait first.  One chain records at a time;
 * begin / end allocate (kernel arguments), launch and wait do not. */
int guffin_hip_chain_begin(void* stream, void** chain);
int guffin_hip_chain_end(void* chain);
int guffin_hip_chain_launch(void* chain);
int guffin_hip_chain_wait(void* chain);
/* Device time of the last replay in nanoseconds, first dispatch's start to last dispatch's end: MetalCommandStats'
 * gpu_duration_ns (metal_command_context.hpp:19-45).  After guffin_hip_chain_wait. */
int guffin_hip_chain_gpu_ns(void* chain, uint64_t* nanoseconds);
/* launches recorded */
int guffin_hip_chain_info(void* chain, uint32_t* launches);
int guffin_hip_chain_destroy(void* chain);

#ifdef __cplusplus
}
#endif
#endif /* GUFFIN_HIP_H */
