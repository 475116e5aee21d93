/*
 * CPU oracle for the H1 speculative decode step — TEST INFRASTRUCTURE ONLY.
 *
 * This library restates, in plain scalar C++, the arithmetic of the reference
 * engine's CPU path for the hot path.  It exists to check the HIP kernels; it
 * is never linked, loaded or called by the shipped library (libguffin_hip.so)
 * and the product fails loudly when its HIP code object is missing rather than
 * falling back to anything here.  Only tests/, __graft_entry__.smoke() and the
 * cpu_baseline leg of bench.py may use it.
 *
 * Every function cites the reference file:line it follows (paths relative to
 * the reference checkout).  Pinning status per function group:
 *
 *   dequant q8_0/q4_k/q6_k   pinned: reference KAT values + hex fixtures +
 *                            compiled reference (oracle/_ref) on random blocks
 *   gemv (sequential fp32)   pinned: compiled reference dot_q*_row_f32 (bit equal),
 *                            unit-vector linearity, brute-force double dot
 *   rms_norm / head norm     pinned: compiled reference rms_norm_f32 (bit equal)
 *   rope (neox, double angle)pinned: compiled reference (scale 1) + closed form
 *   f32->f16 RNE             pinned: the reference's 28 bit cases + numpy
 *   attention                pinned: compiled reference scores/softmax/values composition
 *                            at softcap->large, uniform-K and single-token closed forms
 *   gelu_tanh * up           pinned: compiled reference gelu_tanh_f32 x multiply_f32
 *   top-k selection          pinned: std::partial_sort brute force + reference tie KAT
 *   prepare_token_distribution, speculative law, select:
 *                            pinned: compiled reference sampling.cpp (bit equal) and
 *                            the reference's exact fixtures (lossless_sampling_tests)
 *   compact draft law (u64 CDF): PARITY UNPINNED at the bit level — the reference has
 *                            no CPU implementation (Metal only, tested to 1e-6); this
 *                            file defines the CPU law following gemma3_draft.mm:247-294
 *                            and pins it by invariants (sum 2^32, monotone, uniform ->
 *                            equal bins, top-p 0.5 case, 1e-6 vs double softmax).
 *   vocabulary map (mapped law, mass gather, mapped accept):
 *                            pinned: the reference's mapped case as data (gemma3_draft_tests.cpp:
 *                            404-425: support {12, 511}, half the mass each, proposals 50000 / 511,
 *                            zero mass for the excluded and the unmapped token, NaN refusal); the
 *                            law's edges share the compact law's note above
 *   philox4x32-10            pinned: Random123 known-answer vectors
 */
#pragma once
#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum { GFO_Q8_0 = 0, GFO_Q4_K = 1, GFO_Q6_K = 2 };

/* ---- scalars ---------------------------------------------------------- */
float gfo_f16_to_f32(uint16_t bits);
uint16_t gfo_f32_to_f16_rne(float value);
float gfo_exp_f32(float x); /* deterministic IEEE-only expf used by the draft law */

/* ---- block decode ----------------------------------------------------- */
uint32_t gfo_block_bytes(int dtype);
uint32_t gfo_block_elems(int dtype);
void gfo_dequant(int dtype, const uint8_t* blocks, uint64_t n_blocks, float* out);

/* ---- GEMV: y[r,n] = sum_k x[r,k] * W[k,n], sequential fp32 from 0.0f ---- */
void gfo_gemv(int dtype, const uint8_t* w, const float* x, float* y,
              uint32_t rows, uint32_t K, uint32_t N);
/* same arithmetic per output, columns split over `threads` host threads */
void gfo_gemv_mt(int dtype, const uint8_t* w, const float* x, float* y,
                 uint32_t rows, uint32_t K, uint32_t N, uint32_t threads);
/* as-written variant: rebuilds a bounds-checked block view per element */
void gfo_gemv_as_written(int dtype, const uint8_t* w, const float* x, float* y,
                         uint32_t rows, uint32_t K, uint32_t N);

/* ---- small ops -------------------------------------------------------- */
void gfo_rms_norm(const float* x, const float* gamma, float* y,
                  uint32_t rows, uint32_t width, float eps);
void gfo_rms_norm_add(const float* x, const float* gamma, const float* residual, float* y,
                      uint32_t rows, uint32_t width, float eps);
void gfo_head_rms_norm(const float* x, const float* gamma, float* y,
                       uint32_t rows, uint32_t heads, uint32_t head_dim, float eps);
void gfo_rope_neox(const float* in, float* out, const uint32_t* positions,
                   uint32_t rows, uint32_t heads, uint32_t head_dim, uint32_t rope_dim,
                   float freq_base, float freq_scale);
void gfo_kv_store_f16(const float* raw_k, const float* raw_v, const uint32_t* positions,
                      uint16_t* out_k, uint16_t* out_v, uint32_t rows, uint32_t heads,
                      uint32_t head_dim, uint32_t rope_dim, float freq_base, float freq_scale);
void gfo_geglu(const float* gate, const float* up, float* out, uint64_t n);
void gfo_embed(int dtype, const uint8_t* w, const uint32_t* tokens, float* out,
               uint32_t rows, uint32_t width, float scale);

/* Attention over an fp16 cache.  schedule = 4 u32 per row:
 * {base_first_position, base_token_count, ancestor_offset, ancestor_count}.
 * Tokens [0, base_count) come from ring slot (base_first+t)&row_mask, the rest
 * from private rows ancestors[ancestor_offset + i]. */
void gfo_attention(const float* q, const uint16_t* ring_k, const uint16_t* ring_v,
                   const uint16_t* priv_k, const uint16_t* priv_v,
                   const uint32_t* schedule, const uint32_t* ancestors, float* out,
                   uint32_t rows, uint32_t row_mask, uint32_t q_heads, uint32_t kv_heads,
                   uint32_t head_dim, float scale);

/* ---- head selection ---------------------------------------------------- */
typedef struct { uint32_t token; float logit; } gfo_token_logit;
uint32_t gfo_argmax(const float* logits, uint32_t vocab);
/* top `k` by (logit desc, token asc) followed by the logits of `history` tokens
 * (`k` is the reference's base_candidate_count = top_k + history_count);
 * returns the candidate count, or -1 if a selected logit is not finite. */
int gfo_select_candidates(const float* logits, uint32_t vocab, uint32_t k,
                          const uint32_t* history, uint32_t history_count,
                          gfo_token_logit* out);

/* ---- selection requests ------------------------------------------------ */
/* One verify row's raw sampler history (a ring of `history_window_limit` slots, oldest at
 * `history_head`) plus the hypothetical suffix of tokens before that row, and what the selection
 * needs of it: the window after appending the suffix, without duplicates, first occurrence first.
 * Layouts: VerifierDeviceSelectionRow (include/local_gguf_engine/engine/target_verifier.hpp:114-121)
 * and VerifierResolvedSelectionRow (src/tensor/backends/metal/metal_kernels.mm:91-97). */
typedef struct {
    uint32_t history_token_ids[64]; uint32_t suffix_token_ids[23];
    uint32_t history_head, history_length, history_window_limit, suffix_count;
} gfo_selection_row;
typedef struct {
    uint32_t top_k, base_candidate_count, history_count, reserved; uint32_t history_token_ids[64];
} gfo_resolved_row;
/* append_sampler_history + make_token_selection_request (src/engine/sampling.cpp:329-378) with the
 * status bits of the device version (metal_kernels.mm:2351-2371): 2 for a malformed row (the host
 * version throws), 4 for a token outside the vocabulary (it is skipped).  Returns the status bits. */
uint32_t gfo_selection_request(const gfo_selection_row* raw, uint32_t vocab, uint32_t top_k,
                               int repetition_enabled, gfo_resolved_row* out);

/* ---- sampling law ------------------------------------------------------ */
typedef struct {
    float temperature; uint32_t top_k; float top_p; float min_p; float repetition_penalty;
} gfo_sampler_options;

typedef struct {
    uint32_t count; uint32_t pad;
    double total_sampling_weight;
    uint32_t token[256];
    double probability[256];
    double sampling_weight[256];
} gfo_prepared;

/* returns 0 or a negative error code mirroring the reference's throws */
int gfo_prepare_token_distribution(const gfo_token_logit* cands, uint32_t n,
                                   const gfo_sampler_options* opt,
                                   const uint32_t* history, uint32_t history_count,
                                   gfo_prepared* out);

typedef struct {
    uint32_t count; uint32_t pad;
    uint32_t ids[256];      /* ascending token id */
    uint64_t cdf[257];      /* cdf[0]=0 ... cdf[count]=2^32 */
} gfo_draft_law;

/* compact (top_k<=64) proposal law from full-vocabulary drafter logits.
 * returns 0, 1 if the support overflowed 256 entries (full path needed),
 * negative on invalid input. */
int gfo_draft_law_compact(const float* logits, uint32_t vocab, const gfo_sampler_options* opt,
                          gfo_draft_law* out);
int gfo_draft_law_compact_mapped(const float* logits, uint32_t vocab, const gfo_sampler_options* opt,
                                 const int32_t* draft_to_target, gfo_draft_law* out);
/* full-vocabulary law: cdf has vocab+1 entries */
int gfo_draft_law_full(const float* logits, uint32_t vocab, const gfo_sampler_options* opt,
                       uint64_t* cdf);
int gfo_draft_law_full_mapped(const float* logits, uint32_t vocab, const gfo_sampler_options* opt,
                              const int32_t* draft_to_target, uint64_t* cdf);
uint32_t gfo_draft_select(const gfo_draft_law* law, uint32_t word);
uint32_t gfo_draft_select_full(const uint64_t* cdf, uint32_t vocab, uint32_t word);

typedef struct {
    uint32_t accepted; uint32_t token; uint32_t next_root; uint32_t status;
    double acceptance_probability; double residual_total; uint32_t residual_count; uint32_t pad;
} gfo_spec_result;

/* accept/residual decision from an already prepared target law */
int gfo_spec_from_prepared(const gfo_prepared* target, const gfo_draft_law* law,
                           uint32_t proposal, double u_accept, double u_residual,
                           gfo_spec_result* out);
/* one lossless accept/residual decision + next-root draw (see gfo_sampling.cpp) */
int gfo_spec_accept(const gfo_token_logit* row0, uint32_t n0,
                    const gfo_token_logit* row1, uint32_t n1,
                    const gfo_draft_law* law, uint32_t proposal,
                    const gfo_sampler_options* opt,
                    double u_accept, double u_residual, double u_next,
                    gfo_spec_result* out);
/* the same decision with a sampler history per row (repetition penalty on those tokens) */
int gfo_spec_accept_history(const gfo_token_logit* row0, uint32_t n0, const uint32_t* history0, uint32_t count0,
                            const gfo_token_logit* row1, uint32_t n1, const uint32_t* history1, uint32_t count1,
                            const gfo_draft_law* law, uint32_t proposal, const gfo_sampler_options* opt,
                            double u_accept, double u_residual, double u_next, gfo_spec_result* out);
/* the same decision with q gathered from a full-vocabulary table (cdf: vocab+1 entries) */
/* the same with the drafter's vocabulary map: `law` is in draft ids, `proposal` and the rows in target
 * ids, target_to_draft[t] = the draft id of target token t or -1 (gemma3_draft.mm:659-671, 1570-1578) */
uint64_t gfo_law_mass_mapped(const gfo_draft_law* law, const int32_t* target_to_draft, uint32_t token, uint64_t* begin);
int gfo_spec_accept_mapped(const gfo_token_logit* row0, uint32_t n0, const uint32_t* history0, uint32_t count0,
                           const gfo_token_logit* row1, uint32_t n1, const uint32_t* history1, uint32_t count1,
                           const gfo_draft_law* law, const int32_t* target_to_draft, uint32_t proposal,
                           const gfo_sampler_options* opt, double u_accept, double u_residual, double u_next,
                           gfo_spec_result* out);
int gfo_spec_accept_full_mapped(const gfo_token_logit* row0, uint32_t n0, const gfo_token_logit* row1,
                                uint32_t n1, const uint64_t* cdf, uint32_t vocab, const int32_t* target_to_draft,
                                uint32_t proposal, const gfo_sampler_options* opt, double u_accept,
                                double u_residual, double u_next, gfo_spec_result* out);
int gfo_spec_accept_full(const gfo_token_logit* row0, uint32_t n0, const gfo_token_logit* row1,
                         uint32_t n1, const uint64_t* cdf, uint32_t vocab, uint32_t proposal,
                         const gfo_sampler_options* opt, double u_accept, double u_residual,
                         double u_next, gfo_spec_result* out);

void gfo_philox4x32_10(const uint32_t counter[4], const uint32_t key[2], uint32_t out[4]);
/* draws of one H1 step: word, u_accept, u_residual, u_next */
void gfo_step_draws(uint64_t seed, uint64_t step, uint32_t* word,
                    double* u_accept, double* u_residual, double* u_next);

/* ---- whole-model forward (synthetic Gemma-3 shaped stacks) -------------- */
typedef struct {
    uint32_t hidden, ffn, q_heads, kv_heads, head_dim, layers, vocab;
    uint32_t sliding_window, global_period;   /* layer is local iff l % period != period-1 */
    float local_base, global_base, global_scale, eps;
    uint32_t ring_local, ring_global;         /* ring capacities (powers of two) */
} gfo_model_config;

typedef struct {
    int dtype[7];                 /* q,k,v,o,gate,up,down */
    const uint8_t* w[7];
    const float* norm[6];         /* attn_norm, q_norm, k_norm, post_attn, ffn_norm, post_ffn */
    uint16_t* ring_k; uint16_t* ring_v;
} gfo_layer;

/* Runs `rows` contiguous tokens starting at `position` through the stack (reads the
 * fp16 rings for the prefix, keeps new K/V private), leaves the final-normed hidden
 * rows in out_hidden [rows, hidden].  priv_k/priv_v: [layers][rows][kv_heads*head_dim]. */
void gfo_forward_rows(const gfo_model_config* cfg, const gfo_layer* layers,
                      int embed_dtype, const uint8_t* embed_w, const float* out_norm,
                      const uint32_t* tokens, uint32_t rows, uint32_t position,
                      uint16_t* priv_k, uint16_t* priv_v, float* out_hidden,
                      uint32_t threads);

#ifdef __cplusplus
}
#endif
