// Translation unit for the syntax check of include/guffin_hip_command_context.hpp: every method the
// engine of the reference calls on its command context (metal_command_context.hpp:56-364) is named here
// with the reference's own argument types, so a signature that drifts from the reference fails to compile.
// The two workspace structs repeat the member names of engine::Gemma2MetalSelectionWorkspace and
// engine::TargetSelectionWorkspace, whose headers need a macOS-only include.
#include "guffin_hip_command_context.hpp"

#include <type_traits>

namespace lge = local_gguf_engine;
namespace hipctx = lge::tensor::backends::hip;
using lge::tensor::BackendBuffer;

struct SelectionWorkspace {
    BackendBuffer candidate_runs_a, candidate_runs_b, compact_result, history_token_staging;
};
struct TargetWorkspace {
    BackendBuffer logits_tile, candidate_runs_a, candidate_runs_b, compact_results, raw_request_staging,
        resolved_request_staging, history_token_staging;
    std::uint32_t row_capacity = 0, batch_row_capacity = 0;
};

static_assert(!std::is_copy_constructible_v<hipctx::HipCommandContext>);
static_assert(sizeof(guffin_selection_row) == 364 && sizeof(guffin_resolved_row) == 272);

void drive(const BackendBuffer& a, const BackendBuffer& b, const BackendBuffer& c, const BackendBuffer& d,
           const BackendBuffer& e, const BackendBuffer& f, const BackendBuffer& g, const BackendBuffer& h,
           const SelectionWorkspace& selection, const TargetWorkspace& target,
           const lge::engine::TokenSamplerOptions& options) {
    hipctx::HipCommandContext context("probe", /*concurrent_compute=*/false, /*precise_math=*/true);
    const std::uint32_t words[2] = {1, 2};
    context.restart();
    context.write_u32(a, 7U);
    context.write_u32s(a, 0U, words);
    context.encode_embedding(a, b, c, 1.0F, 0U, 2U);
    context.encode_verifier_matmul(a, b, c, 2U, false, &d);
    context.encode_verifier_matmul(a, b, c, 2U);
    context.encode_target_head_rows(a, 0U, b, c, 2U);
    context.encode_head_rms_norm(a, b, c, 1e-6F, 2U, 16U, 256U);
    context.encode_rms_norm(a, b, c, 1e-6F, 2U, 0U, &d);
    context.encode_rms_norm(a, b, c, 1e-6F);
    context.encode_rms_norm_add(a, b, c, d, 1e-6F, 2U);
    context.encode_verifier_rope(a, b, c, 2U, 16U, 256U, 256U, 1e6F, 0.125F);
    context.encode_verifier_kv_store(a, b, c, d, e, 2U, 8U, 256U, 256U, 1e6F, 1.0F, &f);
    context.encode_verifier_attention(a, b, c, d, e, f, 0U, g, h, a, b, c, 2U, 1023U, 16U, 8U, 256U, 256U, 0.0625F, 0.0F, &d);
    context.encode_verifier_kv_scatter(a, b, c, d, e, 100U, 2U, 2048U, 1023U);
    context.encode_gemma2_kv_cache_copy(a, b, c, d, 100U, 2U, 1023U, 1U);
    context.encode_f16_prefill_attention(a, b, c, d, e, f, 0U, 16U, 8U, 256U, 256U, 1024U, 0.0625F, 0.0F, 1023U, 512U, true, 0U);
    context.encode_gelu_tanh_multiply(a, b, c, 0U, &d);
    context.encode_verifier_input_validation(a, 0U, b, c, 2U, 262144U);
    context.encode_verifier_selection_requests(a, 0U, b, c, d, 2U, options, 262144U);
    const lge::engine::TokenSelectionRequest request;
    const std::array<lge::engine::TokenSelectionRequest, 2> requests {};
    std::uint32_t launches = context.encode_token_candidates(a, selection, request, 0.0F);
    launches += context.encode_token_candidates_width_two(a, selection, requests, 0.0F);
    launches += context.encode_target_token_candidates(a, target, 0U, 2U, 0.0F, false);
    context.encode_memory_barrier();
    context.push_debug_group("probe");
    context.pop_debug_group();
    static_cast<void>(context.commit());
    static_cast<void>(context.wait_until_completed());
    static_cast<void>(context.completion_stats());
    const lge::engine::CompactTokenCandidates one = context.read_token_candidates(selection);
    const std::array<lge::engine::CompactTokenCandidates, 2> two = context.read_token_candidates_width_two(selection);
    std::array<lge::engine::CompactTokenCandidates, 2> rows;
    context.read_target_token_candidates(target, 0U, rows);
    const std::uint32_t status = context.read_verifier_status(a) | context.read_operator_status();
    static_cast<void>(one); static_cast<void>(two); static_cast<void>(status); static_cast<void>(launches);
    context.restart();
    static_cast<void>(context.commit_and_wait());

    // buffers: allocation, views at an offset, weights as tiles and in GGUF order
    const auto descriptor = lge::tensor::TensorDescriptor::from(lge::tensor::Shape::from({2, 3840}), lge::tensor::DType::f32);
    const BackendBuffer fresh = hipctx::allocate_hip_buffer(descriptor);
    const BackendBuffer shared = hipctx::allocate_hip_buffer(descriptor, /*shared=*/true);
    const BackendBuffer view = hipctx::view_hip_buffer(fresh, 4U, descriptor);
    const BackendBuffer tiles = hipctx::upload_weight_tiles(nullptr, descriptor);
    const BackendBuffer canonical = hipctx::upload_canonical(nullptr, descriptor);
    static_cast<void>(hipctx::storage(view).device()); static_cast<void>(shared); static_cast<void>(tiles); static_cast<void>(canonical);
}
