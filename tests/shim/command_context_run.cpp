// Runs include/guffin_hip_command_context.hpp: the methods a Gemma 3 verify pass of the reference's engine calls on
// its command context (src/engine/gemma_target_runtime.cpp:13-221, src/engine/target_verifier_runtime.cpp:349-420),
// in that order, on buffers made through allocate_hip_buffer / view_hip_buffer / upload_weight_tiles, with inputs
// read from a directory and every result written back to it.  tests/test_gpu_command_context.py writes the inputs,
// runs this program on the GPU and compares each result, bit for bit, with the same operators called through the
// C entry points directly.  The exception classes of the error paths are checked here.
//
// usage: command_context_run <directory>
#include "guffin_hip_command_context.hpp"

#include <cstdio>
#include <fstream>
#include <iostream>
#include <sstream>

namespace lge = local_gguf_engine;
namespace hipctx = lge::tensor::backends::hip;
using lge::tensor::BackendBuffer;
using lge::tensor::DType;
using lge::tensor::Shape;
using lge::tensor::TensorDescriptor;

namespace {

std::string g_dir;

std::vector<std::uint8_t> read_file(const std::string& name) {
    std::ifstream in(g_dir + "/" + name, std::ios::binary);
    if (!in) throw std::runtime_error("missing input " + name);
    std::stringstream ss;
    ss << in.rdbuf();
    const std::string s = ss.str();
    return std::vector<std::uint8_t>(s.begin(), s.end());
}
void write_file(const std::string& name, const void* bytes, std::size_t count) {
    std::ofstream out(g_dir + "/" + name, std::ios::binary);
    out.write(static_cast<const char*>(bytes), static_cast<std::streamsize>(count));
}
void dump(const std::string& name, const BackendBuffer& buffer, std::size_t bytes = 0) {
    const std::size_t n = bytes ? bytes : buffer.descriptor().byte_count;
    std::vector<std::uint8_t> host(n);
    hipctx::check_hip(hipMemcpy(host.data(), hipctx::storage(buffer).device(), n, hipMemcpyDeviceToHost), "dump failed");
    write_file(name, host.data(), n);
}
TensorDescriptor f32_rows(std::uint64_t rows, std::uint64_t width) { return TensorDescriptor::from(Shape::from({rows, width}), DType::f32); }
TensorDescriptor words(std::uint64_t count) { return TensorDescriptor::from(Shape::from({count}), DType::f32); }
BackendBuffer upload_words(const std::vector<std::uint8_t>& bytes) {
    BackendBuffer b = hipctx::allocate_hip_buffer(words((bytes.size() + 3) / 4));
    hipctx::check_hip(hipMemcpy(hipctx::storage(b).device(), bytes.data(), bytes.size(), hipMemcpyHostToDevice), "upload failed");
    return b;
}
BackendBuffer tiles_of(const std::string& name, DType dtype, std::uint64_t K, std::uint64_t N) {
    const auto bytes = read_file(name);
    const auto d = TensorDescriptor::from_quantized_gguf_weight_matrix(Shape::from({K, N}), dtype);
    if (bytes.size() != d.byte_count) throw std::runtime_error("weight file has the wrong size: " + name);
    return hipctx::upload_weight_tiles(bytes.data(), d);
}

template <class Exception, class Call>
bool throws(const char* what, Call&& call) {
    try {
        call();
    } catch (const Exception&) {
        return true;
    } catch (const std::exception& e) {
        std::printf("WRONG EXCEPTION for %s: %s\n", what, e.what());
        return false;
    }
    std::printf("NO EXCEPTION for %s\n", what);
    return false;
}

struct TargetWorkspace {   // member names of engine::TargetSelectionWorkspace (target_verifier.hpp:209-219)
    BackendBuffer logits_tile, candidate_runs_a, candidate_runs_b, compact_results, raw_request_staging,
        resolved_request_staging, history_token_staging;
    std::uint32_t row_capacity = 0, batch_row_capacity = 0;
};

}  // namespace

int main(int argc, char** argv) {
    if (argc != 2) { std::fprintf(stderr, "usage: command_context_run <directory>\n"); return 2; }
    g_dir = argv[1];
    try {
        constexpr std::uint32_t H = 3840, QW = 4096, KW = 2048, F = 2048, V = 8192, cap = 64, rows = 2;
        constexpr float eps = 1e-6F;
        hipctx::HipCommandContext context("verify pass", false, true);

        // ---- operands, made the way a plan makes them ---------------------------------------------------------
        const auto embed_bytes = read_file("embed.q6k");
        const auto embed_desc = TensorDescriptor::from_quantized_gguf_weight_matrix(Shape::from({H, V}), DType::q6_k);
        const BackendBuffer embed_rows = hipctx::upload_canonical(embed_bytes.data(), embed_desc);
        const BackendBuffer head_tiles = hipctx::upload_weight_tiles(embed_bytes.data(), embed_desc);   // tied head
        const BackendBuffer wq = tiles_of("wq.q4k", DType::q4_k, H, QW), wk = tiles_of("wk.q4k", DType::q4_k, H, KW),
                            wv = tiles_of("wv.q6k", DType::q6_k, H, KW), wg = tiles_of("wg.q4k", DType::q4_k, H, F),
                            wu = tiles_of("wu.q4k", DType::q4_k, H, F);
        const BackendBuffer attn_norm = upload_words(read_file("attn_norm.f32")), q_norm = upload_words(read_file("q_norm.f32")),
                            k_norm = upload_words(read_file("k_norm.f32"));
        const BackendBuffer positions = upload_words(read_file("positions.u32")), ancestors = upload_words(read_file("ancestors.u32"));
        const BackendBuffer expected_ids = upload_words(read_file("tokens.u32"));
        // K/V rings as views that start 12 bytes into their allocations (tests/tensor/gemma3_metal_tests.cpp:765-774)
        const auto ring_desc = TensorDescriptor::from(Shape::from({cap, KW}), DType::f16);
        const auto ring_parent_desc = TensorDescriptor::from(Shape::from({cap * KW + 8}), DType::f16);
        const auto ring_k_bytes = read_file("ring_k.f16"), ring_v_bytes = read_file("ring_v.f16");
        const BackendBuffer ring_k_parent = hipctx::allocate_hip_buffer(ring_parent_desc), ring_v_parent = hipctx::allocate_hip_buffer(ring_parent_desc);
        const BackendBuffer ring_k = hipctx::view_hip_buffer(ring_k_parent, 12, ring_desc), ring_v = hipctx::view_hip_buffer(ring_v_parent, 12, ring_desc);
        hipctx::check_hip(hipMemcpy(hipctx::storage(ring_k).device(), ring_k_bytes.data(), ring_k_bytes.size(), hipMemcpyHostToDevice), "upload failed");
        hipctx::check_hip(hipMemcpy(hipctx::storage(ring_v).device(), ring_v_bytes.data(), ring_v_bytes.size(), hipMemcpyHostToDevice), "upload failed");
        // attention schedules: host-written shared storage
        const auto schedule_bytes = read_file("schedule.u32");
        const BackendBuffer schedules = hipctx::allocate_hip_buffer(words(schedule_bytes.size() / 4), /*shared=*/true);
        std::memcpy(hipctx::storage(schedules).host(), schedule_bytes.data(), schedule_bytes.size());

        // ---- activations and scratch -------------------------------------------------------------------------------
        const BackendBuffer ids = hipctx::allocate_hip_buffer(words(rows));
        const BackendBuffer x0 = hipctx::allocate_hip_buffer(f32_rows(rows, H)), u = hipctx::allocate_hip_buffer(f32_rows(rows, H));
        const BackendBuffer receipt_u = hipctx::allocate_hip_buffer(words(guffin_hip_receipt_bytes(rows, H) / 4));
        const BackendBuffer q = hipctx::allocate_hip_buffer(f32_rows(rows, QW)), q_own = hipctx::allocate_hip_buffer(f32_rows(rows, QW));
        const BackendBuffer k = hipctx::allocate_hip_buffer(f32_rows(rows, KW)), v = hipctx::allocate_hip_buffer(f32_rows(rows, KW));
        const BackendBuffer qn = hipctx::allocate_hip_buffer(f32_rows(rows, QW)), kn = hipctx::allocate_hip_buffer(f32_rows(rows, KW));
        const BackendBuffer qr = hipctx::allocate_hip_buffer(f32_rows(rows, QW));
        const BackendBuffer priv_k = hipctx::allocate_hip_buffer(TensorDescriptor::from(Shape::from({rows, KW}), DType::f16));
        const BackendBuffer priv_v = hipctx::allocate_hip_buffer(TensorDescriptor::from(Shape::from({rows, KW}), DType::f16));
        // the partitions the context will use: the rows' ring range plus the private rows (as it sizes the launch itself)
        std::uint32_t sched[2][4], first_position = UINT32_MAX, end_position = 0;
        std::memcpy(sched, schedule_bytes.data(), sizeof(sched));
        for (auto& s : sched) if (s[1] > 0) { first_position = std::min(first_position, s[0]); end_position = std::max(end_position, s[0] + s[1]); }
        const std::uint32_t max_tokens = (end_position > first_position ? end_position - first_position : 0U) + rows;
        const std::uint32_t partitions = guffin_hip_attention_partitions(max_tokens, 8);
        const BackendBuffer attn = hipctx::allocate_hip_buffer(f32_rows(rows, QW));
        const BackendBuffer receipt_a = hipctx::allocate_hip_buffer(words(guffin_hip_receipt_bytes(rows, QW) / 4));
        const BackendBuffer partial_out = hipctx::allocate_hip_buffer(words(std::uint64_t(rows) * 16 * partitions * 256));
        const BackendBuffer partial_ml = hipctx::allocate_hip_buffer(words(std::uint64_t(rows) * 16 * partitions * 2));
        const BackendBuffer partial_max = hipctx::view_hip_buffer(partial_ml, 0, words(std::uint64_t(rows) * 16 * partitions));
        const BackendBuffer partial_den = hipctx::view_hip_buffer(partial_ml, std::uint64_t(rows) * 16 * partitions * 4, words(std::uint64_t(rows) * 16 * partitions));
        const BackendBuffer gate = hipctx::allocate_hip_buffer(f32_rows(rows, F)), up = hipctx::allocate_hip_buffer(f32_rows(rows, F)),
                            h = hipctx::allocate_hip_buffer(f32_rows(rows, F));
        const BackendBuffer receipt_h = hipctx::allocate_hip_buffer(words(guffin_hip_receipt_bytes(rows, F) / 4));
        const BackendBuffer status = hipctx::allocate_hip_buffer(words(4));
        const BackendBuffer candidate_runs = hipctx::allocate_hip_buffer(words(guffin_hip_select_workspace_bytes(rows, V, 320) / 4 + 1));
        TargetWorkspace ws {hipctx::allocate_hip_buffer(f32_rows(rows, V)), candidate_runs, candidate_runs,
                            hipctx::allocate_hip_buffer(words(rows * (8 + 384 * 8) / 4)), upload_words(read_file("requests.raw")),
                            hipctx::allocate_hip_buffer(words(rows * sizeof(guffin_resolved_row) / 4)),
                            hipctx::allocate_hip_buffer(words(rows * 64)), rows, rows};
        lge::engine::TokenSamplerOptions options;
        options.temperature = 1.0F; options.top_k = 40; options.top_p = 0.95F; options.min_p = 0.0F; options.repetition_penalty = 1.3F;

        // ---- the pass ------------------------------------------------------------------------------------------------
        const auto token_bytes = read_file("tokens.u32");
        std::uint32_t tokens[2];
        std::memcpy(tokens, token_bytes.data(), 8);
        context.write_u32s(ids, 0, tokens);
        context.encode_verifier_input_validation(ids, 0, expected_ids, status, rows, V);
        context.encode_verifier_selection_requests(ws.raw_request_staging, 0, ws.resolved_request_staging, ws.history_token_staging,
                                                   status, rows, options, V);
        context.encode_embedding(ids, embed_rows, x0, std::sqrt(static_cast<float>(H)));
        context.encode_memory_barrier();
        context.encode_rms_norm(x0, attn_norm, u, eps, rows, 0, &receipt_u);
        context.encode_memory_barrier();
        context.encode_verifier_matmul(u, wq, q, rows, false, &receipt_u);
        context.encode_verifier_matmul(u, wq, q_own, rows);   // no producer receipt: the context makes its own
        context.encode_verifier_matmul(u, wk, k, rows, false, &receipt_u);
        context.encode_verifier_matmul(u, wv, v, rows, false, &receipt_u);
        context.encode_memory_barrier();
        context.encode_head_rms_norm(q, q_norm, qn, eps, rows, 16, 256);
        context.encode_head_rms_norm(k, k_norm, kn, eps, rows, 8, 256);
        context.encode_memory_barrier();
        context.encode_verifier_rope(qn, positions, qr, rows, 16, 256, 256, 1e6F, 0.125F);
        context.encode_verifier_kv_store(kn, v, positions, priv_k, priv_v, rows, 8, 256, 256, 1e6F, 0.125F, &status);
        context.encode_memory_barrier();
        context.encode_verifier_attention(qr, ring_k, ring_v, priv_k, priv_v, schedules, 0, ancestors, attn, partial_out, partial_max,
                                          partial_den, rows, cap - 1, 16, 8, 256, 256, 0.0625F, 0.0F, &receipt_a);
        context.encode_memory_barrier();
        context.encode_verifier_matmul(u, wg, gate, rows, false, &receipt_u);
        context.encode_verifier_matmul(u, wu, up, rows, false, &receipt_u);
        context.encode_memory_barrier();
        context.encode_gelu_tanh_multiply(gate, up, h, 0, &receipt_h);
        context.encode_target_head_rows(u, 0, head_tiles, ws.logits_tile, rows);
        context.encode_memory_barrier();
        const std::uint32_t launches = context.encode_target_token_candidates(ws.logits_tile, ws, 0, rows, 0.0F, false);
        const hipctx::HipCommandStats committed = context.commit();
        const hipctx::HipCommandStats stats = context.wait_until_completed();
        std::array<lge::engine::CompactTokenCandidates, 2> candidates;
        context.read_target_token_candidates(ws, 0, candidates);
        const std::uint32_t verifier_status = context.read_verifier_status(status), operator_status = context.read_operator_status();

        // ---- results ---------------------------------------------------------------------------------------------------
        dump("x0.out", x0); dump("u.out", u); dump("receipt_u.out", receipt_u); dump("q.out", q); dump("q_own.out", q_own);
        dump("k.out", k); dump("v.out", v); dump("qn.out", qn); dump("kn.out", kn); dump("qr.out", qr);
        dump("priv_k.out", priv_k); dump("priv_v.out", priv_v); dump("attn.out", attn); dump("receipt_a.out", receipt_a);
        dump("h.out", h); dump("receipt_h.out", receipt_h); dump("logits.out", ws.logits_tile);
        dump("resolved.out", ws.resolved_request_staging);
        for (int r = 0; r < 2; ++r) {
            std::vector<std::uint32_t> flat;
            flat.push_back(candidates[r].count);
            for (std::uint32_t i = 0; i < candidates[r].count; ++i) {
                flat.push_back(candidates[r].values[i].token);
                std::uint32_t bits;
                std::memcpy(&bits, &candidates[r].values[i].logit, 4);
                flat.push_back(bits);
            }
            write_file("candidates" + std::to_string(r) + ".out", flat.data(), flat.size() * 4);
        }
        std::ostringstream text;
        text << "launches " << launches << "\nverifier_status " << verifier_status << "\noperator_status " << operator_status
             << "\ncommit_count " << stats.commit_count << "\ncommitted_before_wait " << committed.commit_count
             << "\nsynchronous_wait_count " << stats.synchronous_wait_count << "\ncommand_buffer_count " << stats.command_buffer_count
             << "\ncompute_dispatch_count " << stats.compute_dispatch_count << "\nmemory_barrier_count " << stats.memory_barrier_count
             << "\ngpu_duration_ns " << stats.gpu_duration_ns << "\nq4_width_two " << stats.q4_width_two_projection_count
             << "\nq6_width_two " << stats.q6_width_two_projection_count << "\nattention_dispatches " << stats.decode_attention_dispatch_count
             << "\nattention_partitions " << stats.decode_attention_partition_count << "\nattention_tokens " << stats.decode_attention_token_count
             << "\n";

        // ---- a second command buffer: the operators around the pass ----------------------------------------------------
        // (residual norm, the projections on more than two rows, K/V scatter into the 12-byte views and copy out of them,
        // prefill attention over them, candidate selection from host-side requests of one and of two rows)
        bool ok = true;
        ok &= throws<std::logic_error>("encode after commit", [&] { context.encode_memory_barrier(); });
        context.restart();
        constexpr std::uint32_t P = 5;   // rows of the prefill-shaped calls
        const auto upload_rows = [&](const std::string& name, std::uint64_t n_rows, std::uint64_t width, DType dtype) {
            const auto bytes = read_file(name);
            BackendBuffer b = hipctx::allocate_hip_buffer(TensorDescriptor::from(Shape::from({n_rows, width}), dtype));
            if (bytes.size() != b.descriptor().byte_count) throw std::runtime_error("input has the wrong size: " + name);
            hipctx::check_hip(hipMemcpy(hipctx::storage(b).device(), bytes.data(), bytes.size(), hipMemcpyHostToDevice), "upload failed");
            return b;
        };
        const BackendBuffer xp = upload_rows("xp.f32", P, H, DType::f32), qp = upload_rows("qp.f32", P, QW, DType::f32);
        const BackendBuffer chunk_k = upload_rows("chunk_k.f16", P, KW, DType::f16), chunk_v = upload_rows("chunk_v.f16", P, KW, DType::f16);
        const BackendBuffer selected = upload_words(read_file("selected.u32"));
        const BackendBuffer y_add = hipctx::allocate_hip_buffer(f32_rows(rows, H));
        const BackendBuffer yp_matrix = hipctx::allocate_hip_buffer(f32_rows(P, QW)), yp_pairs = hipctx::allocate_hip_buffer(f32_rows(P, QW));
        const BackendBuffer yv_matrix = hipctx::allocate_hip_buffer(f32_rows(P, KW));
        const auto copy_desc = TensorDescriptor::from(Shape::from({16, KW}), DType::f16);
        const BackendBuffer copy_k = hipctx::allocate_hip_buffer(copy_desc), copy_v = hipctx::allocate_hip_buffer(copy_desc);
        hipctx::check_hip(hipMemset(hipctx::storage(copy_k).device(), 0, copy_desc.byte_count), "clearing failed");
        hipctx::check_hip(hipMemset(hipctx::storage(copy_v).device(), 0, copy_desc.byte_count), "clearing failed");
        const BackendBuffer pattn = hipctx::allocate_hip_buffer(f32_rows(P, QW)), pattn_window = hipctx::allocate_hip_buffer(f32_rows(P, QW));
        const BackendBuffer marks = hipctx::allocate_hip_buffer(words(4));
        struct SelectionWorkspace { BackendBuffer candidate_runs_a, compact_result; };   // engine::TokenSelectionWorkspace's members
        const SelectionWorkspace sw {candidate_runs, hipctx::allocate_hip_buffer(words(2 * (8 + 384 * 8) / 4))};
        std::array<lge::engine::TokenSelectionRequest, 2> requests;
        requests[0].top_k = 40; requests[0].history_token_count = 3; requests[0].base_candidate_count = 43;
        requests[0].history_token_ids[0] = 3; requests[0].history_token_ids[1] = 9; requests[0].history_token_ids[2] = 70;
        requests[1].top_k = 1; requests[1].history_token_count = 0; requests[1].base_candidate_count = 1;

        context.write_u32(marks, 0xC0FFEEu);
        context.encode_rms_norm_add(u, attn_norm, x0, y_add, eps, rows);
        context.encode_verifier_matmul(xp, wq, yp_matrix, P, true);     // the matrix-core path
        context.encode_verifier_matmul(xp, wv, yv_matrix, P, true);     // ... on Q6_K tiles
        context.encode_verifier_matmul(xp, wq, yp_pairs, P, false);     // pairs of rows through the decode GEMV
        context.encode_verifier_kv_scatter(priv_k, priv_v, selected, ring_k, ring_v, 40, rows, KW, cap - 1);
        context.encode_memory_barrier();
        context.encode_gemma2_kv_cache_copy(ring_k, ring_v, copy_k, copy_v, 30, 12, cap - 1, 15);
        context.encode_f16_prefill_attention(qp, ring_k, ring_v, chunk_k, chunk_v, pattn, 42, 16, 8, 256, 256, 42 + P, 0.0625F, 0.0F,
                                             cap - 1, P, true, 42);
        context.encode_f16_prefill_attention(qp, ring_k, ring_v, chunk_k, chunk_v, pattn_window, 42, 16, 8, 256, 256, 16, 0.0625F, 0.0F,
                                             cap - 1, P, true, 42);
        const std::uint32_t launches_two = context.encode_token_candidates_width_two(ws.logits_tile, sw, requests, 0.0F);
        const hipctx::HipCommandStats second = context.commit_and_wait();
        const auto pair = context.read_token_candidates_width_two(sw);
        dump("y_add.out", y_add); dump("yp_matrix.out", yp_matrix); dump("yv_matrix.out", yv_matrix); dump("yp_pairs.out", yp_pairs);
        dump("ring_k_after.out", ring_k); dump("ring_v_after.out", ring_v); dump("copy_k.out", copy_k); dump("copy_v.out", copy_v);
        dump("pattn.out", pattn); dump("pattn_window.out", pattn_window); dump("marks.out", marks);
        const auto write_candidates = [&](const std::string& name, const lge::engine::CompactTokenCandidates& c) {
            std::vector<std::uint32_t> flat {c.count};
            for (std::uint32_t i = 0; i < c.count; ++i) {
                flat.push_back(c.values[i].token);
                std::uint32_t logit_bits;
                std::memcpy(&logit_bits, &c.values[i].logit, 4);
                flat.push_back(logit_bits);
            }
            write_file(name, flat.data(), flat.size() * 4);
        };
        write_candidates("pair0.out", pair[0]);
        write_candidates("pair1.out", pair[1]);
        // a third one: a single row
        context.restart();
        const std::uint32_t launches_one = context.encode_token_candidates(ws.logits_tile, sw, requests[0], 0.0F);
        const hipctx::HipCommandStats third = context.commit_and_wait();
        write_candidates("single.out", context.read_token_candidates(sw));
        text << "launches_two " << launches_two << "\nlaunches_one " << launches_one
             << "\nsecond_command_buffers " << second.command_buffer_count << "\nsecond_commits " << second.commit_count
             << "\nq4_generic_tiled " << second.q4_generic_tiled_projection_count << "\nq6_generic_tiled " << second.q6_generic_tiled_projection_count
             << "\nq4_small_batch " << second.q4_small_batch_projection_count << "\nthird_commits " << third.commit_count
             << "\nthird_gpu_duration_ns " << third.gpu_duration_ns << "\n";

        // ---- error paths: the exception classes the engine expects ------------------------------------------------------
        ok &= throws<std::logic_error>("encode after the third commit", [&] { context.encode_memory_barrier(); });
        context.restart();
        ok &= throws<std::invalid_argument>("prefill attention without a staged chunk", [&] {
            context.encode_f16_prefill_attention(qp, ring_k, ring_v, chunk_k, chunk_v, pattn, 42, 16, 8, 256, 256, 42 + P, 0.0625F, 0.0F,
                                                 cap - 1, P, false, 42);
        });
        ok &= throws<std::invalid_argument>("a request outside product bounds", [&] {
            auto bad = requests[0];
            bad.base_candidate_count = 40;   // not top_k + history
            (void)context.encode_token_candidates(ws.logits_tile, sw, bad, 0.0F);
        });
        ok &= throws<std::invalid_argument>("zero rows", [&] { context.encode_verifier_matmul(u, wq, q, 0); });
        ok &= throws<std::invalid_argument>("mismatched inner dimension", [&] { context.encode_verifier_matmul(q, wk, k, rows); });
        ok &= throws<std::invalid_argument>("output too small", [&] { context.encode_verifier_matmul(u, wq, k, rows); });
        ok &= throws<std::invalid_argument>("view off a word", [&] { (void)hipctx::view_hip_buffer(ring_k_parent, 2, ring_desc); });
        ok &= throws<std::invalid_argument>("softcap", [&] {
            context.encode_verifier_attention(qr, ring_k, ring_v, priv_k, priv_v, schedules, 0, ancestors, attn, partial_out, partial_max,
                                              partial_den, rows, cap - 1, 16, 8, 256, 256, 0.0625F, 30.0F, nullptr);
        });
        ok &= throws<std::logic_error>("read before completion", [&] { context.read_target_token_candidates(ws, 0, candidates); });
        ok &= throws<std::logic_error>("wait before commit", [&] { (void)context.wait_until_completed(); });
        (void)context.commit_and_wait();
        ok &= throws<std::logic_error>("restart is needed after completion", [&] { context.encode_memory_barrier(); });
        text << "exceptions " << (ok ? "ok" : "FAILED") << "\n";
        write_file("stats.txt", text.str().data(), text.str().size());
        std::printf("%s", text.str().c_str());
        return ok ? 0 : 1;
    } catch (const std::exception& e) {
        std::fprintf(stderr, "command_context_run: %s\n", e.what());
        return 3;
    }
}
