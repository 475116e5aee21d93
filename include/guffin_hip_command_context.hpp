// HipCommandContext: the command context of the reference's Metal backend
// (src/tensor/backends/metal/metal_command_context.hpp:54-365) over the C entry points of guffin_hip.h.
//
// The engine code of the reference (encode_gemma_target_blocks, the width-two verifier, the drafter)
// talks to its GPU through the methods of MetalCommandContext and through BackendBuffer.  This header
// gives the same methods, with the same argument lists and the same exception classes, for a HIP build:
// a maintainer adds `BackendKind::hip`, routes allocate_backend_buffer / copy_tensor_to_backend to the
// functions below, and instantiates HipCommandContext where the engine instantiates MetalCommandContext.
// It compiles against the reference's public headers (include/local_gguf_engine) and the HIP runtime
// API only; all device work is behind the C functions.  The selection workspaces
// (engine::Gemma2MetalSelectionWorkspace, include/local_gguf_engine/engine/gemma2_metal_plan.hpp:180-189;
// engine::TargetSelectionWorkspace, include/local_gguf_engine/engine/target_verifier.hpp:209-219) are taken
// as template parameters and used by member name, because their headers pull in a macOS-only header
// (runtime/sha256.hpp includes CommonCrypto) and this one has to compile where HIP does.
//
// What differs from the Metal context, because the kernels differ:
//  * Quantised weight matrices live on the device as wave tiles (guffin_hip_repack), marked with
//    TensorPacking::kquant_columns8 in their descriptor; a canonical copy serves encode_embedding.
//  * The `q4_input_sums` buffers hold this library's activation receipt (guffin_hip_receipt_bytes bytes
//    for the producer's rows and width), not the Metal layout; a null pointer makes the consumer build the
//    receipt itself in the context's scratch (guffin_hip_group_sums) before its GEMV.
//  * One in-order stream: encode_memory_barrier has nothing to do, commit() only marks the batch and
//    wait_until_completed() is hipStreamSynchronize.
//  * Candidate results use this library's row record {count, status, 384 x {token, logit}}.
#pragma once

#include "guffin_hip.h"

#include "local_gguf_engine/engine/sampling.hpp"
#include "local_gguf_engine/runtime/backend_error.hpp"
#include "local_gguf_engine/tensor/backend_buffer.hpp"

#include <hip/hip_runtime_api.h>

#include <algorithm>
#include <array>
#include <cmath>
#include <cstddef>
#include <cstdint>
#include <cstring>
#include <memory>
#include <span>
#include <stdexcept>
#include <string>
#include <string_view>
#include <vector>

namespace local_gguf_engine::tensor::backends::hip {

// The enumerator a HIP build adds to runtime::BackendKind (include/local_gguf_engine/runtime/backend_kind.hpp:5-8).
inline constexpr runtime::BackendKind backend_kind = static_cast<runtime::BackendKind>(2);

[[noreturn]] inline void throw_hip(const char* what) {
    throw runtime::BackendError(runtime::BackendErrorCode::metal_execution_failed, backend_kind, what);
}
inline void check_hip(hipError_t rc, const char* what) {
    if (rc != hipSuccess) throw_hip(what);
}
// C return codes to the exception classes the engine expects: argument, shape, capacity and alignment
// errors are std::invalid_argument and are raised before anything is enqueued; state errors are
// std::logic_error; a failed launch or runtime call is runtime::BackendError.
inline void check(int rc) {
    if (rc == GUFFIN_OK) return;
    if (rc == GUFFIN_E_HIP) throw_hip(guffin_hip_last_error());
    if (rc == GUFFIN_E_STATE) throw std::logic_error(guffin_hip_last_error());
    throw std::invalid_argument(guffin_hip_last_error());
}

// ---- buffers ------------------------------------------------------------------------------
// Device bytes plus the descriptor; views share the parent allocation at a byte offset
// (backend_buffer.hpp:17-45).  `shared` allocations are pinned host memory that the device reads in
// place: the attention schedules, which the host writes and the context also reads when it sizes the launch.
class HipBufferStorage final : public detail::BackendBufferStorage {
public:
    HipBufferStorage(std::shared_ptr<void> base, std::size_t offset, TensorDescriptor descriptor, bool shared)
        : base_(std::move(base)), offset_(offset), descriptor_(std::move(descriptor)), shared_(shared) {}
    [[nodiscard]] runtime::BackendKind backend() const noexcept override { return backend_kind; }
    [[nodiscard]] const TensorDescriptor& descriptor() const noexcept override { return descriptor_; }
    [[nodiscard]] void* device() const noexcept { return static_cast<std::byte*>(base_.get()) + offset_; }
    [[nodiscard]] void* host() const noexcept { return shared_ ? device() : nullptr; }
    [[nodiscard]] const std::shared_ptr<void>& base() const noexcept { return base_; }
    [[nodiscard]] std::size_t offset() const noexcept { return offset_; }
    [[nodiscard]] bool shared() const noexcept { return shared_; }

private:
    std::shared_ptr<void> base_;
    std::size_t offset_;
    TensorDescriptor descriptor_;
    bool shared_;
};

[[nodiscard]] inline const HipBufferStorage& storage(const BackendBuffer& buffer) {
    if (buffer.backend() != backend_kind) throw std::invalid_argument("buffer does not belong to the HIP backend");
    return static_cast<const HipBufferStorage&>(backend_buffer_storage(buffer));
}
[[nodiscard]] inline BackendBuffer allocate_hip_buffer(const TensorDescriptor& descriptor, bool shared = false) {
    void* bytes = nullptr;
    const std::size_t size = std::max<std::size_t>(descriptor.byte_count, 16);
    check_hip(shared ? hipHostMalloc(&bytes, size, hipHostMallocDefault) : hipMalloc(&bytes, size), "allocation failed");
    std::shared_ptr<void> base(bytes, [shared](void* p) { shared ? (void)hipHostFree(p) : (void)hipFree(p); });
    if (!shared) check_hip(hipMemset(bytes, 0, size), "clearing a new buffer failed");
    else std::memset(bytes, 0, size);
    return detail::make_backend_buffer(std::make_shared<HipBufferStorage>(std::move(base), 0, descriptor, shared));
}
[[nodiscard]] inline BackendBuffer view_hip_buffer(const BackendBuffer& parent, std::size_t byte_offset,
                                                   const TensorDescriptor& descriptor) {
    const auto& p = storage(parent);
    if (byte_offset % 4 != 0 || byte_offset > p.descriptor().byte_count
        || descriptor.byte_count > p.descriptor().byte_count - byte_offset)
        throw std::invalid_argument("HIP buffer view is outside its parent or not 4-byte aligned");
    return detail::make_backend_buffer(
        std::make_shared<HipBufferStorage>(p.base(), p.offset() + byte_offset, descriptor, p.shared()));
}
[[nodiscard]] inline int guffin_dtype(DType dtype) {
    switch (dtype) {
        case DType::q8_0: return GUFFIN_Q8_0;
        case DType::q4_k: return GUFFIN_Q4_K;
        case DType::q6_k: return GUFFIN_Q6_K;
        default: throw std::invalid_argument("HIP backend: the matrix is not Q8_0, Q4_K or Q6_K");
    }
}
// A quantised [K, N] GGUF weight matrix on the device, repacked once into wave tiles (the counterpart of
// the reference's columns8 upload, include/local_gguf_engine/tensor/kquant_packing.hpp:9-23).
[[nodiscard]] inline BackendBuffer upload_weight_tiles(const void* gguf_bytes, TensorDescriptor descriptor) {
    const int dtype = guffin_dtype(descriptor.dtype);
    const auto K = static_cast<std::uint32_t>(descriptor.shape.dimension(0));
    const auto N = static_cast<std::uint32_t>(descriptor.shape.dimension(1));
    void* canonical = nullptr;
    check_hip(hipMalloc(&canonical, descriptor.byte_count), "allocation failed");
    std::shared_ptr<void> staging(canonical, [](void* p) { (void)hipFree(p); });
    check_hip(hipMemcpy(canonical, gguf_bytes, descriptor.byte_count, hipMemcpyHostToDevice), "weight upload failed");
    TensorDescriptor tiled = descriptor;
    tiled.packing = TensorPacking::kquant_columns8;
    tiled.byte_count = guffin_hip_packed_bytes(dtype, K, N);
    if (tiled.byte_count == 0) throw std::invalid_argument("HIP backend: the matrix shape cannot be tiled");
    auto tiles = allocate_hip_buffer(tiled);
    check(guffin_hip_repack(nullptr, dtype, canonical, storage(tiles).device(), K, N));
    check_hip(hipDeviceSynchronize(), "weight repack failed");
    return tiles;
}
// The same bytes in GGUF order (encode_embedding reads rows of the canonical stream).
[[nodiscard]] inline BackendBuffer upload_canonical(const void* bytes, const TensorDescriptor& descriptor) {
    auto buffer = allocate_hip_buffer(descriptor);
    check_hip(hipMemcpy(storage(buffer).device(), bytes, descriptor.byte_count, hipMemcpyHostToDevice), "upload failed");
    return buffer;
}

// MetalCommandStats (metal_command_context.hpp:19-46) with the fields that have a meaning here.  One in-order stream
// stands for the command buffer and its encoders; projections are counted by weight format and row count
// (decode = one row, width_two = two rows, small_batch = the pairs of a longer run, generic_tiled = the
// matrix-core GEMM of a prefill chunk); gpu_duration_ns is the device time between the batch's first encode
// and its commit (hipEvent pair, read by wait_until_completed).
struct HipCommandStats {
    std::uint32_t command_buffer_count = 0;
    std::uint32_t commit_count = 0;
    std::uint32_t synchronous_wait_count = 0;
    std::uint32_t compute_dispatch_count = 0;
    std::uint32_t memory_barrier_count = 0;
    std::uint32_t transient_buffer_allocation_count = 0;   // stays 0: nothing is allocated after construction
    std::uint64_t gpu_duration_ns = 0;
    std::uint32_t q4_decode_projection_count = 0;
    std::uint32_t q8_decode_projection_count = 0;
    std::uint32_t q8_width_two_projection_count = 0;
    std::uint32_t q4_small_batch_projection_count = 0;
    std::uint32_t q4_width_two_projection_count = 0;
    std::uint32_t q4_generic_tiled_projection_count = 0;
    std::uint32_t q6_decode_projection_count = 0;
    std::uint32_t q6_small_batch_projection_count = 0;
    std::uint32_t q6_width_two_projection_count = 0;
    std::uint32_t q6_generic_tiled_projection_count = 0;
    std::uint32_t decode_attention_dispatch_count = 0;      // verify / decode attention encodes
    std::uint32_t decode_attention_partition_count = 0;     // token partitions of those launches
    std::uint64_t decode_attention_token_count = 0;         // tokens their longest rows attend
};

// ---- the context ----------------------------------------------------------------------------
class HipCommandContext final {
public:
    // scratch_floats bounds the k-slice partial planes and self-made receipts of one GEMV (the largest
    // slices * rows * N of the model, and rows * K / 4 + rows * K): allocated here, once.
    explicit HipCommandContext(std::string_view label, bool /*concurrent_compute*/ = false, bool /*precise_math*/ = false,
                               int device = 0, std::size_t scratch_floats = std::size_t(8) << 20)
        : label_(label), scratch_floats_(scratch_floats) {
        check(guffin_hip_init(device));
        check_hip(hipStreamCreate(&stream_), "stream creation failed");
        check_hip(hipEventCreate(&batch_start_), "event creation failed");
        check_hip(hipEventCreate(&batch_end_), "event creation failed");
        check_hip(hipMalloc(&scratch_, scratch_floats * sizeof(float)), "allocation failed");
        check_hip(hipMalloc(&receipt_, scratch_floats * sizeof(float)), "allocation failed");
        check_hip(hipMalloc(&meta_, kMetaWords * sizeof(std::uint32_t)), "allocation failed");
        check_hip(hipMemset(meta_, 0, kMetaWords * sizeof(std::uint32_t)), "clearing scratch failed");
    }
    ~HipCommandContext() {
        if (stream_) (void)hipStreamSynchronize(stream_);
        (void)hipFree(scratch_);
        (void)hipFree(receipt_);
        (void)hipFree(meta_);
        if (batch_start_) (void)hipEventDestroy(batch_start_);
        if (batch_end_) (void)hipEventDestroy(batch_end_);
        if (stream_) (void)hipStreamDestroy(stream_);
    }
    HipCommandContext(const HipCommandContext&) = delete;
    HipCommandContext& operator=(const HipCommandContext&) = delete;

    // Makes a completed context encodable again (:61): the stream is reused as it is.
    void restart() {
        if (submitted_ && !completed_) throw std::logic_error("HIP command context restarted before completion");
        submitted_ = completed_ = started_ = false;
    }
    [[nodiscard]] hipStream_t stream() const noexcept { return stream_; }

    void write_u32(const BackendBuffer& destination, std::uint32_t value) { write_u32s(destination, 0, {&value, 1}); }
    // hipMemcpyWithStream: ordered on the stream, and back only when the source has been read (`values` may die).
    void write_u32s(const BackendBuffer& destination, std::uint32_t element_offset, std::span<const std::uint32_t> values) {
        require_encodable();
        require_capacity(destination, (std::uint64_t(element_offset) + values.size()) * 4, "write_u32s destination");
        check_hip(hipMemcpyWithStream(u32(destination) + element_offset, values.data(), values.size_bytes(),
                                 hipMemcpyHostToDevice, stream_), "write_u32s failed");
    }

    void encode_embedding(const BackendBuffer& token_ids, const BackendBuffer& weight, const BackendBuffer& output,
                          float scale, std::uint32_t token_offset = 0, std::uint32_t token_count = 0) {
        require_encodable();
        const auto& w = weight.descriptor();
        if (w.packing != TensorPacking::canonical) throw std::invalid_argument("HIP embedding reads the canonical block stream");
        const auto width = dim32(w, 0), vocab = dim32(w, 1);
        const auto available = static_cast<std::uint32_t>(token_ids.descriptor().element_count);
        if (token_offset > available) throw std::invalid_argument("HIP embedding token offset is invalid");
        const auto rows = token_count == 0 ? available - token_offset : token_count;
        if (rows == 0 || rows > available - token_offset) throw std::invalid_argument("HIP embedding token count is invalid");
        require_capacity(output, std::uint64_t(rows) * width * 4, "embedding output");
        check(guffin_hip_embed(stream_, guffin_dtype(w.dtype), dev(weight), u32(token_ids) + token_offset, f32(output), rows,
                               width, scale, vocab, status_word()));
        ++stats_.compute_dispatch_count;
    }

    // y[rows][N] = x[rows][K] W.  rows <= 2 take the decode GEMV, more rows the matrix-core GEMM when the
    // caller allows it (:94) and pairs of rows otherwise, so a row's result never depends on its batch.
    void encode_verifier_matmul(const BackendBuffer& input, const BackendBuffer& weight, const BackendBuffer& output,
                                std::uint32_t row_count, bool allow_prefill_matrix = false,
                                const BackendBuffer* q4_input_sums = nullptr) {
        require_encodable();
        const auto& in = input.descriptor();
        if (in.shape.rank() != 2U) throw std::invalid_argument("HIP verifier matmul requires matrix input rows");
        if (row_count == 0U || row_count > in.shape.dimension(0)) throw std::invalid_argument("HIP verifier matmul row count is invalid");
        const auto K = dim32(in, 1), N = dim32(weight.descriptor(), 1);
        if (K != weight.descriptor().shape.dimension(0)) throw std::invalid_argument("HIP verifier matmul inner dimensions do not match");
        require_capacity(output, std::uint64_t(row_count) * N * 4, "verifier matmul output");
        const int dtype = guffin_dtype(weight.descriptor().dtype);
        if (weight.descriptor().packing == TensorPacking::canonical) {   // GGUF bytes as uploaded
            check(guffin_hip_gemv(stream_, dtype, dev(weight), f32(input), f32(output), row_count, K, N));
            ++stats_.compute_dispatch_count;
            return;
        }
        if (row_count > 2U && allow_prefill_matrix) {
            if (guffin_hip_prefill_image_bytes(row_count, K) > scratch_floats_ * sizeof(float))
                throw std::invalid_argument("HIP prefill matmul exceeds the context's scratch");
            check(guffin_hip_prefill_pack(stream_, f32(input), receipt_, row_count, K));
            check(guffin_hip_prefill_gemm(stream_, dtype, dev(weight), receipt_, f32(output), row_count, K, N));
            stats_.compute_dispatch_count += 2;
            if (dtype == GUFFIN_Q4_K) ++stats_.q4_generic_tiled_projection_count;
            if (dtype == GUFFIN_Q6_K) ++stats_.q6_generic_tiled_projection_count;
            return;
        }
        for (std::uint32_t row = 0; row < row_count; row += 2U) {
            const std::uint32_t rows = std::min(2U, row_count - row);
            const float* x = f32(input) + std::size_t(row) * K;
            const float* sums = nullptr;
            if (q4_input_sums != nullptr && row_count <= 2U) {
                require_capacity(*q4_input_sums, guffin_hip_receipt_bytes(rows, K), "activation receipt");
                sums = f32(*q4_input_sums);
            } else {
                sums = make_receipt(x, rows, K);
            }
            gemv(dtype, dev(weight), x, sums, f32(output) + std::size_t(row) * N, rows, K, N);
            count_projection(dtype, rows, row_count > 2U);
        }
    }
    // Logit rows of the output head (:103): the same GEMV on the head's tiles.
    void encode_target_head_rows(const BackendBuffer& input, std::uint32_t input_row_start, const BackendBuffer& weight,
                                 const BackendBuffer& logits_tile, std::uint32_t row_count) {
        require_encodable();
        const auto& in = input.descriptor();
        if (in.shape.rank() != 2U || row_count == 0U || row_count > 2U || input_row_start > in.shape.dimension(0)
            || row_count > in.shape.dimension(0) - input_row_start)
            throw std::invalid_argument("HIP target head row tile is invalid");
        const auto K = dim32(in, 1), N = dim32(weight.descriptor(), 1);
        if (K != weight.descriptor().shape.dimension(0) || weight.descriptor().packing != TensorPacking::kquant_columns8)
            throw std::invalid_argument("HIP target head expects tiled weights of the input's width");
        require_capacity(logits_tile, std::uint64_t(row_count) * N * 4, "target head logits");
        const float* x = f32(input) + std::size_t(input_row_start) * K;
        gemv(guffin_dtype(weight.descriptor().dtype), dev(weight), x, make_receipt(x, row_count, K), f32(logits_tile),
             row_count, K, N);
        count_projection(guffin_dtype(weight.descriptor().dtype), row_count, false);
    }

    void encode_head_rms_norm(const BackendBuffer& input, const BackendBuffer& weight, const BackendBuffer& output,
                              float epsilon, std::uint32_t row_count, std::uint32_t head_count, std::uint32_t head_dimension) {
        require_encodable();
        const auto bytes = std::uint64_t(row_count) * head_count * head_dimension * 4;
        require_capacity(input, bytes, "head norm input");
        require_capacity(output, bytes, "head norm output");
        require_capacity(weight, std::uint64_t(head_dimension) * 4, "head norm weight");
        check(guffin_hip_head_rms_norm(stream_, f32(input), f32(weight), f32(output), row_count, head_count, head_dimension, epsilon));
        ++stats_.compute_dispatch_count;
    }
    void encode_rms_norm(const BackendBuffer& input, const BackendBuffer& weight, const BackendBuffer& output, float epsilon,
                         std::uint32_t row_count = 0, std::uint32_t input_row_start = 0,
                         const BackendBuffer* q4_input_sums = nullptr) {
        norm(input, weight, nullptr, output, epsilon, row_count, input_row_start, q4_input_sums);
    }
    void encode_rms_norm_add(const BackendBuffer& input, const BackendBuffer& weight, const BackendBuffer& residual,
                             const BackendBuffer& output, float epsilon, std::uint32_t row_count = 0) {
        norm(input, weight, &residual, output, epsilon, row_count, 0, nullptr);
    }

    void encode_verifier_rope(const BackendBuffer& input, const BackendBuffer& positions, const BackendBuffer& output,
                              std::uint32_t row_count, std::uint32_t head_count, std::uint32_t head_dimension,
                              std::uint32_t rope_dimension_count, float frequency_base, float frequency_scale = 1.0F) {
        require_encodable();
        const auto bytes = std::uint64_t(row_count) * head_count * head_dimension * 4;
        require_capacity(input, bytes, "rope input");
        require_capacity(output, bytes, "rope output");
        require_capacity(positions, std::uint64_t(row_count) * 4, "rope positions");
        check(guffin_hip_rope_neox(stream_, f32(input), u32(positions), f32(output), row_count, head_count, head_dimension,
                                   rope_dimension_count, frequency_base, frequency_scale));
        ++stats_.compute_dispatch_count;
    }
    void encode_verifier_kv_store(const BackendBuffer& raw_key, const BackendBuffer& raw_value, const BackendBuffer& positions,
                                  const BackendBuffer& private_key, const BackendBuffer& private_value, std::uint32_t row_count,
                                  std::uint32_t head_count, std::uint32_t head_dimension, std::uint32_t rope_dimension_count,
                                  float frequency_base, float frequency_scale = 1.0F,
                                  const BackendBuffer* numerical_status = nullptr) {
        require_encodable();
        const auto elements = std::uint64_t(row_count) * head_count * head_dimension;
        require_capacity(raw_key, elements * 4, "kv store raw key");
        require_capacity(raw_value, elements * 4, "kv store raw value");
        require_capacity(private_key, elements * 2, "kv store private key");
        require_capacity(private_value, elements * 2, "kv store private value");
        check(guffin_hip_kv_store_f16(stream_, f32(raw_key), f32(raw_value), u32(positions), dev(private_key), dev(private_value),
                                      row_count, head_count, head_dimension, rope_dimension_count, frequency_base,
                                      frequency_scale, numerical_status ? u32(*numerical_status) : status_word()));
        ++stats_.compute_dispatch_count;
    }
    // Schedules are host-written shared storage, complete before this call (:264-266): the launch is sized
    // from them here, on the host.
    void encode_verifier_attention(const BackendBuffer& query, const BackendBuffer& resident_key,
                                   const BackendBuffer& resident_value, const BackendBuffer& private_key,
                                   const BackendBuffer& private_value, const BackendBuffer& schedules,
                                   std::uint64_t schedule_byte_offset, const BackendBuffer& ancestors, const BackendBuffer& output,
                                   const BackendBuffer& partial_output, const BackendBuffer& partial_maxima,
                                   const BackendBuffer& partial_denominators, std::uint32_t row_count,
                                   std::uint32_t cache_row_mask, std::uint32_t query_head_count, std::uint32_t kv_head_count,
                                   std::uint32_t key_dimension, std::uint32_t value_dimension, float scale, float logit_softcap,
                                   const BackendBuffer* q4_input_sums = nullptr) {
        require_encodable();
        if (logit_softcap != 0.0F) throw std::invalid_argument("HIP verifier attention has no logit softcap (Gemma 3 uses none)");
        if (key_dimension != value_dimension) throw std::invalid_argument("HIP verifier attention needs equal key and value widths");
        if (row_count == 0U || row_count > 2U) throw std::invalid_argument("HIP verifier attention takes one or two rows");
        const auto* host = static_cast<const std::byte*>(storage(schedules).host());
        if (host == nullptr || schedule_byte_offset % 16 != 0
            || schedule_byte_offset + std::uint64_t(row_count) * 16 > schedules.descriptor().byte_count)
            throw std::invalid_argument("HIP verifier attention needs host-visible schedule rows");
        std::uint32_t first = UINT32_MAX, last = 0, ancestors_max = 0;
        for (std::uint32_t row = 0; row < row_count; ++row) {   // {base_first_position, base_token_count, ancestor_offset, ancestor_count}
            std::uint32_t s[4];
            std::memcpy(s, host + schedule_byte_offset + row * 16, 16);
            if (s[1] > 0) { first = std::min(first, s[0]); last = std::max(last, s[0] + s[1]); }
            ancestors_max = std::max(ancestors_max, s[3]);
        }
        const auto private_rows = static_cast<std::uint32_t>(private_key.descriptor().shape.dimension(0));
        const std::uint32_t max_tokens = (last > first ? last - first : 0U) + std::max(private_rows, ancestors_max);
        const std::uint32_t partitions = guffin_hip_attention_partitions(max_tokens, kv_head_count);
        const auto heads = std::uint64_t(row_count) * query_head_count;
        require_capacity(partial_output, heads * partitions * value_dimension * 4, "attention partial output");
        // maxima and denominators travel as pairs in one array here: the two buffers must be adjacent views
        // of one allocation of heads * partitions * 2 floats, maxima first.
        if (f32(partial_denominators) != f32(partial_maxima) + heads * partitions)
            throw std::invalid_argument("HIP verifier attention needs maxima and denominators as adjacent halves of one allocation");
        float* sums = nullptr;
        if (q4_input_sums != nullptr) {
            require_capacity(*q4_input_sums, guffin_hip_receipt_bytes(row_count, query_head_count * value_dimension), "activation receipt");
            sums = f32(*q4_input_sums);
        }
        check(guffin_hip_attention_decode(stream_, f32(query), dev(resident_key), dev(resident_value), dev(private_key),
                                          dev(private_value), reinterpret_cast<const std::uint32_t*>(
                                              static_cast<const std::byte*>(storage(schedules).device()) + schedule_byte_offset),
                                          u32(ancestors), f32(output), sums, f32(partial_output), f32(partial_maxima), row_count,
                                          private_rows, max_tokens, cache_row_mask, query_head_count, kv_head_count, key_dimension,
                                          scale, status_word()));
        stats_.compute_dispatch_count += 2;
        ++stats_.decode_attention_dispatch_count;
        stats_.decode_attention_partition_count += partitions;
        stats_.decode_attention_token_count += max_tokens;
    }
    void encode_verifier_kv_scatter(const BackendBuffer& private_key, const BackendBuffer& private_value,
                                    const BackendBuffer& selected_nodes, const BackendBuffer& resident_key,
                                    const BackendBuffer& resident_value, std::uint32_t destination_position,
                                    std::uint32_t row_count, std::uint32_t row_width, std::uint32_t destination_row_mask) {
        require_encodable();
        require_capacity(selected_nodes, std::uint64_t(row_count) * 4, "kv scatter selection");
        check(guffin_hip_kv_scatter(stream_, dev(private_key), dev(private_value), u32(selected_nodes), dev(resident_key),
                                    dev(resident_value), destination_position, row_count, row_width, destination_row_mask));
        ++stats_.compute_dispatch_count;
    }
    void encode_gemma2_kv_cache_copy(const BackendBuffer& source_key, const BackendBuffer& source_value,
                                     const BackendBuffer& destination_key, const BackendBuffer& destination_value,
                                     std::uint32_t position_start, std::uint32_t token_count, std::uint32_t source_row_mask,
                                     std::uint32_t destination_row_mask) {
        require_encodable();
        const auto row_width = dim32(source_key.descriptor(), 1);
        check(guffin_hip_kv_cache_copy(stream_, dev(source_key), dev(source_value), dev(destination_key), dev(destination_value),
                                       position_start, token_count, source_row_mask, destination_row_mask, row_width));
        ++stats_.compute_dispatch_count;
    }
    void encode_f16_prefill_attention(const BackendBuffer& query, const BackendBuffer& key_cache, const BackendBuffer& value_cache,
                                      const BackendBuffer& current_chunk_key, const BackendBuffer& current_chunk_value,
                                      const BackendBuffer& output, std::uint32_t query_position_start, std::uint32_t head_count,
                                      std::uint32_t kv_head_count, std::uint32_t key_length, std::uint32_t value_length,
                                      std::uint32_t attention_token_count, float scale, float logit_softcap,
                                      std::uint32_t cache_row_mask, std::uint32_t query_row_count, bool uses_staged_chunk,
                                      std::uint32_t current_chunk_position_origin = 0U) {
        require_encodable();
        if (logit_softcap != 0.0F || key_length != value_length || !uses_staged_chunk
            || current_chunk_position_origin != query_position_start)
            throw std::invalid_argument("HIP prefill attention takes a staged chunk that starts at the query position, no softcap");
        // attention_token_count is the sliding window of a local layer, or the whole prefix of a global one
        const std::uint32_t window = attention_token_count >= query_position_start + query_row_count ? 0U : attention_token_count;
        require_capacity(output, std::uint64_t(query_row_count) * head_count * value_length * 4, "prefill attention output");
        check(guffin_hip_prefill_attention(stream_, f32(query), dev(key_cache), dev(value_cache), dev(current_chunk_key),
                                           dev(current_chunk_value), f32(output), query_row_count, query_position_start, window,
                                           cache_row_mask, head_count, kv_head_count, key_length, scale, nullptr));
        ++stats_.compute_dispatch_count;
    }
    void encode_gelu_tanh_multiply(const BackendBuffer& gate, const BackendBuffer& up, const BackendBuffer& output,
                                   std::uint64_t element_count = 0, const BackendBuffer* q4_input_sums = nullptr) {
        require_encodable();
        const auto& g = gate.descriptor();
        const auto total = element_count == 0 ? g.element_count : element_count;
        // with a receipt the rows matter (one receipt per row); without, the elements are one long row
        std::uint32_t rows = 1, width = static_cast<std::uint32_t>(total);
        if (q4_input_sums != nullptr) {
            if (g.shape.rank() != 2U || total % g.shape.dimension(1) != 0)
                throw std::invalid_argument("HIP GeGLU with a receipt requires whole matrix rows");
            width = dim32(g, 1);
            rows = static_cast<std::uint32_t>(total / width);
            require_capacity(*q4_input_sums, guffin_hip_receipt_bytes(rows, width), "activation receipt");
        }
        require_capacity(up, total * 4, "GeGLU up");
        require_capacity(output, total * 4, "GeGLU output");
        check(guffin_hip_geglu(stream_, f32(gate), f32(up), 1, 0, f32(output), q4_input_sums ? f32(*q4_input_sums) : nullptr,
                               rows, width));
        ++stats_.compute_dispatch_count;
    }

    void encode_verifier_input_validation(const BackendBuffer& actual_token_ids, std::uint64_t actual_byte_offset,
                                          const BackendBuffer& expected_token_ids, const BackendBuffer& status,
                                          std::uint32_t row_count, std::uint32_t vocabulary_size) {
        require_encodable();
        if (actual_byte_offset % 4 != 0) throw std::invalid_argument("HIP input validation offset must be 4-byte aligned");
        require_capacity(actual_token_ids, actual_byte_offset + std::uint64_t(row_count) * 4, "validated token ids");
        require_capacity(expected_token_ids, std::uint64_t(row_count) * 4, "expected token ids");
        check(guffin_hip_input_validation(stream_, u32(actual_token_ids) + actual_byte_offset / 4, u32(expected_token_ids),
                                          row_count, vocabulary_size, u32(status)));
        ++stats_.compute_dispatch_count;
    }
    void encode_verifier_selection_requests(const BackendBuffer& raw_requests, std::uint64_t raw_byte_offset,
                                            const BackendBuffer& resolved_requests, const BackendBuffer& histories,
                                            const BackendBuffer& status, std::uint32_t row_count,
                                            const engine::TokenSamplerOptions& options, std::uint32_t vocabulary_size) {
        require_encodable();
        // raw rows are engine::VerifierDeviceSelectionRow records (target_verifier.hpp:114-121), the layout of guffin_selection_row
        require_capacity(raw_requests, raw_byte_offset + std::uint64_t(row_count) * sizeof(guffin_selection_row), "raw selection requests");
        require_capacity(resolved_requests, std::uint64_t(row_count) * sizeof(guffin_resolved_row), "resolved selection requests");
        require_capacity(histories, std::uint64_t(row_count) * 64 * 4, "selection histories");
        const auto top_k = static_cast<std::uint32_t>(options.temperature == 0.0F ? 1U : options.top_k);
        check(guffin_hip_selection_requests(stream_, static_cast<const std::byte*>(dev(raw_requests)) + raw_byte_offset, row_count,
                                            vocabulary_size, top_k, options.repetition_penalty != 1.0F ? 1U : 0U,
                                            dev(resolved_requests), u32(histories), u32(status)));
        ++stats_.compute_dispatch_count;
    }

    // One or two logit rows against host-side requests (:326-337).  Returns the launches encoded.
    template <class SelectionWorkspace>
    [[nodiscard]] std::uint32_t encode_token_candidates(const BackendBuffer& logits, const SelectionWorkspace& workspace,
                                                        const engine::TokenSelectionRequest& request, float softcap) {
        return candidates(logits, workspace, {&request, 1}, softcap);
    }
    template <class SelectionWorkspace>
    [[nodiscard]] std::uint32_t encode_token_candidates_width_two(const BackendBuffer& logits, const SelectionWorkspace& workspace,
                                                                  const std::array<engine::TokenSelectionRequest, 2>& requests,
                                                                  float softcap) {
        return candidates(logits, workspace, requests, softcap);
    }
    // Rows of a verify pass against the requests resolved on the device (:338).
    template <class TargetWorkspace>
    [[nodiscard]] std::uint32_t encode_target_token_candidates(const BackendBuffer& logits_tile, const TargetWorkspace& workspace,
                                                               std::uint32_t first_request_row, std::uint32_t row_count,
                                                               float softcap, bool /*greedy_without_history*/) {
        require_encodable();
        if (softcap != 0.0F) throw std::invalid_argument("HIP candidate selection has no softcap (Gemma 3 uses none)");
        if (row_count == 0U || first_request_row > workspace.row_capacity || row_count > workspace.row_capacity - first_request_row)
            throw std::invalid_argument("HIP target-candidate row tile is invalid");
        const auto vocab = dim32(logits_tile.descriptor(), 1);
        require_capacity(workspace.candidate_runs_a, guffin_hip_select_workspace_bytes(row_count, vocab, kCandidateCapacity),
                         "candidate selection workspace");
        require_capacity(workspace.compact_results, std::uint64_t(first_request_row + row_count) * kResultStride, "candidate results");
        auto* results = static_cast<std::byte*>(dev(workspace.compact_results)) + std::size_t(first_request_row) * kResultStride;
        const auto* resolved = static_cast<const std::byte*>(dev(workspace.resolved_request_staging))
            + std::size_t(first_request_row) * sizeof(guffin_resolved_row);
        // a greedy request resolves to top_k = 1 and no history, so the same call serves it
        check(guffin_hip_select_candidates_resolved(stream_, f32(logits_tile), row_count, vocab,
                                                    std::min<std::uint32_t>(kCandidateCapacity, vocab), resolved,
                                                    dev(workspace.candidate_runs_a), results, row_status(row_count)));
        stats_.compute_dispatch_count += 2;
        return 2U;
    }

    void encode_memory_barrier() { require_encodable(); ++stats_.memory_barrier_count; }   // one in-order stream: nothing to enqueue
    void push_debug_group(std::string_view) {}
    void pop_debug_group() {}

    HipCommandStats commit() {
        require_encodable();
        check_hip(hipEventRecord(batch_end_, stream_), "event record failed");
        submitted_ = true;
        ++stats_.commit_count;
        return stats_;
    }
    HipCommandStats wait_until_completed() {
        if (!submitted_) throw std::logic_error("HIP command context waited before commit");
        if (hipStreamSynchronize(stream_) != hipSuccess) throw_hip("the stream failed");
        if (!completed_) {
            float ms = 0.0F;
            if (started_ && hipEventElapsedTime(&ms, batch_start_, batch_end_) == hipSuccess)
                stats_.gpu_duration_ns = static_cast<std::uint64_t>(static_cast<double>(ms) * 1e6);
            else
                stats_.gpu_duration_ns = 0;
        }
        completed_ = true;
        ++stats_.synchronous_wait_count;
        return stats_;
    }
    [[nodiscard]] HipCommandStats completion_stats() const { return stats_; }
    HipCommandStats commit_and_wait() {
        static_cast<void>(commit());
        return wait_until_completed();
    }

    template <class SelectionWorkspace>
    [[nodiscard]] engine::CompactTokenCandidates read_token_candidates(const SelectionWorkspace& workspace) const {
        std::array<engine::CompactTokenCandidates, 1> out;
        read_rows(workspace.compact_result, 0, out);
        return out[0];
    }
    template <class SelectionWorkspace>
    [[nodiscard]] std::array<engine::CompactTokenCandidates, 2> read_token_candidates_width_two(
        const SelectionWorkspace& workspace) const {
        std::array<engine::CompactTokenCandidates, 2> out;
        read_rows(workspace.compact_result, 0, out);
        return out;
    }
    template <class TargetWorkspace>
    void read_target_token_candidates(const TargetWorkspace& workspace, std::uint32_t first_row,
                                      std::span<engine::CompactTokenCandidates> output) const {
        if (first_row > workspace.row_capacity || output.size() > workspace.row_capacity - first_row)
            throw std::invalid_argument("HIP target candidate readback extent is invalid");
        read_rows(workspace.compact_results, first_row, output);
    }
    [[nodiscard]] std::uint32_t read_verifier_status(const BackendBuffer& status) const {
        require_completed("status");
        std::uint32_t word = 0;
        check_hip(hipMemcpy(&word, dev(status), 4, hipMemcpyDeviceToHost), "status readback failed");
        return word;
    }
    // The operators' own status word (GUFFIN_STATUS_* bits of every encode of this context).
    [[nodiscard]] std::uint32_t read_operator_status() const {
        require_completed("status");
        std::uint32_t word = 0;
        check_hip(hipMemcpy(&word, meta_, 4, hipMemcpyDeviceToHost), "status readback failed");
        return word;
    }

private:
    static constexpr std::uint32_t kCandidateCapacity = 320;                 // token_sampler_max_candidates
    static constexpr std::size_t kResultStride = 8 + 384 * sizeof(engine::TokenLogit);   // {count, status, values[384]}
    // meta_: [0] operator status, [1..2] per-row selection status, [16..] two resolved requests of host-side calls
    static constexpr std::uint32_t kMetaRowStatus = 1, kMetaResolved = 16, kMetaWords = 16 + 2 * 68;

    // every encode passes here first: the batch's first one also marks its start on the stream
    void require_encodable() {
        if (submitted_) throw std::logic_error("HIP command context is already committed");
        if (!started_) {
            check_hip(hipEventRecord(batch_start_, stream_), "event record failed");
            started_ = true;
            ++stats_.command_buffer_count;
        }
    }
    void require_completed(const char* what) const {
        if (!completed_) throw std::logic_error(std::string("HIP ") + what + " cannot be read before completion");
    }
    static void require_capacity(const BackendBuffer& buffer, std::uint64_t bytes, const char* what) {
        if (buffer.descriptor().byte_count < bytes) throw std::invalid_argument(std::string("HIP ") + what + " is too small");
    }
    [[nodiscard]] static void* dev(const BackendBuffer& b) { return storage(b).device(); }
    [[nodiscard]] static float* f32(const BackendBuffer& b) { return static_cast<float*>(dev(b)); }
    [[nodiscard]] static std::uint32_t* u32(const BackendBuffer& b) { return static_cast<std::uint32_t*>(dev(b)); }
    [[nodiscard]] static std::uint32_t dim32(const TensorDescriptor& d, std::size_t index) {
        const auto v = d.shape.dimension(index);
        if (v > UINT32_MAX) throw std::invalid_argument("HIP backend: dimension exceeds 32 bits");
        return static_cast<std::uint32_t>(v);
    }
    void count_projection(int dtype, std::uint32_t rows, bool part_of_a_batch) {
        if (dtype == GUFFIN_Q4_K) ++(part_of_a_batch ? stats_.q4_small_batch_projection_count : rows == 2U ? stats_.q4_width_two_projection_count : stats_.q4_decode_projection_count);
        else if (dtype == GUFFIN_Q6_K) ++(part_of_a_batch ? stats_.q6_small_batch_projection_count : rows == 2U ? stats_.q6_width_two_projection_count : stats_.q6_decode_projection_count);
        else ++(rows == 2U ? stats_.q8_width_two_projection_count : stats_.q8_decode_projection_count);
    }
    [[nodiscard]] std::uint32_t* status_word() const { return meta_; }
    [[nodiscard]] std::uint32_t* row_status(std::uint32_t rows) {
        static constexpr std::uint32_t zeros[2] = {0, 0};   // a copy, not a memset: the stream may be under graph capture
        check_hip(hipMemcpyAsync(meta_ + kMetaRowStatus, zeros, std::min(rows, 2U) * 4, hipMemcpyHostToDevice, stream_),
                  "clearing status failed");
        return meta_ + kMetaRowStatus;
    }
    // The consumer's own receipt when the producer left none (q4_input_sums == nullptr).
    [[nodiscard]] const float* make_receipt(const float* x, std::uint32_t rows, std::uint32_t K) {
        if (guffin_hip_receipt_bytes(rows, K) > scratch_floats_ * sizeof(float))
            throw std::invalid_argument("HIP activation receipt exceeds the context's scratch");
        check(guffin_hip_group_sums(stream_, x, static_cast<float*>(receipt_), rows, K));
        ++stats_.compute_dispatch_count;
        return static_cast<const float*>(receipt_);
    }
    void gemv(int dtype, const void* tiles, const float* x, const float* sums, float* y, std::uint32_t rows, std::uint32_t K,
              std::uint32_t N) {
        const std::uint64_t slices = guffin_hip_gemv_packed_slices(dtype, K, N);
        if (slices == 0) throw std::invalid_argument(guffin_hip_last_error());
        if (slices > 1 && slices * rows * N > scratch_floats_) throw std::invalid_argument("HIP GEMV partial planes exceed the context's scratch");
        check(guffin_hip_gemv_packed(stream_, dtype, tiles, x, sums, static_cast<float*>(scratch_), y, rows, K, N));
        stats_.compute_dispatch_count += slices > 1 ? 2 : 1;
    }
    void norm(const BackendBuffer& input, const BackendBuffer& weight, const BackendBuffer* residual, const BackendBuffer& output,
              float epsilon, std::uint32_t row_count, std::uint32_t input_row_start, const BackendBuffer* q4_input_sums) {
        require_encodable();
        const auto& in = input.descriptor();
        if (in.shape.rank() != 2U) throw std::invalid_argument("HIP RMS norm requires matrix input rows");
        const auto width = dim32(in, 1);
        const auto available = dim32(in, 0);
        if (input_row_start > available) throw std::invalid_argument("HIP RMS norm row start is invalid");
        const auto rows = row_count == 0U ? available - input_row_start : row_count;
        if (rows == 0U || rows > available - input_row_start) throw std::invalid_argument("HIP RMS norm row count is invalid");
        require_capacity(weight, std::uint64_t(width) * 4, "RMS norm weight");
        require_capacity(output, std::uint64_t(rows) * width * 4, "RMS norm output");
        if (residual) require_capacity(*residual, std::uint64_t(rows) * width * 4, "RMS norm residual");
        if (q4_input_sums) require_capacity(*q4_input_sums, guffin_hip_receipt_bytes(rows, width), "activation receipt");
        check(guffin_hip_rms_norm(stream_, f32(input) + std::size_t(input_row_start) * width, 1, 0, f32(weight),
                                  residual ? f32(*residual) : nullptr, f32(output), q4_input_sums ? f32(*q4_input_sums) : nullptr,
                                  rows, width, epsilon, status_word()));
        ++stats_.compute_dispatch_count;
    }
    template <class SelectionWorkspace>
    std::uint32_t candidates(const BackendBuffer& logits, const SelectionWorkspace& workspace,
                             std::span<const engine::TokenSelectionRequest> requests, float softcap) {
        require_encodable();
        if (!std::isfinite(softcap) || softcap != 0.0F) throw std::invalid_argument("HIP candidate selection has no softcap (Gemma 3 uses none)");
        const auto rows = static_cast<std::uint32_t>(requests.size());
        const auto vocab = dim32(logits.descriptor(), logits.descriptor().shape.rank() - 1);
        std::array<guffin_resolved_row, 2> resolved {};
        std::uint32_t capacity = 1;
        for (std::uint32_t row = 0; row < rows; ++row) {
            const auto& request = requests[row];
            if (request.top_k == 0U || request.top_k > engine::token_sampler_max_base_candidates
                || request.history_token_count > engine::token_sampler_max_repetition_window
                || request.base_candidate_count != request.top_k + request.history_token_count)
                throw std::invalid_argument("HIP token-candidate request is outside product bounds");
            resolved[row].top_k = request.top_k;
            resolved[row].base_candidate_count = request.base_candidate_count;
            resolved[row].history_count = request.history_token_count;
            std::copy_n(request.history_token_ids.begin(), request.history_token_count, resolved[row].history_token_ids);
            capacity = std::max(capacity, request.base_candidate_count);
        }
        capacity = std::min(capacity, vocab);
        require_capacity(workspace.candidate_runs_a, guffin_hip_select_workspace_bytes(rows, vocab, capacity), "candidate selection workspace");
        require_capacity(workspace.compact_result, std::uint64_t(rows) * kResultStride, "candidate results");
        check_hip(hipMemcpyWithStream(meta_ + kMetaResolved, resolved.data(), rows * sizeof(guffin_resolved_row), hipMemcpyHostToDevice,
                                 stream_), "request upload failed");
        check(guffin_hip_select_candidates_resolved(stream_, f32(logits), rows, vocab, capacity, meta_ + kMetaResolved,
                                                    dev(workspace.candidate_runs_a), dev(workspace.compact_result), row_status(rows)));
        stats_.compute_dispatch_count += 2;
        return 2U;
    }
    void read_rows(const BackendBuffer& results, std::uint32_t first_row, std::span<engine::CompactTokenCandidates> output) const {
        require_completed("candidates");
        require_capacity(results, (std::uint64_t(first_row) + output.size()) * kResultStride, "candidate results");
        std::vector<std::byte> bytes(output.size() * kResultStride);
        check_hip(hipMemcpy(bytes.data(), static_cast<const std::byte*>(dev(results)) + std::size_t(first_row) * kResultStride,
                            bytes.size(), hipMemcpyDeviceToHost), "candidate readback failed");
        for (std::size_t row = 0; row < output.size(); ++row) {
            const auto* record = bytes.data() + row * kResultStride;
            std::uint32_t header[2];   // {count, status}
            std::memcpy(header, record, 8);
            if (header[1] != 0U)   // the reference throws on both faults (metal_command_context.mm:2482-2490)
                throw std::invalid_argument("HIP target-candidate row " + std::to_string(first_row + row)
                                            + ((header[1] & GUFFIN_STATUS_BAD_TOKEN) ? " history token is outside vocabulary"
                                                                                     : " logit must be finite"));
            if (header[0] == 0U || header[0] > engine::token_sampler_max_candidates)
                throw std::runtime_error("HIP target-candidate result count is invalid");
            output[row].count = header[0];
            output[row].readback_bytes = header[0] * static_cast<std::uint32_t>(sizeof(engine::TokenLogit));
            std::memcpy(output[row].values.data(), record + 8, output[row].readback_bytes);
        }
    }

    std::string label_;
    hipStream_t stream_ = nullptr;
    void* scratch_ = nullptr;    // k-slice partial planes of the GEMV being encoded
    void* receipt_ = nullptr;    // self-made activation receipt / prefill operand image
    std::uint32_t* meta_ = nullptr;
    std::size_t scratch_floats_;
    hipEvent_t batch_start_ = nullptr, batch_end_ = nullptr;
    bool submitted_ = false, completed_ = false, started_ = false;
    HipCommandStats stats_;
};

}  // namespace local_gguf_engine::tensor::backends::hip
