// The backend-independent part of the reference's BackendBuffer facade, which its tree defines inside an
// Objective-C++ file (src/tensor/backend_buffer.mm:24-45) next to the Metal arms: what a maintainer moves into a
// portable translation unit when a second device backend is added.  The members' behaviour is fixed by their
// declarations (include/local_gguf_engine/tensor/backend_buffer.hpp:17-70).
#include "local_gguf_engine/tensor/backend_buffer.hpp"

#include <stdexcept>
#include <utility>

namespace local_gguf_engine::tensor {

namespace detail {
BackendBufferStorage::~BackendBufferStorage() = default;

BackendBuffer make_backend_buffer(std::shared_ptr<BackendBufferStorage> storage) { return BackendBuffer(std::move(storage)); }
}  // namespace detail

BackendBuffer::BackendBuffer(std::shared_ptr<detail::BackendBufferStorage> storage) : storage_(std::move(storage)) {
    if (!storage_) throw std::invalid_argument("backend buffer storage is null");
}

runtime::BackendKind BackendBuffer::backend() const noexcept { return storage_->backend(); }

const TensorDescriptor& BackendBuffer::descriptor() const noexcept { return storage_->descriptor(); }

const detail::BackendBufferStorage& backend_buffer_storage(const BackendBuffer& buffer) noexcept { return *buffer.storage_; }

}  // namespace local_gguf_engine::tensor
