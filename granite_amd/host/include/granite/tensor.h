// Tensor: a shaped, strided view of a backend buffer (reference:
// include/granite/tensor.h:19-199, src/core/tensor.cpp:34-102).  Only what the
// attention path touches is restated: allocation in managed memory, mapping,
// views, dim-0 slices, clone/copy.
#pragma once

#include <span>
#include <vector>

#include "granite/backend.h"

namespace granite {

class Tensor {
  public:
    Tensor() = default;

    // Managed allocation on `backend`.  Errors follow src/core/tensor.cpp:34-74:
    // null backend -> NullPointer, backend down -> BackendNotInitialized, empty or
    // non-positive shape -> InvalidShape, larger than the device limit -> OutOfMemory.
    static Result<Tensor> allocate(std::span<const int64_t> shape, DataType dtype,
                                   IComputeBackend* backend);
    static Result<Tensor> allocate(std::initializer_list<int64_t> shape, DataType dtype,
                                   IComputeBackend* backend) {
        return allocate(std::span<const int64_t>(shape.begin(), shape.size()), dtype, backend);
    }
    // Wraps an existing buffer; the tensor does not own it.
    static Tensor from_buffer(BufferHandle buffer, std::span<const int64_t> shape, DataType dtype,
                              IComputeBackend* backend, size_t offset = 0);

    [[nodiscard]] std::span<const int64_t> shape() const { return shape_; }
    [[nodiscard]] std::span<const int64_t> strides() const { return strides_; }
    [[nodiscard]] DataType dtype() const { return dtype_; }
    [[nodiscard]] size_t ndim() const { return shape_.size(); }
    // Negative dims count from the back (size(-1) is the innermost extent).
    [[nodiscard]] int64_t size(int64_t dim) const {
        if (dim < 0) dim += static_cast<int64_t>(shape_.size());
        return shape_.at(static_cast<size_t>(dim));
    }
    [[nodiscard]] size_t numel() const {
        if (shape_.empty()) return 0;
        size_t n = 1;
        for (auto d : shape_) n *= static_cast<size_t>(d);
        return n;
    }
    [[nodiscard]] size_t size_bytes() const { return numel() * dtype_size(dtype_); }
    [[nodiscard]] bool is_contiguous() const;
    [[nodiscard]] bool empty() const { return numel() == 0; }
    [[nodiscard]] bool valid() const { return buffer_.valid(); }
    [[nodiscard]] BufferHandle buffer() const { return buffer_; }
    [[nodiscard]] size_t buffer_offset() const { return offset_; }
    [[nodiscard]] IComputeBackend* backend() const { return backend_; }

    // Host pointer to the first element (maps the buffer; see unmap()).
    template <typename T>
    Result<T*> data() {
        if (!backend_ || !buffer_.valid()) return Error(ErrorCode::InvalidState, "Tensor has no buffer");
        auto mapped = backend_->map_buffer(buffer_);
        if (!mapped.ok()) return mapped.error();
        return reinterpret_cast<T*>(static_cast<char*>(mapped.value()) + offset_);
    }
    template <typename T>
    Result<const T*> data() const {
        if (!backend_ || !buffer_.valid()) return Error(ErrorCode::InvalidState, "Tensor has no buffer");
        auto mapped = backend_->map_buffer(buffer_);
        if (!mapped.ok()) return mapped.error();
        return reinterpret_cast<const T*>(static_cast<const char*>(mapped.value()) + offset_);
    }
    // Ends host access; on a discrete GPU this is what publishes host writes.
    void unmap() const {
        if (backend_ && buffer_.valid()) backend_->unmap_buffer(buffer_);
    }

    [[nodiscard]] Result<Tensor> view(std::span<const int64_t> new_shape) const;
    [[nodiscard]] Result<Tensor> slice(size_t dim, int64_t start, int64_t end) const;
    [[nodiscard]] Result<Tensor> clone() const;
    Result<void> copy_from(const Tensor& src);

    static std::vector<int64_t> compute_strides(std::span<const int64_t> shape);

  private:
    BufferHandle buffer_{};
    size_t offset_ = 0;
    std::vector<int64_t> shape_;
    std::vector<int64_t> strides_;
    DataType dtype_ = DataType::FP32;
    IComputeBackend* backend_ = nullptr;
};

}  // namespace granite
