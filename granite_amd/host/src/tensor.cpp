// Tensor: shape/stride bookkeeping over backend buffers.
#include "granite/tensor.h"

namespace granite {

std::vector<int64_t> Tensor::compute_strides(std::span<const int64_t> shape) {
    std::vector<int64_t> strides(shape.size());
    int64_t run = 1;
    for (size_t i = shape.size(); i-- > 0;) {
        strides[i] = run;
        run *= shape[i];
    }
    return strides;
}

Result<Tensor> Tensor::allocate(std::span<const int64_t> shape, DataType dtype,
                                IComputeBackend* backend) {
    if (!backend) return Error(ErrorCode::NullPointer, "Backend is null");
    if (!backend->is_initialized())
        return Error(ErrorCode::BackendNotInitialized, "Backend not initialized");
    if (shape.empty()) return Error(ErrorCode::InvalidShape, "Shape cannot be empty");
    size_t count = 1;
    for (int64_t d : shape) {
        if (d <= 0) return Error(ErrorCode::InvalidShape, "Shape dimensions must be positive");
        count *= static_cast<size_t>(d);
    }
    const size_t bytes = count * dtype_size(dtype);
    const size_t limit = backend->get_capabilities().max_buffer_size;
    if (bytes > limit)
        return Error(ErrorCode::OutOfMemory, "Tensor of " + std::to_string(bytes) +
                                                 " bytes exceeds the device limit of " +
                                                 std::to_string(limit));
    auto made = backend->create_buffer(BufferDesc::managed(bytes));
    if (!made.ok()) return made.error();
    return from_buffer(made.value(), shape, dtype, backend);
}

Tensor Tensor::from_buffer(BufferHandle buffer, std::span<const int64_t> shape, DataType dtype,
                           IComputeBackend* backend, size_t offset) {
    Tensor t;
    t.buffer_ = buffer;
    t.offset_ = offset;
    t.shape_.assign(shape.begin(), shape.end());
    t.strides_ = compute_strides(shape);
    t.dtype_ = dtype;
    t.backend_ = backend;
    return t;
}

bool Tensor::is_contiguous() const {
    int64_t run = 1;
    for (size_t i = shape_.size(); i-- > 0;) {
        if (shape_[i] != 1 && strides_[i] != run) return false;
        run *= shape_[i];
    }
    return true;
}

Result<Tensor> Tensor::view(std::span<const int64_t> new_shape) const {
    if (!is_contiguous()) return Error(ErrorCode::InvalidState, "view() needs a contiguous tensor");
    size_t count = new_shape.empty() ? 0 : 1;
    for (int64_t d : new_shape) {
        if (d <= 0) return Error(ErrorCode::InvalidShape, "Shape dimensions must be positive");
        count *= static_cast<size_t>(d);
    }
    if (count != numel()) return Error(ErrorCode::ShapeMismatch, "view() must keep the element count");
    return from_buffer(buffer_, new_shape, dtype_, backend_, offset_);
}

Result<Tensor> Tensor::slice(size_t dim, int64_t start, int64_t end) const {
    if (dim >= shape_.size()) return Error(ErrorCode::InvalidArgument, "slice() dimension out of range");
    if (start < 0 || end > shape_[dim] || start >= end)
        return Error(ErrorCode::InvalidArgument, "slice() range out of bounds");
    Tensor t = *this;
    t.offset_ += static_cast<size_t>(start * strides_[dim]) * dtype_size(dtype_);
    t.shape_[dim] = end - start;
    return t;
}

Result<Tensor> Tensor::clone() const {
    if (!valid()) return Error(ErrorCode::InvalidState, "Tensor has no buffer");
    if (!is_contiguous()) return Error(ErrorCode::NotImplemented, "clone() of a strided tensor");
    auto made = allocate(shape_, dtype_, backend_);
    if (!made.ok()) return made.error();
    GRANITE_TRY(backend_->copy_buffer(buffer_, made.value().buffer_, size_bytes(), offset_, 0));
    return made;
}

Result<void> Tensor::copy_from(const Tensor& src) {
    if (!valid() || !src.valid()) return Error(ErrorCode::InvalidState, "Tensor has no buffer");
    if (src.dtype_ != dtype_) return Error(ErrorCode::DTypeMismatch, "copy_from() dtype mismatch");
    if (src.shape_ != shape_) return Error(ErrorCode::ShapeMismatch, "copy_from() shape mismatch");
    if (!is_contiguous() || !src.is_contiguous())
        return Error(ErrorCode::NotImplemented, "copy_from() of strided tensors");
    if (src.backend_ != backend_) return Error(ErrorCode::InvalidArgument, "copy_from() across backends");
    return backend_->copy_buffer(src.buffer_, buffer_, size_bytes(), src.offset_, offset_);
}

}  // namespace granite
