// RoPECache over the HIP library (interface: include/granite/llm.h:173-197 of the reference).
#include "granite/rope.h"

#include <cmath>
#include <string>

#include "granite/hip_backend.h"
#include "granite/hip_compute.h"
#include "granite_hip.h"

namespace granite {

RoPECache::~RoPECache() {
    if (table_backend_) {
        table_backend_->destroy_buffer(cos_dev_);
        table_backend_->destroy_buffer(sin_dev_);
    }
}

// src/llm/rope.cpp:5-22, the same float expressions: the table is what the rotation's
// bit-exactness rests on.
void RoPECache::initialize(int max_seq_len, int head_dim, float theta) {
    if (table_backend_) {
        table_backend_->destroy_buffer(cos_dev_);
        table_backend_->destroy_buffer(sin_dev_);
        table_backend_ = nullptr;
    }
    max_seq_len_ = max_seq_len;
    head_dim_ = head_dim;
    const int half_dim = head_dim / 2;
    cos_.resize(static_cast<size_t>(max_seq_len) * half_dim);
    sin_.resize(static_cast<size_t>(max_seq_len) * half_dim);
    for (int pos = 0; pos < max_seq_len; pos++) {
        for (int i = 0; i < half_dim; i++) {
            float freq = 1.0f / std::pow(theta, static_cast<float>(2 * i) / head_dim);
            float angle = static_cast<float>(pos) * freq;
            cos_[static_cast<size_t>(pos) * half_dim + i] = std::cos(angle);
            sin_[static_cast<size_t>(pos) * half_dim + i] = std::sin(angle);
        }
    }
}

Result<void> RoPECache::ensure_device_tables(IComputeBackend* backend) {
    if (table_backend_ == backend) return {};
    if (table_backend_) {
        table_backend_->destroy_buffer(cos_dev_);
        table_backend_->destroy_buffer(sin_dev_);
        table_backend_ = nullptr;
    }
    const BufferDesc desc = BufferDesc::device(cos_.size() * sizeof(float));
    auto made_cos = backend->create_buffer_from_host(cos_.data(), desc);
    if (!made_cos.ok()) return made_cos.error();
    auto made_sin = backend->create_buffer_from_host(sin_.data(), desc);
    if (!made_sin.ok()) {
        backend->destroy_buffer(made_cos.value());
        return made_sin.error();
    }
    cos_dev_ = made_cos.value();
    sin_dev_ = made_sin.value();
    table_backend_ = backend;
    return {};
}

Result<std::pair<const float*, const float*>> RoPECache::device_tables(IComputeBackend* backend) {
    if (!is_initialized()) return Error(ErrorCode::InvalidState, "RoPE cache not initialized");
    if (!backend || backend->get_type() != BackendType::HIP)
        return Error(ErrorCode::BackendNotSupported, "RoPE tables live on the HIP backend only");
    GRANITE_TRY(ensure_device_tables(backend));
    const auto* c = static_cast<const float*>(hip_device_pointer(backend, cos_dev_));
    const auto* s = static_cast<const float*>(hip_device_pointer(backend, sin_dev_));
    if (!c || !s) return Error(ErrorCode::InternalError, "RoPE tables are not on the device");
    return std::pair<const float*, const float*>{c, s};
}

Result<void> RoPECache::apply(Tensor& q, Tensor& k, int start_pos, IComputeBackend* backend) {
    return run(q, k, nullptr, nullptr, nullptr, start_pos, backend);
}

Result<void> RoPECache::apply_and_append(Tensor& q, Tensor& k, const Tensor& v, Tensor& cache_k,
                                         Tensor& cache_v, int start_pos, IComputeBackend* backend) {
    return run(q, k, &v, &cache_k, &cache_v, start_pos, backend);
}

Result<void> RoPECache::run(Tensor& q, Tensor& k, const Tensor* v, Tensor* cache_k, Tensor* cache_v,
                            int start_pos, IComputeBackend* backend) {
    if (!is_initialized()) return Error(ErrorCode::InvalidState, "RoPE cache not initialized");
    if (q.ndim() != 4 || k.ndim() != 4 || q.size(3) != head_dim_ || k.size(3) != head_dim_ ||
        q.size(1) != k.size(1) || q.size(0) != 1 || k.size(0) != 1)
        return Error(ErrorCode::ShapeMismatch, "RoPE takes [1, seq_len, num_heads, head_dim] Q and K");
    if (q.dtype() != DataType::FP32 || k.dtype() != DataType::FP32)
        return Error(ErrorCode::DTypeMismatch, "RoPE rotates FP32 tensors");
    const int seq_len = static_cast<int>(q.size(1));
    if (start_pos < 0 || start_pos + seq_len > max_seq_len_)
        return Error(ErrorCode::InvalidArgument,
                     "RoPE position out of range: " + std::to_string(start_pos) + " + " +
                         std::to_string(seq_len) + " > " + std::to_string(max_seq_len_));
    if (!backend || backend->get_type() != BackendType::HIP)
        return Error(ErrorCode::BackendNotSupported, "RoPECache::apply runs on the HIP backend only");
    GRANITE_TRY(ensure_device_tables(backend));

    auto ptr = [&](const Tensor& t) -> char* {
        auto* p = static_cast<char*>(hip_device_pointer(backend, t.buffer()));
        return p ? p + t.buffer_offset() : nullptr;
    };
    granite_hip_rope_args a{};
    a.q = ptr(q);
    a.k = ptr(k);
    a.num_heads_q = static_cast<uint32_t>(q.size(2));
    a.num_heads_k = static_cast<uint32_t>(k.size(2));
    a.seq_len = static_cast<uint32_t>(seq_len);
    a.head_dim = static_cast<uint32_t>(head_dim_);
    a.start_pos = static_cast<uint32_t>(start_pos);
    a.cos_table = static_cast<const float*>(hip_device_pointer(backend, cos_dev_));
    a.sin_table = static_cast<const float*>(hip_device_pointer(backend, sin_dev_));
    a.table_positions = static_cast<uint32_t>(max_seq_len_);
    a.write_k_back = 1;
    a.rounding = GRANITE_HIP_ROUND_NEAREST;
    if (!a.q || !a.k || !a.cos_table || !a.sin_table)
        return Error(ErrorCode::InternalError, "Tensor buffers do not belong to the HIP backend");
    if (v) {
        if (v->ndim() != 4 || v->size(1) != k.size(1) || v->size(2) != k.size(2) ||
            v->size(3) != head_dim_ || cache_k->ndim() != 3 || cache_k->size(0) != k.size(2) ||
            cache_k->size(2) != head_dim_ || cache_v->ndim() != 3 ||
            cache_v->size(0) != cache_k->size(0) || cache_v->size(1) != cache_k->size(1) ||
            cache_v->size(2) != head_dim_)
            return Error(ErrorCode::ShapeMismatch,
                         "append takes V like K and caches [num_kv_heads, max_len, head_dim]");
        if (v->dtype() != DataType::FP32 || cache_k->dtype() != DataType::FP16 ||
            cache_v->dtype() != DataType::FP16)
            return Error(ErrorCode::DTypeMismatch, "V is FP32, the cache rows are FP16");
        if (start_pos + seq_len > cache_k->size(1))
            return Error(ErrorCode::InvalidArgument, "KV cache overflow");
        a.v = ptr(*v);
        a.cache_k = ptr(*cache_k);
        a.cache_v = ptr(*cache_v);
        a.max_seq_len = static_cast<uint32_t>(cache_k->size(1));
        if (!a.v || !a.cache_k || !a.cache_v)
            return Error(ErrorCode::InternalError, "Tensor buffers do not belong to the HIP backend");
    }
    HipCompute compute;
    return compute.rope_append(a);
}

}  // namespace granite
