// PagedDecodeBatch: block-table / length assembly and the two launches per layer of a
// batched decode step (the integration src/llm/batch_scheduler.cpp:391-452 leaves open).
#include "granite/paged_batch.h"

#include <string>

#include "granite/hip_backend.h"
#include "granite/hip_compute.h"
#include "granite_hip.h"

namespace granite {

Result<void> PagedDecodeBatch::initialize(PagedKVPool* pool, int max_batch, int max_blocks_per_seq,
                                          IComputeBackend* backend) {
    if (!pool || !pool->is_initialized())
        return Error(ErrorCode::InvalidState, "PagedKVPool not initialized");
    if (max_batch <= 0 || max_blocks_per_seq <= 0)
        return Error(ErrorCode::InvalidArgument, "Batch and block-table sizes must be positive");
    if (!backend || backend->get_type() != BackendType::HIP)
        return Error(ErrorCode::BackendNotSupported, "PagedDecodeBatch runs on the HIP backend only");
    pool_ = pool;
    backend_ = backend;
    max_batch_ = max_batch;
    max_blocks_ = max_blocks_per_seq;
    batch_ = 0;
    GRANITE_TRY_ASSIGN(tables, Tensor::allocate({max_batch, max_blocks_per_seq}, DataType::INT32, backend));
    GRANITE_TRY_ASSIGN(lens, Tensor::allocate({max_batch}, DataType::INT32, backend));
    GRANITE_TRY_ASSIGN(positions, Tensor::allocate({max_batch}, DataType::INT32, backend));
    tables_ = std::move(tables);
    lens_ = std::move(lens);
    positions_ = std::move(positions);
    host_tables_.assign(size_t(max_batch) * max_blocks_per_seq, 0);
    host_lens_.assign(max_batch, 0);
    host_positions_.assign(max_batch, -1);
    return {};
}

Result<std::vector<int>> PagedDecodeBatch::begin_step(std::span<const int> slots) {
    if (!pool_) return Error(ErrorCode::InvalidState, "PagedDecodeBatch not initialized");
    if (slots.empty() || static_cast<int>(slots.size()) > max_batch_)
        return Error(ErrorCode::InvalidArgument,
                     "Batch of " + std::to_string(slots.size()) + " sequences, at most " +
                         std::to_string(max_batch_));
    const int block_size = pool_->block_manager().block_size();
    std::vector<int> failed;
    batch_ = static_cast<int>(slots.size());
    for (int b = 0; b < batch_; ++b) {
        PagedKVCache& cache = pool_->get_cache(slots[b]);
        int32_t* row = host_tables_.data() + size_t(b) * max_blocks_;
        const bool fits = (cache.seq_len() + 1 + block_size - 1) / block_size <= max_blocks_;
        if (!fits || !cache.append_tokens(1)) {
            // src/llm/batch_scheduler.cpp:433-437: the request fails, the others go on
            failed.push_back(slots[b]);
            host_lens_[b] = 0;
            host_positions_[b] = -1;
            continue;
        }
        const std::vector<int>& table = cache.block_table();
        for (size_t i = 0; i < table.size(); ++i) row[i] = table[i];
        host_lens_[b] = cache.seq_len();
        host_positions_[b] = cache.seq_len() - 1;
    }
    std::vector<int32_t> lens32(host_lens_.begin(), host_lens_.begin() + batch_);
    GRANITE_TRY(backend_->write_buffer(tables_.buffer(), host_tables_.data(),
                                       size_t(batch_) * max_blocks_ * sizeof(int32_t)));
    GRANITE_TRY(backend_->write_buffer(lens_.buffer(), lens32.data(), lens32.size() * sizeof(int32_t)));
    GRANITE_TRY(backend_->write_buffer(positions_.buffer(), host_positions_.data(),
                                       size_t(batch_) * sizeof(int32_t)));
    return failed;
}

Result<void> PagedDecodeBatch::run_layer(int layer, Tensor& q, Tensor& k, const Tensor& v, Tensor& out,
                                         float scale, RoPECache* rope, float freq_base) {
    if (!pool_ || batch_ == 0) return Error(ErrorCode::InvalidState, "begin_step() has not been called");
    BlockManager& blocks = pool_->block_manager();
    const PagedKVConfig& cfg = blocks.config();
    if (layer < 0 || layer >= cfg.num_layers) return Error(ErrorCode::InvalidArgument, "Invalid layer index");
    if (q.ndim() != 3 || k.ndim() != 3 || v.ndim() != 3 || out.ndim() != 3 || q.size(0) != batch_ ||
        k.size(0) != batch_ || v.size(0) != batch_ || out.size(0) != batch_ ||
        k.size(1) != cfg.num_kv_heads || v.size(1) != cfg.num_kv_heads || out.size(1) != q.size(1) ||
        q.size(2) != cfg.head_dim || k.size(2) != cfg.head_dim || v.size(2) != cfg.head_dim ||
        out.size(2) != cfg.head_dim || q.size(1) % cfg.num_kv_heads != 0)
        return Error(ErrorCode::ShapeMismatch,
                     "run_layer takes q/out [B, num_heads, D] and k/v [B, num_kv_heads, D]");
    if (q.dtype() != DataType::FP32 || k.dtype() != DataType::FP32 || v.dtype() != DataType::FP32 ||
        out.dtype() != DataType::FP32)
        return Error(ErrorCode::DTypeMismatch, "run_layer takes FP32 tensors");

    auto ptr = [&](const Tensor& t) -> char* {
        auto* p = static_cast<char*>(hip_device_pointer(backend_, t.buffer()));
        return p ? p + t.buffer_offset() : nullptr;
    };
    granite_hip_rope_args r{};
    r.q = ptr(q);
    r.k = ptr(k);
    r.v = ptr(v);
    r.cache_k = ptr(blocks.k_cache(layer));
    r.cache_v = ptr(blocks.v_cache(layer));
    r.block_table = reinterpret_cast<const int32_t*>(ptr(tables_));
    r.positions = reinterpret_cast<const int32_t*>(ptr(positions_));
    r.table_stride = max_blocks_;
    r.max_blocks_per_seq = static_cast<uint32_t>(max_blocks_);
    r.block_size = static_cast<uint32_t>(blocks.block_size());
    r.num_heads_q = static_cast<uint32_t>(q.size(1));
    r.num_heads_k = static_cast<uint32_t>(cfg.num_kv_heads);
    r.seq_len = static_cast<uint32_t>(batch_);
    r.head_dim = static_cast<uint32_t>(cfg.head_dim);
    r.freq_base = freq_base;
    r.write_k_back = 1;
    r.rounding = rounding_;
    if (rope) {
        if (rope->head_dim() != cfg.head_dim)
            return Error(ErrorCode::ShapeMismatch, "RoPE tables are for another head size");
        GRANITE_TRY_ASSIGN(tables, rope->device_tables(backend_));
        r.cos_table = tables.first;
        r.sin_table = tables.second;
        r.table_positions = static_cast<uint32_t>(rope->max_seq_len());
    }
    char* out_ptr = ptr(out);
    if (!r.q || !r.k || !r.v || !r.cache_k || !r.cache_v || !r.block_table || !r.positions || !out_ptr)
        return Error(ErrorCode::InternalError, "Tensor buffers do not belong to the HIP backend");
    HipCompute compute;
    GRANITE_TRY(compute.rope_append(r));
    return compute.batched_paged_attention_decode(
        r.q, r.cache_k, r.cache_v, ptr(tables_), ptr(lens_), out_ptr, static_cast<uint32_t>(batch_),
        r.num_heads_q, r.num_heads_k, r.head_dim, r.block_size, static_cast<uint32_t>(max_blocks_), scale);
}

}  // namespace granite
