// KVCache, KVCachePool, BlockManager, PagedKVCache, PagedKVPool: host
// bookkeeping as in the reference (src/llm/kv_cache.cpp, kv_cache_pool.cpp,
// paged_kv_cache.cpp), K/V bytes in HBM.
#include "granite/kv_cache.h"

#include <string>

#include "granite/hip_backend.h"
#include "granite/hip_compute.h"
#include "granite_hip.h"

namespace granite {

// ---- KVCache ---------------------------------------------------------------

Result<KVCache> KVCache::allocate(const ModelConfig& config, int max_seq_len,
                                  IComputeBackend* backend) {
    KVCache cache;
    cache.max_seq_len_ = max_seq_len;
    cache.num_kv_heads_ = config.num_kv_heads;
    cache.head_dim_ = config.head_dim;
    cache.backend_ = backend;
    const int64_t shape[4] = {1, config.num_kv_heads, max_seq_len, config.head_dim};
    for (int l = 0; l < config.num_layers; ++l) {
        Layer layer;
        GRANITE_TRY_ASSIGN(k, Tensor::allocate(shape, DataType::FP16, backend));
        layer.keys = std::move(k);
        GRANITE_TRY_ASSIGN(v, Tensor::allocate(shape, DataType::FP16, backend));
        layer.values = std::move(v);
        cache.layers_.push_back(std::move(layer));
    }
    return cache;
}

Result<void> KVCache::append(int layer, const Tensor& keys, const Tensor& values) {
    if (layer < 0 || layer >= static_cast<int>(layers_.size()))
        return Error(ErrorCode::InvalidArgument, "Invalid layer index");
    if (keys.ndim() != 4 || values.ndim() != 4 || keys.size(1) != num_kv_heads_ ||
        keys.size(3) != head_dim_ || values.size(1) != num_kv_heads_ ||
        values.size(2) != keys.size(2) || values.size(3) != head_dim_)
        return Error(ErrorCode::ShapeMismatch,
                     "append() takes [1, num_kv_heads, new_len, head_dim] keys and values");
    if (keys.dtype() != DataType::FP16 || values.dtype() != DataType::FP16)
        return Error(ErrorCode::DTypeMismatch, "KV cache rows are FP16");
    const int new_len = static_cast<int>(keys.size(2));
    if (current_len_ + new_len > max_seq_len_)
        return Error(ErrorCode::InvalidArgument,
                     "KV cache overflow: " + std::to_string(current_len_) + " + " +
                         std::to_string(new_len) + " > " + std::to_string(max_seq_len_));
    if (!backend_ || backend_->get_type() != BackendType::HIP)
        return Error(ErrorCode::BackendNotSupported, "KVCache::append runs on the HIP backend only");

    Layer& dst = layers_[layer];
    auto ptr = [&](const Tensor& t) -> char* {
        auto* p = static_cast<char*>(hip_device_pointer(backend_, t.buffer()));
        return p ? p + t.buffer_offset() : nullptr;
    };
    char* ck = ptr(dst.keys);
    char* cv = ptr(dst.values);
    const char* nk = ptr(keys);
    const char* nv = ptr(values);
    if (!ck || !cv || !nk || !nv)
        return Error(ErrorCode::InternalError, "Tensor buffers do not belong to the HIP backend");
    HipCompute compute;
    GRANITE_TRY(compute.kv_cache_append_f16(ck, cv, nk, nv, static_cast<uint32_t>(num_kv_heads_),
                                            static_cast<uint32_t>(head_dim_),
                                            static_cast<uint32_t>(current_len_),
                                            static_cast<uint32_t>(new_len),
                                            static_cast<uint32_t>(max_seq_len_)));
    if (layer == static_cast<int>(layers_.size()) - 1) current_len_ += new_len;
    return {};
}

std::pair<Tensor, Tensor> KVCache::get(int layer) const {
    if (layer < 0 || layer >= static_cast<int>(layers_.size())) return {Tensor{}, Tensor{}};
    return {layers_[layer].keys, layers_[layer].values};
}

size_t KVCache::memory_bytes() const {
    size_t total = 0;
    for (const Layer& l : layers_) total += l.keys.size_bytes() + l.values.size_bytes();
    return total;
}

// ---- KVCachePool -------------------------------------------------------------

Result<void> KVCachePool::allocate(int num_slots, const ModelConfig& config, int max_seq_len,
                                   IComputeBackend* backend) {
    caches_.clear();
    in_use_.assign(num_slots > 0 ? static_cast<size_t>(num_slots) : 0, false);
    for (int i = 0; i < num_slots; ++i) {
        auto made = KVCache::allocate(config, max_seq_len, backend);
        if (!made.ok())
            return Error(ErrorCode::AllocationFailed,
                         "Failed to allocate KV cache slot " + std::to_string(i));
        caches_.push_back(std::move(made).take());
    }
    return {};
}

int KVCachePool::acquire_slot() {
    for (size_t i = 0; i < in_use_.size(); ++i) {
        if (in_use_[i]) continue;
        in_use_[i] = true;
        caches_[i].clear();
        return static_cast<int>(i);
    }
    return -1;
}

void KVCachePool::release_slot(int slot) {
    if (slot >= 0 && slot < static_cast<int>(in_use_.size())) in_use_[slot] = false;
}

int KVCachePool::num_free_slots() const {
    int n = 0;
    for (bool used : in_use_) n += used ? 0 : 1;
    return n;
}

// ---- BlockManager ------------------------------------------------------------

Result<void> BlockManager::initialize(const PagedKVConfig& config, IComputeBackend* backend) {
    if (config.num_blocks <= 0 || config.block_size <= 0)
        return Error(ErrorCode::InvalidArgument, "Invalid block configuration");
    config_ = config;
    num_blocks_ = config.num_blocks;
    block_size_ = config.block_size;
    free_stack_.resize(num_blocks_);
    for (int i = 0; i < num_blocks_; ++i) free_stack_[i] = i;  // top of stack = highest index
    taken_.assign(num_blocks_, false);
    num_free_ = num_blocks_;

    const int64_t shape[3] = {int64_t(num_blocks_) * block_size_, config.num_kv_heads,
                              config.head_dim};
    k_pool_.clear();
    v_pool_.clear();
    for (int l = 0; l < config.num_layers; ++l) {
        auto k = Tensor::allocate(shape, DataType::FP16, backend);
        auto v = Tensor::allocate(shape, DataType::FP16, backend);
        if (!k.ok() || !v.ok())
            return Error(ErrorCode::AllocationFailed,
                         "Failed to allocate paged KV blocks for layer " + std::to_string(l));
        k_pool_.push_back(std::move(k).take());
        v_pool_.push_back(std::move(v).take());
    }
    return {};
}

int BlockManager::allocate_block() {
    if (num_free_ == 0) return -1;
    const int block = free_stack_[--num_free_];
    taken_[block] = true;
    return block;
}

void BlockManager::free_block(int block) {
    if (block < 0 || block >= num_blocks_ || !taken_[block]) return;
    taken_[block] = false;
    free_stack_[num_free_++] = block;
}

// ---- PagedKVCache ------------------------------------------------------------

void PagedKVCache::release() {
    if (!manager_) return;
    for (int block : table_) manager_->free_block(block);
    table_.clear();
    seq_len_ = 0;
}

bool PagedKVCache::append_tokens(int num_tokens) {
    if (!manager_) return false;
    const int bs = manager_->block_size();
    const int target_len = seq_len_ + num_tokens;
    const int blocks_needed = (target_len + bs - 1) / bs;
    while (static_cast<int>(table_.size()) < blocks_needed) {
        const int block = manager_->allocate_block();
        if (block < 0) return false;
        table_.push_back(block);
    }
    seq_len_ = target_len;
    return true;
}

int PagedKVCache::get_physical_block(int token_pos) const {
    if (!manager_) return -1;
    const int logical = token_pos / manager_->block_size();
    return logical < static_cast<int>(table_.size()) ? table_[logical] : -1;
}

int PagedKVCache::get_block_offset(int token_pos) const {
    return manager_ ? token_pos % manager_->block_size() : 0;
}

void PagedKVCache::truncate(int new_len) {
    if (new_len >= seq_len_ || !manager_) return;
    const int bs = manager_->block_size();
    const int keep = new_len == 0 ? 0 : (new_len + bs - 1) / bs;
    while (static_cast<int>(table_.size()) > keep) {
        manager_->free_block(table_.back());
        table_.pop_back();
    }
    seq_len_ = new_len;
}

// ---- PagedKVPool -------------------------------------------------------------

Result<void> PagedKVPool::initialize(const ModelConfig& config, int max_sequences,
                                     int max_total_tokens, int block_size,
                                     IComputeBackend* backend) {
    if (block_size <= 0) return Error(ErrorCode::InvalidArgument, "Invalid block configuration");
    PagedKVConfig paged;
    paged.block_size = block_size;
    paged.num_blocks = (max_total_tokens + block_size - 1) / block_size;
    paged.num_layers = config.num_layers;
    paged.num_kv_heads = config.num_kv_heads;
    paged.head_dim = config.head_dim;
    GRANITE_TRY(manager_.initialize(paged, backend));
    caches_.assign(max_sequences > 0 ? static_cast<size_t>(max_sequences) : 0,
                   PagedKVCache(&manager_));
    in_use_.assign(caches_.size(), false);
    return {};
}

int PagedKVPool::acquire_slot() {
    for (size_t i = 0; i < in_use_.size(); ++i) {
        if (in_use_[i]) continue;
        in_use_[i] = true;
        caches_[i].clear();
        return static_cast<int>(i);
    }
    return -1;
}

void PagedKVPool::release_slot(int slot) {
    if (slot < 0 || slot >= static_cast<int>(in_use_.size()) || !in_use_[slot]) return;
    caches_[slot].release();
    in_use_[slot] = false;
}

int PagedKVPool::num_free_slots() const {
    int n = 0;
    for (bool used : in_use_) n += used ? 0 : 1;
    return n;
}

Result<void> commit_tree_path(PagedKVCache& sequence, int original_len,
                              std::span<const int> accepted_nodes, std::span<const Tensor> k_tree,
                              std::span<const Tensor> v_tree, IComputeBackend* backend) {
    BlockManager* blocks = sequence.block_manager();
    if (!blocks || !blocks->is_initialized())
        return Error(ErrorCode::InvalidState, "Sequence has no block manager");
    const PagedKVConfig& cfg = blocks->config();
    if (original_len < 0 || static_cast<int>(k_tree.size()) != cfg.num_layers ||
        v_tree.size() != k_tree.size())
        return Error(ErrorCode::InvalidArgument, "One K and one V tree tensor per layer");
    if (!backend || backend->get_type() != BackendType::HIP)
        return Error(ErrorCode::BackendNotSupported, "commit_tree_path runs on the HIP backend only");
    int64_t num_nodes = 0;
    for (size_t l = 0; l < k_tree.size(); ++l) {
        const Tensor &k = k_tree[l], &v = v_tree[l];
        if (k.ndim() != 3 || v.ndim() != 3 || k.size(0) != cfg.num_kv_heads || k.size(2) != cfg.head_dim ||
            v.size(0) != k.size(0) || v.size(1) != k.size(1) || v.size(2) != k.size(2) ||
            (l > 0 && k.size(1) != num_nodes))
            return Error(ErrorCode::ShapeMismatch, "Tree K/V are [num_kv_heads, num_nodes, head_dim]");
        if (k.dtype() != DataType::FP16 || v.dtype() != DataType::FP16)
            return Error(ErrorCode::DTypeMismatch, "Tree K/V rows are FP16");
        num_nodes = k.size(1);
    }
    const int n = static_cast<int>(accepted_nodes.size());
    for (int node : accepted_nodes)
        if (node < 0 || node >= num_nodes) return Error(ErrorCode::InvalidArgument, "Accepted node outside the tree");
    const int target_len = original_len + n;
    if (sequence.seq_len() > target_len) {
        sequence.truncate(target_len);
    } else if (sequence.seq_len() < target_len && !sequence.append_tokens(target_len - sequence.seq_len())) {
        return Error(ErrorCode::AllocationFailed, "No free blocks for the accepted tokens");
    }
    if (n == 0) return {};

    std::vector<int32_t> nodes32(accepted_nodes.begin(), accepted_nodes.end());
    std::vector<int32_t> table(sequence.block_table().begin(), sequence.block_table().end());
    GRANITE_TRY_ASSIGN(d_nodes, backend->create_buffer_from_host(nodes32.data(), BufferDesc::device(nodes32.size() * 4)));
    auto made = backend->create_buffer_from_host(table.data(), BufferDesc::device(table.size() * 4));
    if (!made.ok()) {
        backend->destroy_buffer(d_nodes);
        return made.error();
    }
    const BufferHandle d_table = made.value();
    auto ptr = [&](const Tensor& t) -> char* {
        auto* p = static_cast<char*>(hip_device_pointer(backend, t.buffer()));
        return p ? p + t.buffer_offset() : nullptr;
    };
    Result<void> status;
    for (int l = 0; l < cfg.num_layers && status.ok(); ++l) {
        status = hip_status_to_result(
            granite_hip_kv_commit_accepted(
                ptr(k_tree[l]), ptr(v_tree[l]), GRANITE_HIP_F16, cfg.head_dim, num_nodes * cfg.head_dim,
                static_cast<uint32_t>(num_nodes),
                static_cast<const int32_t*>(hip_device_pointer(backend, d_nodes)), static_cast<uint32_t>(n),
                ptr(blocks->k_cache(l)), ptr(blocks->v_cache(l)),
                static_cast<const int32_t*>(hip_device_pointer(backend, d_table)),
                static_cast<uint32_t>(cfg.num_kv_heads), static_cast<uint32_t>(cfg.head_dim),
                static_cast<uint32_t>(original_len), static_cast<uint32_t>(blocks->block_size()), 0,
                GRANITE_HIP_ROUND_TRUNCATE),
            "granite_hip_kv_commit_accepted");
    }
    (void)backend->wait_for_completion();  // the two small buffers are released below
    backend->destroy_buffer(d_nodes);
    backend->destroy_buffer(d_table);
    return status;
}

}  // namespace granite
