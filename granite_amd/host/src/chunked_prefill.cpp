// ChunkedPrefill: the per-layer chunk loop of forward_prefill_raw
// (src/llm/transformer.mm:3467-3477, 3681-3866) over the HIP attention path.
#include "granite/chunked_prefill.h"

#include <algorithm>
#include <string>

#include "granite/hip_backend.h"
#include "granite/hip_compute.h"
#include "granite_hip.h"

namespace granite {

int prefill_chunk_tokens(int num_tokens, uint32_t prefill_chunk_size) {
    int chunk_tokens = num_tokens;
    if (prefill_chunk_size > 0 && prefill_chunk_size < static_cast<uint32_t>(num_tokens)) {
        int requested = static_cast<int>(prefill_chunk_size);
        if (requested < 32) requested = 32;
        chunk_tokens = std::min(num_tokens, requested);
    }
    return chunk_tokens;
}

Result<void> ChunkedPrefill::initialize(PagedKVCache* sequence, int max_blocks_per_seq,
                                        IComputeBackend* backend) {
    if (!sequence || !sequence->block_manager() || !sequence->block_manager()->is_initialized())
        return Error(ErrorCode::InvalidState, "Paged sequence has no initialized block pool");
    if (max_blocks_per_seq <= 0)
        return Error(ErrorCode::InvalidArgument, "Block-table size must be positive");
    if (!backend || backend->get_type() != BackendType::HIP)
        return Error(ErrorCode::BackendNotSupported, "ChunkedPrefill runs on the HIP backend only");
    GRANITE_TRY_ASSIGN(table, Tensor::allocate({max_blocks_per_seq}, DataType::INT32, backend));
    table_ = std::move(table);
    backend_ = backend;
    sequence_ = sequence;
    cache_ = nullptr;
    max_blocks_ = max_blocks_per_seq;
    open_ = false;
    return {};
}

Result<void> ChunkedPrefill::initialize(KVCache* cache, IComputeBackend* backend) {
    if (!cache || !cache->is_allocated()) return Error(ErrorCode::InvalidState, "KV cache not allocated");
    if (!backend || backend->get_type() != BackendType::HIP)
        return Error(ErrorCode::BackendNotSupported, "ChunkedPrefill runs on the HIP backend only");
    backend_ = backend;
    cache_ = cache;
    sequence_ = nullptr;
    open_ = false;
    return {};
}

Result<void> ChunkedPrefill::plan(int num_tokens, uint32_t prefill_chunk_size) {
    const int chunk_tokens = prefill_chunk_tokens(num_tokens, prefill_chunk_size);
    starts_.clear();
    lens_.clear();
    for (int chunk_start = 0; chunk_start < num_tokens; chunk_start += chunk_tokens) {
        starts_.push_back(chunk_start);
        lens_.push_back(std::min(chunk_tokens, num_tokens - chunk_start));
    }
    num_tokens_ = num_tokens;
    return {};
}

Result<void> ChunkedPrefill::begin(int num_tokens, uint32_t prefill_chunk_size) {
    if (!backend_) return Error(ErrorCode::InvalidState, "ChunkedPrefill not initialized");
    if (num_tokens <= 0) return Error(ErrorCode::InvalidArgument, "A prompt has at least one token");
    abort();  // a prompt left open (a run_* call failed and the caller starts over) gives its tokens back
    if (sequence_) {
        const int block_size = sequence_->block_manager()->block_size();
        base_ = sequence_->seq_len();
        if ((int64_t(base_) + num_tokens + block_size - 1) / block_size > max_blocks_)
            return Error(ErrorCode::InvalidArgument,
                         "Prompt of " + std::to_string(num_tokens) + " tokens behind " +
                             std::to_string(base_) + " exceeds the block table");
        // PagedKVCache::append_tokens keeps what it took when the pool runs dry half way
        // (src/llm/paged_kv_cache.cpp:131-139) and truncate() cannot give it back at an
        // unchanged length, so the room is checked first.
        const int missing = static_cast<int>((int64_t(base_) + num_tokens + block_size - 1) / block_size) -
                            sequence_->num_blocks();
        if (missing > sequence_->block_manager()->num_free_blocks() || !sequence_->append_tokens(num_tokens))
            return Error(ErrorCode::AllocationFailed, "Block pool exhausted");
        std::vector<int32_t> table(sequence_->block_table().begin(), sequence_->block_table().end());
        GRANITE_TRY(backend_->write_buffer(table_.buffer(), table.data(), table.size() * sizeof(int32_t)));
    } else {
        base_ = cache_->seq_len();
        if (base_ + num_tokens > cache_->max_seq_len())
            return Error(ErrorCode::InvalidArgument,
                         "KV cache overflow: " + std::to_string(base_) + " + " +
                             std::to_string(num_tokens) + " > " + std::to_string(cache_->max_seq_len()));
    }
    GRANITE_TRY(plan(num_tokens, prefill_chunk_size));
    open_ = true;
    return {};
}

void ChunkedPrefill::abort() {
    if (open_ && sequence_) sequence_->truncate(base_);  // frees the blocks past the old length
    open_ = false;
}

Result<void> ChunkedPrefill::run_chunk(int layer, int chunk, Tensor& q, Tensor& k, const Tensor& v,
                                       Tensor& out, float scale, RoPECache* rope, float freq_base) {
    if (!open_) return Error(ErrorCode::InvalidState, "begin() has not been called");
    if (chunk < 0 || chunk >= num_chunks()) return Error(ErrorCode::InvalidArgument, "Invalid chunk index");
    const int len = lens_[chunk];
    const int start = base_ + starts_[chunk];  // position of the chunk's first token

    int num_kv_heads, head_dim;
    Tensor cache_k, cache_v;
    if (sequence_) {
        BlockManager& blocks = *sequence_->block_manager();
        const PagedKVConfig& cfg = blocks.config();
        if (layer < 0 || layer >= cfg.num_layers) return Error(ErrorCode::InvalidArgument, "Invalid layer index");
        num_kv_heads = cfg.num_kv_heads;
        head_dim = cfg.head_dim;
        cache_k = blocks.k_cache(layer);
        cache_v = blocks.v_cache(layer);
    } else {
        auto kv = cache_->get(layer);
        if (kv.first.numel() == 0) return Error(ErrorCode::InvalidArgument, "Invalid layer index");
        num_kv_heads = cache_->num_kv_heads();
        head_dim = cache_->head_dim();
        cache_k = kv.first;
        cache_v = kv.second;
    }
    if (q.ndim() != 3 || k.ndim() != 3 || v.ndim() != 3 || out.ndim() != 3 || q.size(0) != len ||
        k.size(0) != len || v.size(0) != len || out.size(0) != len || k.size(1) != num_kv_heads ||
        v.size(1) != num_kv_heads || out.size(1) != q.size(1) || q.size(2) != head_dim ||
        k.size(2) != head_dim || v.size(2) != head_dim || out.size(2) != head_dim ||
        q.size(1) % num_kv_heads != 0)
        return Error(ErrorCode::ShapeMismatch,
                     "run_chunk takes q/out [chunk, num_heads, D] and k/v [chunk, num_kv_heads, D]");
    if (q.dtype() != DataType::FP32 || k.dtype() != DataType::FP32 || v.dtype() != DataType::FP32 ||
        out.dtype() != DataType::FP32)
        return Error(ErrorCode::DTypeMismatch, "run_chunk takes FP32 tensors");
    if (!q.is_contiguous() || !k.is_contiguous() || !v.is_contiguous() || !out.is_contiguous())
        return Error(ErrorCode::InvalidArgument, "run_chunk takes contiguous tensors");

    auto ptr = [&](const Tensor& t) -> char* {
        auto* p = static_cast<char*>(hip_device_pointer(backend_, t.buffer()));
        return p ? p + t.buffer_offset() : nullptr;
    };
    // 1. rotation at start = chunk_start and append at curr_len = chunk_start, one launch
    granite_hip_rope_args r{};
    r.q = ptr(q);
    r.k = ptr(k);
    r.v = ptr(v);
    r.cache_k = ptr(cache_k);
    r.cache_v = ptr(cache_v);
    r.num_heads_q = static_cast<uint32_t>(q.size(1));
    r.num_heads_k = static_cast<uint32_t>(num_kv_heads);
    r.seq_len = static_cast<uint32_t>(len);
    r.head_dim = static_cast<uint32_t>(head_dim);
    r.start_pos = static_cast<uint32_t>(start);
    r.freq_base = freq_base;
    r.write_k_back = 1;
    r.rounding = rounding_;
    if (sequence_) {
        r.block_table = reinterpret_cast<const int32_t*>(ptr(table_));
        r.block_size = static_cast<uint32_t>(sequence_->block_manager()->block_size());
        r.max_blocks_per_seq = static_cast<uint32_t>(sequence_->num_blocks());
    } else {
        r.max_seq_len = static_cast<uint32_t>(cache_->max_seq_len());
    }
    if (rope) {
        if (rope->head_dim() != head_dim)
            return Error(ErrorCode::ShapeMismatch, "RoPE tables are for another head size");
        GRANITE_TRY_ASSIGN(tables, rope->device_tables(backend_));
        r.cos_table = tables.first;
        r.sin_table = tables.second;
        r.table_positions = static_cast<uint32_t>(rope->max_seq_len());
    }
    char* out_ptr = ptr(out);
    if (!r.q || !r.k || !r.v || !r.cache_k || !r.cache_v || !out_ptr || (sequence_ && !r.block_table))
        return Error(ErrorCode::InternalError, "Tensor buffers do not belong to the HIP backend");
    HipCompute compute;
    GRANITE_TRY(compute.rope_append(r));

    // 2. causal attention of the chunk over everything appended so far: seq_q = chunk,
    // seq_kv = chunk_start + chunk, start_pos = chunk_start (transformer.mm:3851-3866)
    granite_hip_attention_args a{};
    a.q = r.q;
    a.q_dtype = GRANITE_HIP_F32;
    a.q_tok_stride = q.size(1) * head_dim;
    a.q_head_stride = head_dim;
    a.out = out_ptr;
    a.out_dtype = GRANITE_HIP_F32;
    a.out_tok_stride = a.q_tok_stride;
    a.out_head_stride = head_dim;
    a.k_cache = r.cache_k;
    a.v_cache = r.cache_v;
    a.block_table = r.block_table;
    a.block_size = r.block_size;
    a.max_seq = r.max_seq_len;
    a.cache_len = static_cast<uint32_t>(start + len);
    a.mask_mode = GRANITE_HIP_MASK_CAUSAL;
    a.start_pos = static_cast<uint32_t>(start);
    a.seq_q = static_cast<uint32_t>(len);
    a.num_heads = r.num_heads_q;
    a.num_kv_heads = r.num_heads_k;
    a.head_dim = r.head_dim;
    a.scale = scale;
    return compute.attention(a);
}

Result<void> ChunkedPrefill::run_layer(int layer, Tensor& q, Tensor& k, const Tensor& v, Tensor& out,
                                       float scale, RoPECache* rope, float freq_base) {
    if (!open_) return Error(ErrorCode::InvalidState, "begin() has not been called");
    if (q.ndim() != 3 || k.ndim() != 3 || v.ndim() != 3 || out.ndim() != 3 || q.size(0) != num_tokens_ ||
        k.size(0) != num_tokens_ || v.size(0) != num_tokens_ || out.size(0) != num_tokens_)
        return Error(ErrorCode::ShapeMismatch, "run_layer takes tensors of num_tokens rows");
    if (!q.is_contiguous() || !k.is_contiguous() || !v.is_contiguous() || !out.is_contiguous())
        return Error(ErrorCode::InvalidArgument, "run_layer takes contiguous tensors");
    for (int c = 0; c < num_chunks(); ++c) {
        GRANITE_TRY_ASSIGN(qc, q.slice(0, starts_[c], starts_[c] + lens_[c]));
        GRANITE_TRY_ASSIGN(kc, k.slice(0, starts_[c], starts_[c] + lens_[c]));
        GRANITE_TRY_ASSIGN(vc, v.slice(0, starts_[c], starts_[c] + lens_[c]));
        GRANITE_TRY_ASSIGN(oc, out.slice(0, starts_[c], starts_[c] + lens_[c]));
        GRANITE_TRY(run_chunk(layer, c, qc, kc, vc, oc, scale, rope, freq_base));
    }
    return {};
}

void ChunkedPrefill::finish() {
    if (!open_) return;
    if (cache_) cache_->increment_seq_len(num_tokens_);
    open_ = false;
}

}  // namespace granite
