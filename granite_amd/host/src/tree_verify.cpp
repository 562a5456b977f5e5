// TreeVerify and select_attention_path: see granite/tree_verify.h.
#include "granite/tree_verify.h"

#include <string>

#include "granite/hip_backend.h"
#include "granite/hip_compute.h"
#include "granite_hip.h"

namespace granite {

Result<AttentionPath> select_attention_path(const AttentionRequest& r) {
    if (r.total_tokens <= 0 || r.start_pos < 0)
        return Error(ErrorCode::InvalidArgument, "attention needs at least one token at a position >= 0");
    const bool is_decode = r.total_tokens == 1;
    // paged attention first, for all layers unconditionally (transformer.mm:4847-4858)
    if (is_decode && r.paged_attention) return AttentionPath::PagedDecode;
    // a context beyond the offloaded GPU cache leaves the GPU (:4861-4872)
    if (r.has_gpu_cache && r.kv_cache_offload && r.start_pos + r.total_tokens > r.gpu_cache_max_seq_len)
        return Error(ErrorCode::BackendNotSupported,
                     "context of " + std::to_string(r.start_pos + r.total_tokens) + " tokens exceeds the GPU cache (" +
                         std::to_string(r.gpu_cache_max_seq_len) +
                         "): the reference continues on its CPU path, which this build does not have");
    if (is_decode && r.has_gpu_cache) {
        if (r.gpu_cache_len == r.start_pos) return AttentionPath::FullDecode;  // :4878-4888
        if (r.gpu_cache_len < r.start_pos && r.host_cache_len >= r.start_pos)   // :4890-4909
            return AttentionPath::SyncThenFullDecode;
        return Error(ErrorCode::InvalidState,
                     "GPU cache holds " + std::to_string(r.gpu_cache_len) + " tokens, the step starts at " +
                         std::to_string(r.start_pos) + " (the reference falls back to its CPU path here)");
    }
    if (!is_decode && r.has_gpu_cache && r.start_pos == 0) return AttentionPath::Prefill;  // :4915
    return Error(ErrorCode::InvalidState,
                 r.has_gpu_cache ? "a prefill that does not start at position 0 is served by the chunked prefill "
                                   "driver, not by attention_gpu (the reference falls back to its CPU path here)"
                                 : "no GPU cache allocated (the reference falls back to its CPU path here)");
}

Result<void> TreeVerify::initialize(PagedKVCache* sequence, int max_blocks_per_seq, int max_nodes,
                                    IComputeBackend* backend) {
    if (!sequence || !sequence->block_manager() || !sequence->block_manager()->is_initialized())
        return Error(ErrorCode::InvalidState, "Sequence has no block manager");
    if (max_blocks_per_seq <= 0 || max_nodes <= 0)
        return Error(ErrorCode::InvalidArgument, "Block-table and tree sizes must be positive");
    if (!backend || backend->get_type() != BackendType::HIP)
        return Error(ErrorCode::BackendNotSupported, "TreeVerify runs on the HIP backend only");
    const PagedKVConfig& cfg = sequence->block_manager()->config();
    sequence_ = sequence;
    backend_ = backend;
    max_blocks_ = max_blocks_per_seq;
    max_nodes_ = max_nodes;
    GRANITE_TRY_ASSIGN(table, Tensor::allocate({max_blocks_per_seq}, DataType::INT32, backend));
    GRANITE_TRY_ASSIGN(parents, Tensor::allocate({max_nodes}, DataType::INT32, backend));
    table_ = std::move(table);
    parents_ = std::move(parents);
    k_tree_.clear();
    v_tree_.clear();
    num_nodes_ = 0;
    layer_done_.assign(cfg.num_layers, false);
    open_ = false;
    return {};
}

Result<void> TreeVerify::begin(std::span<const int> parent_indices) {
    if (!sequence_) return Error(ErrorCode::InvalidState, "TreeVerify not initialized");
    const int n = static_cast<int>(parent_indices.size());
    if (n <= 0 || n > max_nodes_)
        return Error(ErrorCode::InvalidArgument,
                     "Tree of " + std::to_string(n) + " nodes, at most " + std::to_string(max_nodes_));
    for (int i = 0; i < n; ++i)
        if (parent_indices[i] >= n || parent_indices[i] < -1)
            return Error(ErrorCode::InvalidArgument, "Parent pointer outside the tree");
    if (sequence_->num_blocks() > max_blocks_)
        return Error(ErrorCode::InvalidArgument, "Sequence has more blocks than the device table holds");
    std::vector<int32_t> parents32(parent_indices.begin(), parent_indices.end());
    std::vector<int32_t> table32(sequence_->block_table().begin(), sequence_->block_table().end());
    GRANITE_TRY(backend_->write_buffer(parents_.buffer(), parents32.data(), parents32.size() * sizeof(int32_t)));
    if (!table32.empty())
        GRANITE_TRY(backend_->write_buffer(table_.buffer(), table32.data(), table32.size() * sizeof(int32_t)));
    // the tree's K/V rows per layer, [num_kv_heads, num_nodes, D] FP16 as the kernel indexes them
    // (the reference allocates them per call, transformer.mm:2264-2276; here only when the tree
    // size changes)
    if (n != num_nodes_ || k_tree_.empty()) {
        const PagedKVConfig& cfg = sequence_->block_manager()->config();
        k_tree_.clear();
        v_tree_.clear();
        for (int l = 0; l < cfg.num_layers; ++l) {
            GRANITE_TRY_ASSIGN(kt, Tensor::allocate({cfg.num_kv_heads, n, cfg.head_dim}, DataType::FP16, backend_));
            GRANITE_TRY_ASSIGN(vt, Tensor::allocate({cfg.num_kv_heads, n, cfg.head_dim}, DataType::FP16, backend_));
            k_tree_.push_back(std::move(kt));
            v_tree_.push_back(std::move(vt));
        }
    }
    num_nodes_ = n;
    original_ = sequence_->seq_len();
    layer_done_.assign(layer_done_.size(), false);
    open_ = true;
    return {};
}

Result<void> TreeVerify::run_layer(int layer, const Tensor& q, const Tensor& k, const Tensor& v, Tensor& out,
                                   float scale) {
    if (!open_) return Error(ErrorCode::InvalidState, "begin() has not been called");
    BlockManager& blocks = *sequence_->block_manager();
    const PagedKVConfig& cfg = blocks.config();
    if (layer < 0 || layer >= cfg.num_layers) return Error(ErrorCode::InvalidArgument, "Invalid layer index");
    const int64_t n = num_nodes_;
    if (q.ndim() != 3 || k.ndim() != 3 || v.ndim() != 3 || out.ndim() != 3 || q.size(0) != n || k.size(0) != n ||
        v.size(0) != n || out.size(0) != n || k.size(1) != cfg.num_kv_heads || v.size(1) != cfg.num_kv_heads ||
        out.size(1) != q.size(1) || q.size(2) != cfg.head_dim || k.size(2) != cfg.head_dim ||
        v.size(2) != cfg.head_dim || out.size(2) != cfg.head_dim || q.size(1) % cfg.num_kv_heads != 0)
        return Error(ErrorCode::ShapeMismatch,
                     "run_layer takes q/out [num_nodes, num_heads, D] and k/v [num_nodes, num_kv_heads, D]");
    if (q.dtype() != DataType::FP32 || k.dtype() != DataType::FP32 || v.dtype() != DataType::FP32 ||
        out.dtype() != DataType::FP32)
        return Error(ErrorCode::DTypeMismatch, "run_layer takes FP32 tensors");
    auto ptr = [&](const Tensor& t) -> char* {
        auto* p = static_cast<char*>(hip_device_pointer(backend_, t.buffer()));
        return p ? p + t.buffer_offset() : nullptr;
    };
    char *q_ptr = ptr(q), *k_ptr = ptr(k), *v_ptr = ptr(v), *out_ptr = ptr(out);
    char *kt = ptr(k_tree_[layer]), *vt = ptr(v_tree_[layer]);
    if (!q_ptr || !k_ptr || !v_ptr || !out_ptr || !kt || !vt)
        return Error(ErrorCode::InternalError, "Tensor buffers do not belong to the HIP backend");
    const uint32_t hkv = static_cast<uint32_t>(cfg.num_kv_heads), d = static_cast<uint32_t>(cfg.head_dim);
    const uint32_t hq = static_cast<uint32_t>(q.size(1));
    // [num_nodes, Hkv, D] float -> [Hkv, num_nodes, D] half, truncating (transformer.mm:2295-2304):
    // the append into a "cache" of exactly num_nodes rows per head, starting at row 0
    GRANITE_TRY(hip_status_to_result(
        granite_hip_kv_cache_append_ex(kt, vt, k_ptr, v_ptr, GRANITE_HIP_F32, int64_t(hkv) * d, d, hkv, d, 0,
                                       static_cast<uint32_t>(n), static_cast<uint32_t>(n),
                                       GRANITE_HIP_ROUND_TRUNCATE),
        "granite_hip_kv_cache_append_ex"));
    granite_hip_attention_args a{};
    a.q = q_ptr;
    a.q_dtype = GRANITE_HIP_F32;
    a.q_tok_stride = int64_t(hq) * d;
    a.q_head_stride = d;
    a.out = out_ptr;
    a.out_dtype = GRANITE_HIP_F32;
    a.out_tok_stride = int64_t(hq) * d;
    a.out_head_stride = d;
    a.seq_q = static_cast<uint32_t>(n);
    a.num_heads = hq;
    a.num_kv_heads = hkv;
    a.head_dim = d;
    a.scale = scale;
    a.k_cache = ptr(blocks.k_cache(layer));
    a.v_cache = ptr(blocks.v_cache(layer));
    a.cache_len = static_cast<uint32_t>(original_);
    a.block_table = reinterpret_cast<const int32_t*>(ptr(table_));
    a.block_size = static_cast<uint32_t>(blocks.block_size());
    a.k_extra = kt;
    a.v_extra = vt;
    a.extra_len = static_cast<uint32_t>(n);
    a.parents = reinterpret_cast<const int32_t*>(ptr(parents_));
    a.mask_mode = GRANITE_HIP_MASK_TREE;
    HipCompute compute;
    GRANITE_TRY(compute.attention(a));
    layer_done_[layer] = true;
    return {};
}

Result<void> TreeVerify::commit(std::span<const int> accepted_nodes) {
    if (!open_) return Error(ErrorCode::InvalidState, "begin() has not been called");
    for (bool done : layer_done_)
        if (!done) return Error(ErrorCode::InvalidState, "commit() before every layer has run");
    for (int node : accepted_nodes)
        if (node < 0 || node >= num_nodes_) return Error(ErrorCode::InvalidArgument, "Accepted node outside the tree");
    GRANITE_TRY(commit_tree_path(*sequence_, original_, accepted_nodes, k_tree_, v_tree_, backend_));
    open_ = false;
    return {};
}

}  // namespace granite
