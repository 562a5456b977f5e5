// The attention side of tree verification in speculative decoding, and the decision
// TransformerModel::attention_gpu takes about which GPU attention call applies.
//
// SpeculativeRunner::verify_tree (src/llm/speculative_runner.cpp:586-674) forwards all
// nodes of a SpeculationTree through the target model with tree attention
// (TransformerModel::attention_tree_gpu, src/llm/transformer.mm:2146-2402: reshape Q to
// [num_heads, num_nodes, D], cast the tree's K/V to FP16 as [num_kv_heads, num_nodes, D],
// upload the parent pointers, one attention_tree call per layer), picks the longest path
// the target agrees with and brings the target cache to "original + accepted" tokens
// (:871-882).  TreeVerify is that sequence around a paged sequence: per layer the cast and
// the tree attention over the paged prefix, then the commit of the accepted nodes' K/V rows
// (commit_tree_path) with the blocks past the new length freed.
#pragma once

#include <span>
#include <vector>

#include "granite/backend.h"
#include "granite/error.h"
#include "granite/kv_cache.h"
#include "granite/tensor.h"

namespace granite {

/// Which attention call serves one TransformerModel::attention_gpu invocation
/// (src/llm/transformer.mm:4837-5051).
enum class AttentionPath {
    PagedDecode,          ///< attention_paged_gpu: one token, paged attention active (:4850-4858)
    FullDecode,           ///< attention_full_gpu: one token, GPU cache holds exactly start_pos tokens (:4878-4888)
    SyncThenFullDecode,   ///< GPU cache behind the host cache: sync_cpu_to_gpu_kv_cache on layer 0, then FullDecode (:4890-4909)
    Prefill,              ///< several tokens at start_pos 0 with a GPU cache (:4915-5046)
};

/// What attention_gpu looks at.
struct AttentionRequest {
    int total_tokens = 1;             ///< batch * seq_len of the hidden states
    int start_pos = 0;
    int layer = 0;
    bool paged_attention = false;     ///< TransformerModel::is_paged_attention()
    bool has_gpu_cache = false;       ///< gpu_kv_cache_ allocated
    bool kv_cache_offload = false;    ///< RuntimeConfig::kv_cache_offload
    int gpu_cache_max_seq_len = 0;
    int gpu_cache_len = 0;            ///< gpu_kv_cache_->seq_len()
    int host_cache_len = -1;          ///< kv_cache->seq_len(), -1 without a host cache
};

/// The branch attention_gpu takes, in its order.  Where the reference leaves the GPU (a
/// context beyond the offloaded cache :4863-4872, a GPU cache ahead of the host cache :4911,
/// a prefill that does not start at position 0 or has no GPU cache :5050) it calls its CPU
/// attention(); this build has no CPU path, so those branches are errors that name the
/// branch (BackendNotSupported for the offload overflow, InvalidState for the others).
[[nodiscard]] Result<AttentionPath> select_attention_path(const AttentionRequest& request);

class TreeVerify {
public:
    /// sequence: the target's paged sequence (its BlockManager's pools are the caches of all
    /// layers); max_blocks_per_seq bounds its block table on the device; max_nodes the tree.
    [[nodiscard]] Result<void> initialize(PagedKVCache* sequence, int max_blocks_per_seq, int max_nodes,
                                          IComputeBackend* backend);

    /// Starts a verification: the prefix is what the sequence holds now (original length),
    /// the tree's parent pointers and the block table go to the device.  Nothing is appended
    /// to the sequence (attention_tree_gpu appends nothing either).
    [[nodiscard]] Result<void> begin(std::span<const int> parent_indices);

    /// One layer.  q [num_nodes, num_heads, D] and k, v [num_nodes, num_kv_heads, D], FP32 on
    /// the backend, rows in node order (already rotated: the reference rotates every node at
    /// start_pos + its index, transformer.mm:2250-2262).  k and v are cast to FP16 with the
    /// reference's truncating conversion (:2295-2304) into [num_kv_heads, num_nodes, D] and
    /// kept for the commit; out [num_nodes, num_heads, D] FP32 receives, for every node,
    /// attention over the whole prefix, its ancestors and itself.
    [[nodiscard]] Result<void> run_layer(int layer, const Tensor& q, const Tensor& k, const Tensor& v,
                                         Tensor& out, float scale);

    /// After the last layer: the accepted nodes' K/V rows (path order) become positions
    /// original .. of every layer's pool, the sequence is brought to original + accepted
    /// tokens and the surplus blocks are freed.  run_layer must have run for every layer.
    [[nodiscard]] Result<void> commit(std::span<const int> accepted_nodes);

    [[nodiscard]] int original_len() const { return original_; }
    [[nodiscard]] int num_nodes() const { return num_nodes_; }
    [[nodiscard]] const Tensor& k_tree(int layer) const { return k_tree_[layer]; }
    [[nodiscard]] const Tensor& v_tree(int layer) const { return v_tree_[layer]; }

private:
    IComputeBackend* backend_ = nullptr;
    PagedKVCache* sequence_ = nullptr;
    int max_blocks_ = 0, max_nodes_ = 0, num_nodes_ = 0, original_ = 0;
    Tensor table_, parents_;             // INT32 on the device
    std::vector<Tensor> k_tree_, v_tree_;  // per layer [num_kv_heads, num_nodes, D] FP16
    std::vector<bool> layer_done_;
    bool open_ = false;
};

}  // namespace granite
