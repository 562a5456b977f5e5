// KV-cache state on either side of the attention kernels: the contiguous
// per-sequence cache, the block pool with per-sequence block tables, the slot
// pools for continuous batching and the speculation tree.  In the reference
// these classes are declared in include/granite/llm.h (KVCache :117-167,
// SpeculationTree :293-353, KVCachePool :846-881, PagedKVConfig :888-894,
// BlockManager :898-947, PagedKVCache :951-993, PagedKVPool :996-1037); names,
// argument meaning and error behaviour follow them.
//
// Bookkeeping (lengths, block tables, free lists) lives on the host exactly as
// in the reference; K/V bytes live in HBM.  KVCache::append therefore runs the
// device append kernel and requires a HIP backend.
#pragma once

#include <cstdint>
#include <utility>
#include <span>
#include <vector>

#include "granite/tensor.h"

namespace granite {

// The fields of ModelConfig (include/granite/llm.h:40-64) the KV state reads.
struct ModelConfig {
    int num_layers = 0;
    int num_heads = 0;
    int num_kv_heads = 0;
    int head_dim = 0;
    int max_seq_len = 0;
};

class KVCache {
  public:
    KVCache() = default;

    // One K and one V tensor [1, num_kv_heads, max_seq_len, head_dim] FP16 per layer.
    [[nodiscard]] static Result<KVCache> allocate(const ModelConfig& config, int max_seq_len,
                                                  IComputeBackend* backend);

    // keys/values: [1, num_kv_heads, new_len, head_dim] FP16.  Rows land at
    // seq_len() .. seq_len()+new_len-1; the length advances only when the last
    // layer is appended (src/llm/kv_cache.cpp:55-107).  A bad layer or an append
    // past max_seq_len is InvalidArgument.
    Result<void> append(int layer, const Tensor& keys, const Tensor& values);

    // Whole-capacity tensors of a layer; two empty tensors for a bad index.
    [[nodiscard]] std::pair<Tensor, Tensor> get(int layer) const;

    [[nodiscard]] int seq_len() const { return current_len_; }
    [[nodiscard]] int max_seq_len() const { return max_seq_len_; }
    void clear() { current_len_ = 0; }
    void increment_seq_len(int delta = 1) { current_len_ += delta; }
    void set_seq_len(int len) { current_len_ = len; }
    // Speculative rollback: only shrinks, never below zero; data stays in place.
    void truncate(int new_len) {
        if (new_len >= 0 && new_len < current_len_) current_len_ = new_len;
    }
    [[nodiscard]] size_t memory_bytes() const;
    [[nodiscard]] bool is_allocated() const { return !layers_.empty(); }
    [[nodiscard]] int num_kv_heads() const { return num_kv_heads_; }
    [[nodiscard]] int head_dim() const { return head_dim_; }

  private:
    struct Layer {
        Tensor keys, values;
    };
    std::vector<Layer> layers_;
    int max_seq_len_ = 0, current_len_ = 0, num_kv_heads_ = 0, head_dim_ = 0;
    IComputeBackend* backend_ = nullptr;
};

class KVCachePool {
  public:
    [[nodiscard]] Result<void> allocate(int num_slots, const ModelConfig& config, int max_seq_len,
                                        IComputeBackend* backend);
    // Lowest free slot, cleared; -1 when all are taken.
    int acquire_slot();
    void release_slot(int slot);
    KVCache& get_cache(int slot) { return caches_[slot]; }
    const KVCache& get_cache(int slot) const { return caches_[slot]; }
    bool is_slot_in_use(int slot) const { return in_use_[slot]; }
    int num_slots() const { return static_cast<int>(caches_.size()); }
    int num_free_slots() const;

  private:
    std::vector<KVCache> caches_;
    std::vector<bool> in_use_;
};

struct PagedKVConfig {
    int block_size = 16;
    int num_blocks = 256;
    int num_layers = 0;
    int num_kv_heads = 0;
    int head_dim = 0;
};

// Owns the K/V pools [num_blocks * block_size, num_kv_heads, head_dim] FP16 per
// layer and a LIFO free list: the block freed last is handed out first
// (src/llm/paged_kv_cache.cpp:73-99).
class BlockManager {
  public:
    [[nodiscard]] Result<void> initialize(const PagedKVConfig& config, IComputeBackend* backend);
    int allocate_block();             // -1 when the pool is exhausted
    void free_block(int block_idx);   // out-of-range and double frees are ignored
    [[nodiscard]] int num_free_blocks() const { return num_free_; }
    [[nodiscard]] int num_total_blocks() const { return num_blocks_; }
    [[nodiscard]] int block_size() const { return block_size_; }
    [[nodiscard]] Tensor& k_cache(int layer) { return k_pool_[layer]; }
    [[nodiscard]] const Tensor& k_cache(int layer) const { return k_pool_[layer]; }
    [[nodiscard]] Tensor& v_cache(int layer) { return v_pool_[layer]; }
    [[nodiscard]] const Tensor& v_cache(int layer) const { return v_pool_[layer]; }
    [[nodiscard]] bool is_initialized() const { return !k_pool_.empty(); }
    [[nodiscard]] const PagedKVConfig& config() const { return config_; }

  private:
    PagedKVConfig config_;
    int num_blocks_ = 0, block_size_ = 0, num_free_ = 0;
    std::vector<int> free_stack_;
    std::vector<bool> taken_;
    std::vector<Tensor> k_pool_, v_pool_;
};

// One sequence's logical-to-physical block table over a shared BlockManager.
class PagedKVCache {
  public:
    PagedKVCache() = default;
    explicit PagedKVCache(BlockManager* block_manager) : manager_(block_manager) {}

    void release();
    // Grows the table to cover seq_len()+num_tokens.  On exhaustion returns
    // false with the blocks taken so far kept and the length unchanged.
    [[nodiscard]] bool append_tokens(int num_tokens);
    [[nodiscard]] int seq_len() const { return seq_len_; }
    [[nodiscard]] int num_blocks() const { return static_cast<int>(table_.size()); }
    [[nodiscard]] const std::vector<int>& block_table() const { return table_; }
    [[nodiscard]] int get_physical_block(int token_pos) const;  // -1 past the table
    [[nodiscard]] int get_block_offset(int token_pos) const;
    void clear() { release(); }
    void truncate(int new_len);  // frees the blocks past ceil(new_len / block_size)
    [[nodiscard]] BlockManager* block_manager() { return manager_; }

  private:
    BlockManager* manager_ = nullptr;
    std::vector<int> table_;
    int seq_len_ = 0;
};

class PagedKVPool {
  public:
    [[nodiscard]] Result<void> initialize(const ModelConfig& config, int max_sequences,
                                          int max_total_tokens, int block_size,
                                          IComputeBackend* backend);
    [[nodiscard]] int acquire_slot();
    void release_slot(int slot);
    [[nodiscard]] PagedKVCache& get_cache(int slot) { return caches_[slot]; }
    [[nodiscard]] const PagedKVCache& get_cache(int slot) const { return caches_[slot]; }
    [[nodiscard]] BlockManager& block_manager() { return manager_; }
    [[nodiscard]] int num_free_slots() const;
    [[nodiscard]] int num_free_blocks() const { return manager_.num_free_blocks(); }
    [[nodiscard]] bool is_initialized() const { return manager_.is_initialized(); }

  private:
    BlockManager manager_;
    std::vector<PagedKVCache> caches_;
    std::vector<bool> in_use_;
};

// Candidate continuations of a draft model; get_parent_indices() is what the
// tree-attention mask is built from (src/llm/speculation_tree.cpp:13-143).
class SpeculationTree {
  public:
    struct Node {
        int32_t token;
        int parent_idx;  // -1 for the root
        int depth;
        float log_prob;
        std::vector<int> children;
    };

    void build(int width, int depth);  // no-op: the runner adds the nodes
    int add_node(int32_t token, int parent_idx, float log_prob = 0.0f);
    std::vector<int> get_leaves() const;
    std::vector<int> get_path(int node_idx) const;  // root .. node
    std::vector<int> get_parent_indices() const;
    std::vector<int32_t> flatten_tokens() const;    // breadth first from node 0
    size_t size() const { return nodes_.size(); }
    const Node& node(int idx) const { return nodes_[idx]; }
    Node& node(int idx) { return nodes_[idx]; }
    const Node* get_node(int idx) const {
        return idx >= 0 && idx < static_cast<int>(nodes_.size()) ? &nodes_[idx] : nullptr;
    }
    int max_depth() const;
    void clear() { nodes_.clear(); }
    // Longest root path whose tokens equal target_choices position by position;
    // at the first mismatch the target's own token closes the path.
    std::vector<int32_t> find_accepted_path(const std::vector<int32_t>& target_choices) const;
    // The node indices of that path's tree nodes, root first (the closing token of a
    // mismatch is the target's own and has no node).  Not in the reference: it is what the
    // commit below needs.
    std::vector<int> find_accepted_nodes(const std::vector<int32_t>& target_choices) const;

  private:
    std::vector<Node> nodes_;
};

// Commit of an accepted path into a sequence's paged cache: the sequence is brought to
// original_len + accepted_nodes.size() tokens (blocks past that are freed, as the runner's
// truncate does, src/llm/speculative_runner.cpp:871-882; missing ones are allocated) and, for
// every layer, rows original_len .. receive the K/V of the accepted tree nodes in path order
// out of k_tree[layer] / v_tree[layer] ([num_kv_heads, num_nodes, head_dim] FP16).  The
// reference's runner presumes those rows are already in the cache, yet nothing on its tree
// path writes them: the semantics here are this build's.
[[nodiscard]] Result<void> commit_tree_path(PagedKVCache& sequence, int original_len,
                                            std::span<const int> accepted_nodes,
                                            std::span<const Tensor> k_tree,
                                            std::span<const Tensor> v_tree, IComputeBackend* backend);

}  // namespace granite
