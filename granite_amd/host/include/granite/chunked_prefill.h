// Chunked prefill of one sequence: the loop of TransformerModel::forward_prefill_raw
// (src/llm/transformer.mm:3467-3477 chunk size rule, :3681-3866 per-layer loop) around
// the attention path.  For every layer the prompt is walked in chunks; for each chunk
//   RoPE at start = chunk_start   ->  KV append at curr_len = chunk_start
//   ->  causal attention with seq_q = chunk, seq_kv = chunk_start + chunk, start_pos = chunk_start
// (the rotation and the append are one launch here).  The reference runs that loop over
// its contiguous GPU cache; the same loop is offered over a paged sequence (PagedKVCache),
// which is what a long prompt in a serving pool needs.  Positions continue from the tokens
// the sequence already holds, so a prompt may also extend an earlier prefix.
#pragma once

#include <vector>

#include "granite/backend.h"
#include "granite/error.h"
#include "granite/kv_cache.h"
#include "granite/rope.h"
#include "granite/tensor.h"

namespace granite {

/// Tokens per chunk for a prompt of num_tokens with RuntimeConfig::prefill_chunk_size
/// (src/llm/transformer.mm:3467-3477): 0, or a size not below the prompt, means one
/// pass; a request below 32 is raised to 32.
[[nodiscard]] int prefill_chunk_tokens(int num_tokens, uint32_t prefill_chunk_size);

class ChunkedPrefill {
public:
    /// Target: a paged sequence.  max_blocks_per_seq bounds its block table on the device.
    [[nodiscard]] Result<void> initialize(PagedKVCache* sequence, int max_blocks_per_seq,
                                          IComputeBackend* backend);
    /// Target: the contiguous cache [num_kv_heads, max_seq_len, head_dim] of a KVCache.
    [[nodiscard]] Result<void> initialize(KVCache* cache, IComputeBackend* backend);

    /// Plans a prompt of num_tokens behind the tokens the sequence holds.  Paged: takes the
    /// blocks for all of them now (all chunks of a layer run before the next layer starts)
    /// and uploads the block table; when the pool has too few free blocks nothing is
    /// taken and AllocationFailed returned.  Contiguous: InvalidArgument on overflow
    /// (src/llm/kv_cache.cpp:61-65).  A prompt that is still open (begin() without finish())
    /// is aborted first.
    [[nodiscard]] Result<void> begin(int num_tokens, uint32_t prefill_chunk_size);

    [[nodiscard]] int num_chunks() const { return static_cast<int>(starts_.size()); }
    [[nodiscard]] int chunk_start(int i) const { return starts_[i]; }  // inside the prompt
    [[nodiscard]] int chunk_len(int i) const { return lens_[i]; }
    [[nodiscard]] int base_len() const { return base_; }  // tokens held before the prompt

    /// One chunk of one layer.  q [chunk_len, num_heads, D], k and v [chunk_len, num_kv_heads,
    /// D], out [chunk_len, num_heads, D], FP32 on the backend: rows chunk_start .. of the
    /// prompt's projections.  q and k are rotated in place at positions base + chunk_start ..,
    /// the rotated k and v appended to the layer's cache rows of those positions, and out
    /// receives causal attention over everything up to each row.  Chunks of a layer must be
    /// run in order (chunk i reads what chunks 0 .. i-1 appended).
    [[nodiscard]] Result<void> run_chunk(int layer, int chunk, Tensor& q, Tensor& k, const Tensor& v,
                                         Tensor& out, float scale, RoPECache* rope,
                                         float freq_base = 10000.0f);

    /// All chunks of one layer: q/out [num_tokens, num_heads, D], k/v [num_tokens,
    /// num_kv_heads, D].  The reference's inner loop (transformer.mm:3681-3866).
    [[nodiscard]] Result<void> run_layer(int layer, Tensor& q, Tensor& k, const Tensor& v, Tensor& out,
                                         float scale, RoPECache* rope, float freq_base = 10000.0f);

    /// After the last layer: the contiguous cache's length advances by the prompt
    /// (increment on the last layer, transformer.mm:4822-4824); a paged sequence already has
    /// its length from begin().
    void finish();

    /// Gives up an open prompt: a paged sequence is truncated back to base_len() (its length
    /// was advanced by begin(), so after a failed run_chunk / run_layer it would otherwise
    /// cover rows that were never written) and the blocks past it are freed; a contiguous
    /// cache's length was never advanced.  A failed run_* call must be followed by abort()
    /// (or by a new begin(), which does it).  No effect when nothing is open.
    void abort();
    [[nodiscard]] bool is_open() const { return open_; }

    /// Float -> half conversion of the appended rows: GRANITE_HIP_ROUND_NEAREST (the GPU
    /// path's, default) or GRANITE_HIP_ROUND_TRUNCATE (the CPU path's).
    void set_rounding(int rounding) { rounding_ = rounding; }

private:
    [[nodiscard]] Result<void> plan(int num_tokens, uint32_t prefill_chunk_size);

    IComputeBackend* backend_ = nullptr;
    PagedKVCache* sequence_ = nullptr;
    KVCache* cache_ = nullptr;
    int max_blocks_ = 0;
    Tensor table_;  // [max_blocks] INT32 on the device (paged)
    int base_ = 0, num_tokens_ = 0;
    std::vector<int> starts_, lens_;
    int rounding_ = 1;
    bool open_ = false;
};

}  // namespace granite
