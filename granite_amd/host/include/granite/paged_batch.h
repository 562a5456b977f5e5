// One decode step for a batch of sequences that live in a PagedKVPool.
//
// The reference's BatchScheduler::process_batch_paged (src/llm/batch_scheduler.cpp:391-452)
// takes a token for every request from its PagedKVCache and then falls back to sequential
// processing ("full batched attention kernel integration is a future enhancement").  This
// class is that integration: it takes the tokens the same way, puts the block tables, lengths
// and positions of the batch on the device, and runs, per layer, one rotate-and-append launch
// and one batched paged decode (MetalCompute::batched_paged_attention_decode,
// include/granite/metal_compute.h:906-920) for all sequences together.
#pragma once

#include <span>
#include <vector>

#include "granite/backend.h"
#include "granite/error.h"
#include "granite/kv_cache.h"
#include "granite/rope.h"
#include "granite/tensor.h"

namespace granite {

class PagedDecodeBatch {
public:
    /// max_blocks_per_seq bounds the context of a sequence (times the pool's block size).
    [[nodiscard]] Result<void> initialize(PagedKVPool* pool, int max_batch, int max_blocks_per_seq,
                                          IComputeBackend* backend);

    /// Takes one more token for every slot (PagedKVCache::append_tokens(1), as the reference's
    /// loop does) and uploads the batch's block tables, lengths and positions.  Row b of the
    /// batch is slots[b].  A slot whose token cannot be allocated, or whose context would
    /// exceed max_blocks_per_seq, is reported in the returned list and takes no part in the
    /// step (its row is computed as an empty sequence: nothing is appended, its output row is
    /// left untouched); the others go on, as in the reference.
    [[nodiscard]] Result<std::vector<int>> begin_step(std::span<const int> slots);

    /// One layer of the step.  q [B, num_heads, D], k and v [B, num_kv_heads, D], out
    /// [B, num_heads, D], all FP32 on the backend; B is the batch of begin_step.  q and k are
    /// rotated in place at each sequence's last position (rope's tables; pass nullptr to
    /// evaluate from freq_base), the rotated k and v are appended to the layer's pool, and out
    /// receives the attention of every sequence over its whole context.
    [[nodiscard]] Result<void> run_layer(int layer, Tensor& q, Tensor& k, const Tensor& v, Tensor& out,
                                         float scale, RoPECache* rope, float freq_base = 10000.0f);

    /// Float -> half conversion of the appended rows: GRANITE_HIP_ROUND_NEAREST (the GPU
    /// path's, default) or GRANITE_HIP_ROUND_TRUNCATE (the CPU path's).
    void set_rounding(int rounding) { rounding_ = rounding; }

    [[nodiscard]] int batch_size() const { return batch_; }
    [[nodiscard]] const std::vector<int>& seq_lens() const { return host_lens_; }

private:
    PagedKVPool* pool_ = nullptr;
    IComputeBackend* backend_ = nullptr;
    int max_batch_ = 0, max_blocks_ = 0, batch_ = 0;
    int rounding_ = 1;
    Tensor tables_, lens_, positions_;  // [max_batch, max_blocks], [max_batch], [max_batch] INT32
    std::vector<int32_t> host_tables_;
    std::vector<int> host_lens_;
    std::vector<int32_t> host_positions_;
};

}  // namespace granite
