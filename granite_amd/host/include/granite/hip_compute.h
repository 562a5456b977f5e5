// HipCompute: the MI355X counterpart of MetalCompute's attention-path methods
// (reference: include/granite/metal_compute.h:24-48, 784-920, 944).  Same method
// names, argument order and meaning; MTL::Buffer* becomes HipBuffer* (a device
// pointer).  Every method is a thin call into the C ABI of libgranite_hip.so;
// there is no host implementation behind it.
#pragma once

#include <cstddef>
#include <cstdint>
#include <utility>

#include "granite/error.h"

struct granite_hip_attention_args;
struct granite_hip_decode_args;
struct granite_hip_rope_args;

namespace granite {

using HipBuffer = void;  // device memory handed out by HipCompute::create_buffer

class HipCompute {
  public:
    // device_index -1 means device 0.  Fails with BackendNotSupported
    // when the GPU library cannot run (no gfx950 device).
    Result<void> initialize(int device_index = -1);
    void shutdown();
    bool is_initialized() const;
    void sync();
    void commit() {}  // launches are already asynchronous on the stream

    HipBuffer* create_buffer(size_t size, bool shared = true);
    void release_buffer(HipBuffer* buffer);
    Result<void> upload(HipBuffer* dst, const void* src, size_t bytes, size_t dst_offset = 0);
    Result<void> download(void* dst, const HipBuffer* src, size_t bytes, size_t src_offset = 0);

    // [num_kv_heads, max_seq_len, head_dim] half, zero filled.
    std::pair<HipBuffer*, HipBuffer*> create_kv_cache(uint32_t num_kv_heads, uint32_t max_seq_len,
                                                      uint32_t head_dim);

    // new_k/new_v: [new_len, num_kv_heads, head_dim] float (the layout the
    // reference kernel indexes); caches [num_kv_heads, max_seq_len, head_dim] half.
    Result<void> kv_cache_append(HipBuffer* cache_k, HipBuffer* cache_v, HipBuffer* new_k,
                                 HipBuffer* new_v, uint32_t num_kv_heads, uint32_t head_dim,
                                 uint32_t current_len, uint32_t new_len, uint32_t max_seq_len);
    // FP16 source [num_kv_heads, new_len, head_dim]: KVCache::append's layout.
    Result<void> kv_cache_append_f16(HipBuffer* cache_k, HipBuffer* cache_v, const HipBuffer* new_k,
                                     const HipBuffer* new_v, uint32_t num_kv_heads,
                                     uint32_t head_dim, uint32_t current_len, uint32_t new_len,
                                     uint32_t max_seq_len);

    Result<void> multihead_attention(HipBuffer* Q, HipBuffer* K, HipBuffer* V, HipBuffer* output,
                                     uint32_t num_heads, uint32_t num_kv_heads, uint32_t seq_q,
                                     uint32_t seq_kv, uint32_t head_dim, float scale,
                                     uint32_t max_seq = 0);
    Result<void> attention_tree(HipBuffer* Q, HipBuffer* K_cache, HipBuffer* V_cache,
                                HipBuffer* K_tree, HipBuffer* V_tree, HipBuffer* parent_indices,
                                HipBuffer* output, uint32_t num_heads, uint32_t num_kv_heads,
                                uint32_t num_nodes, uint32_t cache_len, uint32_t head_dim,
                                float scale);
    Result<void> paged_attention_decode(HipBuffer* Q, HipBuffer* K_cache, HipBuffer* V_cache,
                                        HipBuffer* block_table, HipBuffer* output,
                                        uint32_t num_heads, uint32_t num_kv_heads, uint32_t seq_len,
                                        uint32_t head_dim, uint32_t block_size, float scale);
    Result<void> paged_kv_cache_append(HipBuffer* new_k, HipBuffer* new_v, HipBuffer* K_cache,
                                       HipBuffer* V_cache, HipBuffer* block_table,
                                       uint32_t num_kv_heads, uint32_t head_dim, uint32_t start_pos,
                                       uint32_t new_len, uint32_t block_size);
    Result<void> batched_paged_attention_decode(HipBuffer* Q, HipBuffer* K_cache,
                                                HipBuffer* V_cache, HipBuffer* block_tables,
                                                HipBuffer* seq_lens, HipBuffer* output,
                                                uint32_t batch_size, uint32_t num_heads,
                                                uint32_t num_kv_heads, uint32_t head_dim,
                                                uint32_t block_size, uint32_t max_blocks_per_seq,
                                                float scale);
    Result<void> paged_kv_gather(HipBuffer* dst_k, HipBuffer* dst_v, const HipBuffer* K_cache,
                                 const HipBuffer* V_cache, const HipBuffer* block_table,
                                 uint32_t num_kv_heads, uint32_t head_dim, uint32_t len,
                                 uint32_t block_size, uint32_t max_seq_len);

    // MetalCompute::rope_multihead (include/granite/metal_compute.h:728-739): q [seq, Hq, D]
    // and k [seq, Hkv, D] float, rotated in place, cos/sin evaluated on the device.
    Result<void> rope_multihead(HipBuffer* q, HipBuffer* k, uint32_t num_heads_q,
                                uint32_t num_heads_k, uint32_t seq_len, uint32_t head_dim,
                                uint32_t start_pos, float freq_base = 10000.0f);
    // The rotation (from cos/sin tables or evaluated) fused with the K/V append.
    Result<void> rope_append(const granite_hip_rope_args& args);

    // MetalCompute::fused_qkv_matvec_q4k (include/granite/metal_compute.h:683-694): the three
    // attention projections of one token from Q4_K weights [N, K/256] in one launch; x [K],
    // yq [Nq], yk and yv [Nkv] float.
    Result<void> fused_qkv_matvec_q4k(HipBuffer* x, HipBuffer* Wq, HipBuffer* Wk, HipBuffer* Wv,
                                      HipBuffer* yq, HipBuffer* yk, HipBuffer* yv, uint32_t K,
                                      uint32_t Nq, uint32_t Nkv);
    // The same for the tokens of a batched decode step: x [batch, K], yq [batch, Nq], yk and
    // yv [batch, Nkv], the layouts PagedDecodeBatch::run_layer takes.
    Result<void> fused_qkv_matvec_q4k_batched(HipBuffer* x, HipBuffer* Wq, HipBuffer* Wk,
                                              HipBuffer* Wv, HipBuffer* yq, HipBuffer* yk,
                                              HipBuffer* yv, uint32_t K, uint32_t Nq, uint32_t Nkv,
                                              uint32_t batch);
    // MetalCompute::matvec_q4k (metal_compute.h:73-79): y [N] = W x, the output projection.
    Result<void> matvec_q4k(HipBuffer* x, HipBuffer* W, HipBuffer* y, uint32_t K, uint32_t N);

    // General entry points (strided Q/out, fp16 or fp32, paged or contiguous
    // keys, causal / tree masks, optional log-sum-exp).
    Result<void> attention(const granite_hip_attention_args& args);
    Result<void> decode_attention(const granite_hip_decode_args& args);

    // Scratch memory of the split-K launches.  MetalCompute's calls only enqueue
    // (src/backend/metal/metal_compute.mm:150-207); here a launch that needs more scratch
    // than the library holds waits for the device and reallocates, so a caller with a
    // serving loop asks once what its largest launches need and reserves it up front,
    // or passes a buffer of its own to the *_ws forms, which never allocate.
    size_t workspace_bytes() const;
    Result<void> reserve_workspace(size_t bytes);
    Result<size_t> attention_workspace_required(const granite_hip_attention_args& args);
    Result<size_t> decode_workspace_required(const granite_hip_decode_args& args);
    Result<void> attention_ws(const granite_hip_attention_args& args, HipBuffer* workspace,
                              size_t workspace_bytes);
    Result<void> decode_attention_ws(const granite_hip_decode_args& args, HipBuffer* workspace,
                                     size_t workspace_bytes);
};

// Process-wide instance, initialised on first use; nullptr when the GPU
// library cannot run (the caller must treat that as "backend unavailable").
HipCompute* get_hip_compute();

// Maps a C-ABI status to an ErrorCode (0 -> ok).
Result<void> hip_status_to_result(int status, const char* what);

}  // namespace granite
