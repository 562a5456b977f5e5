// HipCompute: MetalCompute-shaped methods over the C ABI of libgranite_hip.so.
#include "granite/hip_compute.h"

#include <mutex>
#include <string>

#include "granite_hip.h"

namespace granite {

Result<void> hip_status_to_result(int status, const char* what) {
    if (status == GRANITE_HIP_OK) return {};
    ErrorCode code;
    switch (status) {
        case GRANITE_HIP_EINVAL: code = ErrorCode::InvalidArgument; break;
        case GRANITE_HIP_ENOTINIT: code = ErrorCode::BackendNotInitialized; break;
        case GRANITE_HIP_ENOMEM: code = ErrorCode::AllocationFailed; break;
        case GRANITE_HIP_EUNSUPPORTED: code = ErrorCode::NotImplemented; break;
        case GRANITE_HIP_ENULL: code = ErrorCode::NullPointer; break;
        case GRANITE_HIP_EOVERFLOW: code = ErrorCode::InvalidArgument; break;  // kv_cache.cpp:61-65
        case GRANITE_HIP_ESCRATCH: code = ErrorCode::InvalidArgument; break;
        default: code = ErrorCode::ExecutionFailed; break;                     // a hipError_t
    }
    return Error(code, std::string(what) + ": " + granite_hip_error_string(status));
}

#define HIP_CALL(expr) hip_status_to_result((expr), #expr)

Result<void> HipCompute::initialize(int device_index) {
    int status = granite_hip_init(device_index < 0 ? 0 : device_index);
    if (status == GRANITE_HIP_OK) return {};
    return Error(ErrorCode::BackendNotSupported,
                 std::string("granite_hip_init: ") + granite_hip_error_string(status));
}

void HipCompute::shutdown() { (void)granite_hip_shutdown(); }
bool HipCompute::is_initialized() const { return granite_hip_is_initialized() != 0; }
void HipCompute::sync() { (void)granite_hip_sync(); }

HipBuffer* HipCompute::create_buffer(size_t size, bool /*shared*/) {
    // MetalCompute's `shared` picks CPU-visible storage on unified memory; a
    // discrete GPU keeps compute buffers in HBM either way and moves bytes
    // with upload()/download().
    void* p = nullptr;
    if (granite_hip_malloc(&p, size, GRANITE_HIP_MEM_DEVICE) != GRANITE_HIP_OK) return nullptr;
    return p;
}
void HipCompute::release_buffer(HipBuffer* buffer) {
    (void)granite_hip_free(buffer, GRANITE_HIP_MEM_DEVICE);
}
Result<void> HipCompute::upload(HipBuffer* dst, const void* src, size_t bytes, size_t off) {
    return HIP_CALL(granite_hip_memcpy_h2d(static_cast<char*>(dst) + off, src, bytes));
}
Result<void> HipCompute::download(void* dst, const HipBuffer* src, size_t bytes, size_t off) {
    return HIP_CALL(granite_hip_memcpy_d2h(dst, static_cast<const char*>(src) + off, bytes));
}

std::pair<HipBuffer*, HipBuffer*> HipCompute::create_kv_cache(uint32_t num_kv_heads,
                                                              uint32_t max_seq_len,
                                                              uint32_t head_dim) {
    const size_t bytes = size_t(num_kv_heads) * max_seq_len * head_dim * sizeof(uint16_t);
    HipBuffer* k = create_buffer(bytes);
    HipBuffer* v = create_buffer(bytes);
    if (!k || !v || granite_hip_memset(k, 0, bytes) != GRANITE_HIP_OK ||
        granite_hip_memset(v, 0, bytes) != GRANITE_HIP_OK) {
        release_buffer(k);
        release_buffer(v);
        return {nullptr, nullptr};
    }
    return {k, v};
}

Result<void> HipCompute::kv_cache_append(HipBuffer* cache_k, HipBuffer* cache_v, HipBuffer* new_k,
                                         HipBuffer* new_v, uint32_t num_kv_heads, uint32_t head_dim,
                                         uint32_t current_len, uint32_t new_len,
                                         uint32_t max_seq_len) {
    return HIP_CALL(granite_hip_kv_cache_append(cache_k, cache_v, new_k, new_v, num_kv_heads,
                                                head_dim, current_len, new_len, max_seq_len));
}

Result<void> HipCompute::kv_cache_append_f16(HipBuffer* cache_k, HipBuffer* cache_v,
                                             const HipBuffer* new_k, const HipBuffer* new_v,
                                             uint32_t num_kv_heads, uint32_t head_dim,
                                             uint32_t current_len, uint32_t new_len,
                                             uint32_t max_seq_len) {
    return HIP_CALL(granite_hip_kv_cache_append_ex(
        cache_k, cache_v, new_k, new_v, GRANITE_HIP_F16, /*tok stride*/ head_dim,
        /*head stride*/ int64_t(new_len) * head_dim, num_kv_heads, head_dim, current_len, new_len,
        max_seq_len, GRANITE_HIP_ROUND_TRUNCATE));
}

Result<void> HipCompute::multihead_attention(HipBuffer* Q, HipBuffer* K, HipBuffer* V,
                                             HipBuffer* output, uint32_t num_heads,
                                             uint32_t num_kv_heads, uint32_t seq_q, uint32_t seq_kv,
                                             uint32_t head_dim, float scale, uint32_t max_seq) {
    return HIP_CALL(granite_hip_multihead_attention(Q, K, V, output, num_heads, num_kv_heads, seq_q,
                                                    seq_kv, head_dim, scale, max_seq));
}

Result<void> HipCompute::attention_tree(HipBuffer* Q, HipBuffer* K_cache, HipBuffer* V_cache,
                                        HipBuffer* K_tree, HipBuffer* V_tree,
                                        HipBuffer* parent_indices, HipBuffer* output,
                                        uint32_t num_heads, uint32_t num_kv_heads,
                                        uint32_t num_nodes, uint32_t cache_len, uint32_t head_dim,
                                        float scale) {
    return HIP_CALL(granite_hip_attention_tree(
        Q, K_cache, V_cache, K_tree, V_tree, static_cast<const int32_t*>(parent_indices), output,
        num_heads, num_kv_heads, num_nodes, cache_len, head_dim, scale));
}

Result<void> HipCompute::paged_attention_decode(HipBuffer* Q, HipBuffer* K_cache,
                                                HipBuffer* V_cache, HipBuffer* block_table,
                                                HipBuffer* output, uint32_t num_heads,
                                                uint32_t num_kv_heads, uint32_t seq_len,
                                                uint32_t head_dim, uint32_t block_size,
                                                float scale) {
    return HIP_CALL(granite_hip_paged_attention_decode(
        Q, K_cache, V_cache, static_cast<const int32_t*>(block_table), output, num_heads,
        num_kv_heads, seq_len, head_dim, block_size, scale));
}

Result<void> HipCompute::paged_kv_cache_append(HipBuffer* new_k, HipBuffer* new_v,
                                               HipBuffer* K_cache, HipBuffer* V_cache,
                                               HipBuffer* block_table, uint32_t num_kv_heads,
                                               uint32_t head_dim, uint32_t start_pos,
                                               uint32_t new_len, uint32_t block_size) {
    return HIP_CALL(granite_hip_paged_kv_cache_append(
        new_k, new_v, K_cache, V_cache, static_cast<const int32_t*>(block_table), num_kv_heads,
        head_dim, start_pos, new_len, block_size));
}

Result<void> HipCompute::batched_paged_attention_decode(
    HipBuffer* Q, HipBuffer* K_cache, HipBuffer* V_cache, HipBuffer* block_tables,
    HipBuffer* seq_lens, HipBuffer* output, uint32_t batch_size, uint32_t num_heads,
    uint32_t num_kv_heads, uint32_t head_dim, uint32_t block_size, uint32_t max_blocks_per_seq,
    float scale) {
    return HIP_CALL(granite_hip_batched_paged_attention_decode(
        Q, K_cache, V_cache, static_cast<const int32_t*>(block_tables),
        static_cast<const int32_t*>(seq_lens), output, batch_size, num_heads, num_kv_heads,
        head_dim, block_size, max_blocks_per_seq, scale));
}

Result<void> HipCompute::paged_kv_gather(HipBuffer* dst_k, HipBuffer* dst_v,
                                         const HipBuffer* K_cache, const HipBuffer* V_cache,
                                         const HipBuffer* block_table, uint32_t num_kv_heads,
                                         uint32_t head_dim, uint32_t len, uint32_t block_size,
                                         uint32_t max_seq_len) {
    return HIP_CALL(granite_hip_paged_kv_gather(dst_k, dst_v, K_cache, V_cache,
                                                static_cast<const int32_t*>(block_table),
                                                num_kv_heads, head_dim, len, block_size,
                                                max_seq_len));
}

Result<void> HipCompute::rope_multihead(HipBuffer* q, HipBuffer* k, uint32_t num_heads_q,
                                        uint32_t num_heads_k, uint32_t seq_len, uint32_t head_dim,
                                        uint32_t start_pos, float freq_base) {
    return HIP_CALL(granite_hip_rope_multihead(q, k, num_heads_q, num_heads_k, seq_len, head_dim,
                                               start_pos, freq_base));
}

Result<void> HipCompute::rope_append(const granite_hip_rope_args& args) {
    return HIP_CALL(granite_hip_rope_append(&args));
}

Result<void> HipCompute::attention(const granite_hip_attention_args& args) {
    return HIP_CALL(granite_hip_attention(&args));
}
Result<void> HipCompute::decode_attention(const granite_hip_decode_args& args) {
    return HIP_CALL(granite_hip_decode_attention(&args));
}

Result<void> HipCompute::fused_qkv_matvec_q4k(HipBuffer* x, HipBuffer* Wq, HipBuffer* Wk,
                                              HipBuffer* Wv, HipBuffer* yq, HipBuffer* yk,
                                              HipBuffer* yv, uint32_t K, uint32_t Nq, uint32_t Nkv) {
    return HIP_CALL(granite_hip_fused_qkv_matvec_q4k(x, Wq, Wk, Wv, yq, yk, yv, K, Nq, Nkv));
}
Result<void> HipCompute::fused_qkv_matvec_q4k_batched(HipBuffer* x, HipBuffer* Wq, HipBuffer* Wk,
                                                      HipBuffer* Wv, HipBuffer* yq, HipBuffer* yk,
                                                      HipBuffer* yv, uint32_t K, uint32_t Nq,
                                                      uint32_t Nkv, uint32_t batch) {
    return HIP_CALL(granite_hip_fused_qkv_matvec_q4k_batched(x, K, Wq, Wk, Wv, yq, yk, yv, Nq, Nkv, K,
                                                             Nq, Nkv, batch));
}
Result<void> HipCompute::matvec_q4k(HipBuffer* x, HipBuffer* W, HipBuffer* y, uint32_t K, uint32_t N) {
    return HIP_CALL(granite_hip_matvec_q4k(x, W, y, K, N));
}

size_t HipCompute::workspace_bytes() const { return granite_hip_workspace_bytes(); }
Result<void> HipCompute::reserve_workspace(size_t bytes) {
    return HIP_CALL(granite_hip_reserve_workspace(bytes));
}
Result<size_t> HipCompute::attention_workspace_required(const granite_hip_attention_args& args) {
    size_t bytes = 0;
    GRANITE_TRY(HIP_CALL(granite_hip_attention_workspace_required(&args, &bytes)));
    return bytes;
}
Result<size_t> HipCompute::decode_workspace_required(const granite_hip_decode_args& args) {
    size_t bytes = 0;
    GRANITE_TRY(HIP_CALL(granite_hip_decode_workspace_required(&args, &bytes)));
    return bytes;
}
Result<void> HipCompute::attention_ws(const granite_hip_attention_args& args, HipBuffer* workspace,
                                      size_t workspace_bytes) {
    return HIP_CALL(granite_hip_attention_ws(&args, workspace, workspace_bytes));
}
Result<void> HipCompute::decode_attention_ws(const granite_hip_decode_args& args,
                                             HipBuffer* workspace, size_t workspace_bytes) {
    return HIP_CALL(granite_hip_decode_attention_ws(&args, workspace, workspace_bytes));
}

HipCompute* get_hip_compute() {
    static HipCompute instance;
    static std::mutex guard;
    std::lock_guard<std::mutex> lock(guard);
    if (!instance.is_initialized() && !instance.initialize().ok()) return nullptr;
    return &instance;
}

}  // namespace granite
