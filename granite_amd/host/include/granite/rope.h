// RoPECache with the reference's interface (include/granite/llm.h:173-197) whose apply()
// runs on the GPU: the cos/sin tables are built on the host exactly as
// src/llm/rope.cpp:5-22 builds them, kept on the device as well, and apply() rotates Q and K
// there with those very values (src/llm/rope.cpp:24-92 is the loop it stands for).
#pragma once

#include <utility>
#include <vector>

#include "granite/backend.h"
#include "granite/error.h"
#include "granite/tensor.h"

namespace granite {

class RoPECache {
public:
    RoPECache() = default;
    ~RoPECache();
    RoPECache(const RoPECache&) = delete;
    RoPECache& operator=(const RoPECache&) = delete;

    /// Builds the cos/sin tables [max_seq_len, head_dim/2].
    void initialize(int max_seq_len, int head_dim, float theta = 10000.0f);

    /// Rotates q and k ([batch, seq_len, num_heads, head_dim], FP32, batch 1 as in the
    /// reference's indexing) in place, positions start_pos .. start_pos + seq_len - 1.
    /// The tensors must live on a HIP backend (other backends: BackendNotSupported).
    Result<void> apply(Tensor& q, Tensor& k, int start_pos, IComputeBackend* backend);

    /// The same rotation and, in the same pass, the append of the rotated k and of v
    /// ([batch, seq_len, num_kv_heads, head_dim] FP32) to a contiguous FP16 cache
    /// [num_kv_heads, max_cache_len, head_dim] at rows start_pos .. (round to nearest).
    Result<void> apply_and_append(Tensor& q, Tensor& k, const Tensor& v, Tensor& cache_k,
                                  Tensor& cache_v, int start_pos, IComputeBackend* backend);

    /// Device copies of the tables on `backend` (made on first use): cos, sin.
    Result<std::pair<const float*, const float*>> device_tables(IComputeBackend* backend);
    [[nodiscard]] int max_seq_len() const { return max_seq_len_; }
    [[nodiscard]] int head_dim() const { return head_dim_; }

    [[nodiscard]] const std::vector<float>& cos_cache() const { return cos_; }
    [[nodiscard]] const std::vector<float>& sin_cache() const { return sin_; }
    [[nodiscard]] bool is_initialized() const { return !cos_.empty(); }

private:
    Result<void> run(Tensor& q, Tensor& k, const Tensor* v, Tensor* cache_k, Tensor* cache_v,
                     int start_pos, IComputeBackend* backend);
    Result<void> ensure_device_tables(IComputeBackend* backend);

    std::vector<float> cos_;  // [max_seq_len, head_dim/2]
    std::vector<float> sin_;
    int max_seq_len_ = 0;
    int head_dim_ = 0;
    // device copies of the tables, owned through the backend that made them
    IComputeBackend* table_backend_ = nullptr;
    BufferHandle cos_dev_{};
    BufferHandle sin_dev_{};
};

}  // namespace granite
