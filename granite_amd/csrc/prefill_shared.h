// Declarations shared by the two prefill kernel files: the launch parameters that
// launch_attention() fills in, the softmax constants, and the launcher of the direct-to-LDS kernel.
#pragma once

#include "common.h"

namespace ghip {

constexpr float kNegBig = -1.0e30f;
constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;
constexpr uint32_t kMaxFusedNodes = 256;  // largest tree whose ancestor mask a workgroup builds itself
constexpr float kProbLimit = 16384.0f;  // a row's probabilities of a sub-tile may sum to this much

enum : int { kRowsContiguous = 0, kRowsPagedPow2 = 1, kRowsPagedAny = 2 };

struct AttnParams {
    const void* q;
    void* out;
    float* lse;
    int64_t q_tok_stride, q_head_stride, out_tok_stride, out_head_stride;
    const uint16_t* k;
    const uint16_t* v;
    const int32_t* table;
    uint32_t block_size;
    int bs_shift;
    int64_t a_tok_stride, a_head_stride;
    uint32_t cache_len;
    const uint16_t* k_extra;
    const uint16_t* v_extra;
    uint32_t extra_len;
    const uint32_t* tree_mask;      // ancestor bit matrix in memory (trees beyond kMaxFusedNodes)
    const int32_t* tree_parents;    // or: parent pointers, the workgroup builds its own matrix in LDS
    uint32_t mask_words;
    int mask_mode;
    uint32_t start_pos, seq_q, num_heads, group;
    float scale_log2;
    uint32_t q_tiles, n_splits;  // the grid: q_tiles * num_heads * n_splits workgroups
    // split-K over the key tiles (n_splits > 1): unnormalised partial results
    float* part_o;   // [split, head, q, D]
    float* part_ml;  // [split, head, q, 2] = (reference max, sum)
    void* final_out;
    int64_t final_tok_stride, final_head_stride;
};

// The direct-to-LDS form of the tiles kernel (prefill_dma.hip): same grid, same partial-result
// layout and same merge launch as attention_tiles_kernel.  Only for head size 128, no extra
// key segment, and a contiguous cache or a paged one whose block size is a power of two of at
// least 8 tokens; the caller checks that.
int launch_tiles_dma(const AttnParams& p, dim3 grid, bool q_f32, bool out_f32);
size_t tiles_dma_lds_bytes();

}  // namespace ghip
