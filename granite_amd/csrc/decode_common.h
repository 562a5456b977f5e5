// Pieces shared by the two decode attention kernels (decode.hip: one workgroup
// per fixed chunk; decode_stream.hip: persistent waves over a flat tile list).
#pragma once

#include "common.h"

namespace ghip {

constexpr int kTile = 32;         // tokens per wave step
constexpr int kWavesPerWG = 4;
constexpr float kNegBig = -1.0e30f;
constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;

struct DecodeParams {
    uint32_t* plan;  // stream kernel, for its merge: [per, total, pad, pad, prefix[batch + 1]]
    const void* q;
    const uint16_t* k;
    const uint16_t* v;
    const int32_t* tables;
    const int32_t* seq_lens;
    float* part_o;   // chunk kernel: [B, Hq, max_chunks, D]; stream kernel: [piece, part_cap, D]
    float* part_ml;  // same, [.., 2] = (max, sum)
    float* out;
    float* lse;
    uint32_t batch, num_heads, num_kv_heads, group, q_groups;
    uint32_t head_dim;  // 128 or 64; the kernels are instantiated per head size
    uint32_t block_size, max_blocks;
    int bs_shift;  // log2(block_size) or -1
    int64_t tok_stride, head_stride;
    uint32_t max_tokens;  // bound on any sequence length
    uint32_t chunk_tokens, max_chunks;
    uint32_t workers, min_per;  // stream kernel: workers in the grid, smallest share of one
    uint32_t part_cap;          // stream kernel: query heads a piece slot holds
    float scale_log2;
};

// Token handled by slot j (0..7) of lane group g in the PV contraction.
__device__ __forceinline__ uint32_t tau(uint32_t g, uint32_t j) {
    return j < 4 ? 4 * g + j : 16 + 4 * g + (j - 4);
}

__device__ __forceinline__ half8 as_half8(uint4v x) { return __builtin_bit_cast(half8, x); }

// How token positions map to rows of the K/V arrays.
enum : int { kRowsContiguous = 0, kRowsPagedPow2 = 1, kRowsPagedAny = 2 };

// Physical row of token tok0 + (lane & 31), clamped to the sequence: one table
// read per lane per tile.  Every other lane fetches the rows it needs from
// these 32 values with a cross-lane read, so the K/V loads of a tile depend on
// a single earlier global load instead of one table lookup each.  Branch-free
// on purpose: a load inside a conditional forces a full wait at the join.
template <int kRows>
__device__ __forceinline__ uint32_t tile_row(const DecodeParams& p, const int32_t* table,
                                             uint32_t tok0, uint32_t lane, uint32_t len) {
    const uint32_t tok = min(tok0 + (lane & 31), len - 1);
    if constexpr (kRows == kRowsContiguous) {
        return tok;
    } else if constexpr (kRows == kRowsPagedPow2) {
        return (uint32_t(table[tok >> p.bs_shift]) << p.bs_shift) + (tok & (p.block_size - 1));
    } else {
        const uint32_t blk = tok / p.block_size;
        return uint32_t(table[blk]) * p.block_size + (tok - blk * p.block_size);
    }
}

__device__ __forceinline__ uint32_t lane_read(uint32_t v, uint32_t src_lane) {
    return uint32_t(__builtin_amdgcn_ds_bpermute(int(src_lane << 2), int(v)));
}


constexpr uint32_t kPlanHeader = 4;  // words in front of prefix[]

// The stream kernel keeps the prefix sums and the sequence lengths in LDS
// (60 KiB at most); larger batches go through the chunk kernel.
constexpr uint32_t kStreamMaxPrefix = 7680;
bool decode_stream_supports(uint32_t batch);
int launch_decode_stream(DecodeParams p, bool q_f32, int rows, const ScratchSource& scratch);

}  // namespace ghip
