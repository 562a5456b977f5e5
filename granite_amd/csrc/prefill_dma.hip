// Causal GQA prefill / chunked prefill for gfx950 with K/V tiles moved global -> LDS without
// passing through registers, and an inner loop whose every buffer offset is an immediate.
//
// Stands in for
//   flash_attention_prefill     src/backend/metal/kernels/metal_shaders_attention.h:1447-1660
// and follows the arithmetic of the CPU path it is checked against:
//   TransformerModel::attention       src/llm/transformer.mm:1779-1840
// (fp32 scores and softmax, no epsilon, key k visible iff k <= start_pos + q).
//
// It shares the grid, the partial-result layout and the merge launch of attention_tiles_kernel
// (prefill.hip), and its arithmetic: S^T = K Q^T and O^T = V^T P^T on v_mfma_f32_32x32x16_f16,
// a wave owning 32 query rows, the three-stage pipeline over 32-key sub-tiles (scores of
// j + 1, softmax of j, second product of j - 1 in one phase, a softmax element after every
// MFMA) and the lazy softmax reference.  What differs:
//
// * Tiles are staged with global_load_lds_dwordx4: a wave-wide instruction moves 64 x 16
//   bytes into 1 KiB of LDS, lane i's piece landing at M0 + 16 i; which piece of global memory
//   a lane asks for decides the layout.  No staging registers, no LDS store instructions, and
//   a tile in flight costs nothing but entries of the memory counter.  The 8 keys a wave
//   stages per tile lie in one block of a paged cache (block sizes of 8 tokens and more), so
//   the block-table entry is a scalar load and an address is a scalar base plus a lane
//   constant: no vector arithmetic per tile.  A ragged last tile falls back to per-lane
//   addresses with the key index clamped.
//     K tile: sixteen transfers of 8 keys x 128 bytes, key-major (lane i: key i >> 3, so
//       eight consecutive lanes fetch one whole 128-byte line; with the keys across the lanes
//       instead, a transfer touched eight lines eight times over and the causal prefill ran
//       2.4 % slower), the eight 16-byte pieces of a half row XOR-swizzled with the key's low
//       bits and the transfers 1152 bytes apart, so that the 16 lanes of an operand read (16
//       keys, one piece) fall into all 64 banks; the address of an operand is one of four lane
//       registers plus an immediate.
//     V tile: row-major 64 x 256 bytes, the four 64-byte chunks of a row XOR-swizzled with
//       the key's low two bits, as ds_read_b64_tr_b16 wants them (see prefill.hip); a transfer
//       is 4 keys x 256 bytes.
//   Four K and four V tiles are in LDS: of K the two being read, one landed, one in flight;
//   of V the same a tile later.  One wait for the memory counter and one barrier per tile.
// * The loop is unrolled four times, so the buffer a phase reads is a compile-time constant
//   and the steady state carries no buffer rotation, no per-tile row arithmetic and no mask
//   bookkeeping.  There is one code path: at the two ends of a wave's key range a stage that
//   does not apply runs on whatever its buffers hold and is made harmless.
//
// * A wave that has run out of keys (the early run under the causal pairing, the empty run of a
//   launch with few rows) stages its partner's share of every tile as well as its own, and the
//   partner, alone on its SIMD and bound by its own instruction stream, issues no transfer
//   (kHandOver; see the loops).
//
// * Tree-masked launches (kTree): the tree's own keys follow the cache's on the key axis from the
//   next tile boundary on and are staged with per-lane addresses; the rows' ancestor masks are
//   built in LDS from the parent pointers.  Launches of at most 64 rows (kSplit): two waves per
//   row block, each a sub-tile of every tile.  Both are described at the kernel.
//
// Limits (the caller checks them and uses attention_tiles_kernel otherwise): head size 128,
// an extra key segment only as the tree of a tree-masked launch of at most kMaxFusedNodes nodes
// behind a non-empty cache, contiguous cache or paged cache with a power-of-two block size >= 8.
// Queries fp16 or fp32 (fp32 as an fp16 head and an fp16 remainder: two MFMAs per step of the
// scores on one K operand).
//
// kRB, the number of 32-row blocks a wave owns, is 1.  With 2 (-DGHIP_DMA_RB=2: four waves of
// 64 rows, one per SIMD) an LDS operand read feeds two MFMAs; that form needs 434 registers per
// lane, the compiler keeps every MFMA result in accumulation registers and moves scores and
// probabilities between the two register files with about two extra vector instructions per
// MFMA, and it measured slower (chunked prefill 525 against 506 us on the same box, the causal
// prefill 68 against 52 us: there a wave then owns a SIMD and the longest row block's walk is
// not shared).
//
// Algorithmic work: 4 * D flops per visible (query, key) pair.
#include <type_traits>

#include "prefill_shared.h"

namespace ghip {
namespace {

constexpr int kD = 128;
#ifndef GHIP_DMA_RB
#define GHIP_DMA_RB 1
#endif

constexpr int kRB = GHIP_DMA_RB;  // 32-row blocks per wave
constexpr int kWaves = 8 / kRB;
constexpr int kWBM = 256;       // query rows per workgroup
constexpr int kWBN = 64;        // keys per tile
constexpr int kWThreads = 64 * kWaves;
constexpr int kWaveKeys = kWBN / kWaves;  // keys of a tile one wave stages: 8 (or 16)
constexpr int kStages = 4;                // tiles of K, and of V, in LDS
constexpr uint32_t kKChunk = 1152;            // bytes between the 1 KiB transfers of a K tile
constexpr uint32_t kKTile = 16 * kKChunk;     // 18432
constexpr uint32_t kVTile = kWBN * kD * 2;    // 16384
constexpr uint32_t kVRegion = kStages * kKTile;
constexpr uint32_t kEntryRegion = kStages * (kKTile + kVTile);  // 139264
constexpr uint32_t kEntries = 64;  // block-table entries a wave keeps in LDS: those of its next 64 tiles
constexpr size_t kDmaLds = kEntryRegion + size_t(kWaves) * kEntries * sizeof(uint32_t);
constexpr int kSteps = kD / 16;   // MFMAs of the scores of a sub-tile and row block
constexpr int kBlocks = kD / 32;  // 32-row head-dim blocks of O^T
constexpr int kSlots = 2 * kRB * kSteps;  // MFMAs of a phase; side work is issued after each
constexpr int kTransfers = 2 * (kWaveKeys / 8) + kWaveKeys / 4;  // per wave and tile (K + V)

template <int kV>
using IC = std::integral_constant<int, kV>;

typedef __attribute__((address_space(3))) unsigned char lds_byte;

__device__ __forceinline__ half8 as_half8(uint4v x) { return __builtin_bit_cast(half8, x); }

// One wave-wide transfer of 64 x 16 bytes from global memory straight into LDS: lane i's 16
// bytes land at LDS address lds_addr + 16 i.  Counted by vmcnt like any load; nothing tells
// the compiler that LDS changes, so every use is fenced by hand (wait + barrier).
// Scalar base + 32-bit lane offset:
__device__ __forceinline__ void dma_rows(uint32_t lds_addr, const void* sbase, uint32_t lane_off) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                 :
                 : "s"(lds_addr), "v"(lane_off), "s"(sbase));
}
// 64-bit address per lane:
__device__ __forceinline__ void dma_lanes(uint32_t lds_addr, const void* addr) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off"
                 :
                 : "s"(lds_addr), "v"(addr));
}
template <int kCount>
__device__ __forceinline__ void wait_transfers() {
    asm volatile("s_waitcnt vmcnt(%0)" : : "n"(kCount));
}

//
// kSplit (launches of at most 64 query rows, always with kHandOver): a row block is two of a
// workgroup's eight waves' worth of rows at most, so four of the first run's waves would find
// two idle.  Instead waves 0 and 1 take the even 32-key sub-tiles of every tile for row blocks 0
// and 1 and waves 2 and 3 the odd ones for the same rows: one phase per tile and wave instead
// of two (scores of tile it + 1, softmax of tile it, second product of tile it - 1, each of the
// wave's own sub-tile), four SIMDs computing instead of two, and the two halves of a row
// block's (m, l, O) combined through LDS at the end.
template <bool kQF32, bool kOutF32, bool kPaged, bool kHandOver, bool kTree, bool kSplit>
__global__ void __launch_bounds__(kWThreads, 2 / kRB) attention_tiles_dma_kernel(AttnParams p) {
    static_assert(!kSplit || (kHandOver && kRB == 1), "the split form is a hand-over form");
    extern __shared__ __attribute__((aligned(16))) unsigned char s_raw[];
    const uint32_t lds0 = uint32_t(uintptr_t((lds_byte*)s_raw));  // LDS address of the tile buffers

    const uint32_t tid = threadIdx.x;
    const uint32_t lane = tid & 63;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t n = lane & 31;  // query row inside a row block / MFMA row index m
    const uint32_t g = lane >> 5;  // MFMA k-group (0/1)

    // ---- which (query tile, head, key split): as in attention_tiles_kernel, ids remapped so
    // that the workgroups streaming the same K/V range run on one XCD and share its L2
    uint32_t job = blockIdx.x;
    {
        constexpr uint32_t kXcds = 8;
        const uint32_t total = gridDim.x;
        if (total % kXcds == 0) job = (job % kXcds) * (total / kXcds) + job / kXcds;
    }
    const uint32_t members = p.group * p.q_tiles;
    const uint32_t gidx = job / members, member = job - gidx * members;
    const uint32_t split = gidx % p.n_splits;
    const uint32_t head = (gidx / p.n_splits) * p.group + member / p.q_tiles;
    const uint32_t kvh = head / p.group;
    // two runs of 128 rows (half the waves each); under a causal mask the k-th run from the end
    // and the k-th from the start, so that every workgroup of a head has the same amount of work
    constexpr uint32_t kHalf = kWBM / 2;
    constexpr uint32_t kRunWaves = kWaves / 2, kWaveRows = 32 * kRB;
    const uint32_t slot = member % p.q_tiles;
    const uint32_t halves = (p.seq_q + kHalf - 1) / kHalf;
    const bool causal = p.mask_mode == GRANITE_HIP_MASK_CAUSAL;
    const uint32_t late_half = causal ? halves - 1 - slot : 2 * (p.q_tiles - 1 - slot) + 1;
    const uint32_t early_half = causal ? slot : late_half - 1;
    const bool second_run = wave >= kRunWaves;
    const bool run_live = !second_run || early_half < late_half;
    const uint32_t my_half = causal ? (second_run ? early_half : late_half)
                                    : (second_run ? late_half : early_half);
    // (split form: waves 2 and 3 have the rows of waves 0 and 1)
    const uint32_t row_wave = kSplit ? wave % 2 : wave % kRunWaves;
    const uint32_t my_sub = kSplit ? (wave % kRunWaves) / 2 : 0u;  // the sub-tile of every tile a split wave takes
    const uint32_t q0 = run_live ? my_half * kHalf + kWaveRows * row_wave : p.seq_q;
    const bool wave_active = q0 < p.seq_q;

    // ---- keys this workgroup visits: those of its later run
    uint32_t len_a = p.cache_len;
    if (causal) {
        const uint32_t q_last = min((late_half + 1) * kHalf, p.seq_q) - 1;
        len_a = min(len_a, p.start_pos + q_last + 1);
    }
    // A tree launch (kTree): the tree's own keys, the extra segment [num_kv_heads, extra_len, D],
    // follow the cache's on the key axis from the next tile boundary on, so that a tile holds
    // keys of one segment only.  Keys len_a .. pad_a - 1 do not exist (masked like a ragged end);
    // key pad_a + j is tree node j, visible to a row iff the row's ancestor mask has bit j.  Query row
    // r is node r mod extra_len: the launcher lays the rows of several heads of a KV group end to
    // end when the tree is small (seq_q a multiple of extra_len).
    const uint32_t len_b = kTree ? p.extra_len : 0u;
    const uint32_t pad_a = (len_a + kWBN - 1) / kWBN * kWBN;
    const uint32_t len_v = kTree ? pad_a + len_b : len_a;  // end of the key axis
    const uint32_t all_tiles = (len_v + kWBN - 1) / kWBN;
    // (32-bit products: the launcher refuses shapes where tiles x splits does not fit; a 64-bit
    // division here is a hundred scalar instructions in front of the first load)
    const uint32_t t_begin = all_tiles * split / p.n_splits;
    const uint32_t n_tiles = all_tiles * (split + 1) / p.n_splits;

    // ---- sub-tiles (32 keys, numbered from key 0) this wave computes: [j_begin, j_end); from
    // j_mask on a sub-tile holds a key some row of the wave must not see
    uint32_t j_end = 0, j_mask = 0;
    const uint32_t j_begin = 2 * t_begin;
    {
        uint32_t vis_end = 0;
        if (wave_active) {
            vis_end = len_v;
            if (causal) vis_end = min(vis_end, p.start_pos + min(q0 + kWaveRows, p.seq_q));
            vis_end = min(vis_end, n_tiles * kWBN);
        }
        j_end = max((vis_end + 31) / 32, j_begin);
        j_mask = len_a / 32;
        if (causal) j_mask = min(j_mask, (p.start_pos + q0 + 1) / 32);
    }

    // ---- Q^T as B operands: lane (n, g), row block rb, step s holds Q[q0 + 32 rb + n][16 s + 8 g .. +7]
    // (float queries: an fp16 head and an fp16 remainder, two MFMAs per step of the scores on the
    // same K operand, so float queries lose nothing)
    half8 bq[kRB][kSteps];
    half8 bq_lo[kQF32 ? kRB : 1][kQF32 ? kSteps : 1];
    uint32_t q_row[kRB];
#pragma unroll
    for (int rb = 0; rb < kRB; rb++) {
        q_row[rb] = q0 + 32 * rb + n;
        const uint32_t q_ld = min(q_row[rb], p.seq_q - 1);
        const int64_t qoff = int64_t(q_ld) * p.q_tok_stride + int64_t(head) * p.q_head_stride;
        if constexpr (kQF32) {
            const float* qp = static_cast<const float*>(p.q) + qoff + 8 * g;
#pragma unroll
            for (int s = 0; s < kSteps; s++) {
                const float4v x0 = *reinterpret_cast<const float4v*>(qp + 16 * s);
                const float4v x1 = *reinterpret_cast<const float4v*>(qp + 16 * s + 4);
                const float x[8] = {x0.x, x0.y, x0.z, x0.w, x1.x, x1.y, x1.z, x1.w};
                half8 hi, lo;
#pragma unroll
                for (int i = 0; i < 8; i++) {
                    const _Float16 h = static_cast<_Float16>(x[i]);
                    hi[i] = h;
                    lo[i] = static_cast<_Float16>(x[i] - static_cast<float>(h));
                }
                bq[rb][s] = hi;
                bq_lo[rb][s] = lo;
            }
        } else {
            const uint16_t* qp = static_cast<const uint16_t*>(p.q) + qoff + 8 * g;
#pragma unroll
            for (int s = 0; s < kSteps; s++) bq[rb][s] = as_half8(*reinterpret_cast<const uint4v*>(qp + 16 * s));
        }
    }

    float m_ref[kRB];  // reference maxima (log2 domain) the probabilities are relative to
    float l_run[kRB];  // lane-partial sums (the two k-groups are added at the end)
    float16v oacc[kRB][kBlocks];
#pragma unroll
    for (int rb = 0; rb < kRB; rb++) {
        m_ref[rb] = kNegBig;
        l_run[rb] = 0.0f;
#pragma unroll
        for (int t = 0; t < kBlocks; t++)
#pragma unroll
            for (int r = 0; r < 16; r++) oacc[rb][t][r] = 0.0f;
    }

    // ---- tree launches: the ancestor masks.  Row i has bit j set iff tree node i may attend node
    // j: itself and its ancestors (src/llm/transformer.mm:822-840).  A workgroup whose share of
    // the keys reaches the tree's own builds them in LDS from the parent pointers, one thread per
    // node, at most num_nodes steps, so a malformed array cannot hang it.  The pointers are
    // requested here and the masks are built in the prologue, behind the first tiles' transfers.
    __shared__ int32_t s_parent[kTree ? kMaxFusedNodes : 1];
    __shared__ uint32_t s_rowmask[kTree ? kMaxFusedNodes * (kMaxFusedNodes / 32) : 1];
    static_assert(!kTree || kMaxFusedNodes <= uint32_t(kWThreads), "one thread per node");
    const bool build_masks = kTree && t_begin < n_tiles && n_tiles * kWBN > pad_a;  // uniform over the workgroup
    int32_t my_parent = -1;
    if constexpr (kTree) {
        if (build_masks && tid < len_b) my_parent = p.tree_parents[tid];
    }
    auto build_tree_masks = [&]() __attribute__((always_inline)) {  // by every thread; leaves one barrier to the caller
        if (tid < len_b) s_parent[tid] = my_parent;
        for (uint32_t i = tid; i < len_b * p.mask_words; i += kWThreads) s_rowmask[i] = 0;
        __syncthreads();
        if (tid < len_b) {
            uint32_t* row = s_rowmask + tid * p.mask_words;
            row[tid >> 5] |= 1u << (tid & 31);
            int32_t cur = my_parent;
            for (uint32_t step = 0; step < len_b && cur >= 0 && cur < int32_t(len_b); step++) {
                row[uint32_t(cur) >> 5] |= 1u << (uint32_t(cur) & 31);
                cur = s_parent[cur];
            }
        }
    };

    // ---- staging.  Wave w moves keys kWaveKeys w .. + kWaveKeys - 1 of a tile.
    const int64_t stride_bytes = p.a_tok_stride * 2;  // between consecutive tokens of one KV head
    const unsigned char* const k_bytes = reinterpret_cast<const unsigned char*>(p.k + size_t(kvh) * p.a_head_stride);
    const unsigned char* const v_bytes = reinterpret_cast<const unsigned char*>(p.v + size_t(kvh) * p.a_head_stride);
    // the tree's keys of this KV head: rows of 2 D bytes one after the other (null without a tree)
    const unsigned char* const kx_bytes =
        kTree ? reinterpret_cast<const unsigned char*>(p.k_extra + size_t(kvh) * len_b * kD) : nullptr;
    const unsigned char* const vx_bytes =
        kTree ? reinterpret_cast<const unsigned char*>(p.v_extra + size_t(kvh) * len_b * kD) : nullptr;
    // byte offset of tree key `key` of the key axis inside them, clamped to the last node
    auto extra_row = [&](uint32_t key) __attribute__((always_inline)) -> uint64_t {
        return uint64_t(min(key - pad_a, len_b - 1)) * uint64_t(2 * kD);
    };
    // K transfer (a, h): key 8 a + (lane >> 3) of the wave's, whose slot lane & 7 receives the 16-byte
    // piece slot ^ key of half h of the row: eight consecutive lanes fetch one 128-byte line
    const uint32_t k_lane_off = uint32_t((lane >> 3) * stride_bytes) + 16 * ((lane & 7) ^ (lane >> 3));
    // V transfer j: keys 4 j + (lane >> 4) of the wave's; the lane's slot (lane & 15) holds 16-byte
    // piece slot ^ 4 (key & 3) of the row
    const uint32_t v_swizzled = 16 * ((lane & 15) ^ (((lane >> 4) & 3) << 2));
    const uint32_t v_lane_off = uint32_t((lane >> 4) * stride_bytes) + v_swizzled;
    // Block-table entries.  The keys of a wave's share of a tile lie in one block, so a share
    // needs one entry per tile.  Those of its next 64 tiles are kept in an LDS region of the
    // share's own (touched only by the wave that stages the share at the time; a barrier lies
    // between two that do), refilled with one vector load every 64 tiles: the compiler's wait for
    // that load also waits for the transfers in flight, which is why it is not issued per tile;
    // a read from LDS is counted apart from them.
    // All of these take the wave `sw` whose share of a tile is meant: normally the wave itself; a
    // wave that has run out of keys also stages the share of its partner that still computes
    // (see the loops below).
    uint32_t* const s_entries_all = reinterpret_cast<uint32_t*>(s_raw + kEntryRegion);
    auto fill_entries = [&](uint32_t sw, uint32_t first_tile) __attribute__((always_inline)) {  // of tiles first_tile .. + 63
        if constexpr (kPaged) {
            const uint32_t key = min(first_tile + lane, n_tiles - 1) * kWBN + kWaveKeys * sw;
            s_entries_all[sw * kEntries + lane] = uint32_t(p.table[min(key, len_a - 1) >> p.bs_shift]);
        }
    };
    auto group_entry = [&](uint32_t sw, uint32_t tile) __attribute__((always_inline)) -> uint32_t {  // one value for the wave, in every lane
        if constexpr (!kPaged) return 0u;
        return s_entries_all[sw * kEntries + (tile - t_begin) % kEntries];
    };
    // the same entry straight from the table (when a wave takes a share over)
    auto table_entry = [&](uint32_t sw, uint32_t tile) __attribute__((always_inline)) -> uint32_t {
        if constexpr (!kPaged) return 0u;
        const uint32_t key = min(tile, n_tiles - 1) * kWBN + kWaveKeys * sw;
        return uint32_t(p.table[min(key, len_a - 1) >> p.bs_shift]);
    };
    // row of the pool / cache that holds the first key of `tile` in the share of wave sw
    auto group_row = [&](uint32_t sw, uint32_t tile, uint32_t entry) __attribute__((always_inline)) -> uint32_t {
        const uint32_t key = tile * kWBN + kWaveKeys * sw;
        if constexpr (!kPaged) return key;
        return (__builtin_amdgcn_readfirstlane(entry) << p.bs_shift) + (key & (p.block_size - 1));
    };
    auto lane_row = [&](uint32_t key) __attribute__((always_inline)) -> uint32_t {  // any key, clamped to the last one
        key = min(key, len_a - 1);
        if constexpr (!kPaged) return key;
        return (uint32_t(p.table[key >> p.bs_shift]) << p.bs_shift) + (key & (p.block_size - 1));
    };
    // the share of wave sw of the K (V) tile into buffer `buf`; `row` is the share's group row
    // (unused for a ragged tile)
    auto stage_k = [&](uint32_t sw, uint32_t tile, uint32_t buf, uint32_t row) __attribute__((always_inline)) {
        const uint32_t dst = lds0 + buf * kKTile + (kWaveKeys / 8) * sw * kKChunk;
        if (kTree && tile * kWBN >= pad_a) {  // a tile of the tree's keys: per-lane addresses
#pragma unroll
            for (uint32_t a = 0; a < kWaveKeys / 8; a++) {
                const unsigned char* src = kx_bytes + extra_row(tile * kWBN + kWaveKeys * sw + 8 * a + (lane >> 3)) +
                                           16 * ((lane & 7) ^ (lane >> 3));
                dma_lanes(dst + a * kKChunk, src);
                dma_lanes(dst + (8 + a) * kKChunk, src + 128);
            }
        } else if ((tile + 1) * kWBN <= len_a) {
            const unsigned char* base = k_bytes + uint64_t(__builtin_amdgcn_readfirstlane(row)) * uint64_t(stride_bytes);
#pragma unroll
            for (uint32_t a = 0; a < kWaveKeys / 8; a++) {
                dma_rows(dst + a * kKChunk, base + 8 * a * stride_bytes, k_lane_off);
                dma_rows(dst + (8 + a) * kKChunk, base + 8 * a * stride_bytes + 128, k_lane_off);
            }
        } else {
#pragma unroll
            for (uint32_t a = 0; a < kWaveKeys / 8; a++) {
                const uint32_t r = lane_row(tile * kWBN + kWaveKeys * sw + 8 * a + (lane >> 3));
                const unsigned char* src = k_bytes + uint64_t(r) * uint64_t(stride_bytes) + 16 * ((lane & 7) ^ (lane >> 3));
                dma_lanes(dst + a * kKChunk, src);
                dma_lanes(dst + (8 + a) * kKChunk, src + 128);
            }
        }
    };
    auto stage_v = [&](uint32_t sw, uint32_t tile, uint32_t buf, uint32_t row) __attribute__((always_inline)) {
        const uint32_t dst = lds0 + kVRegion + buf * kVTile + kWaveKeys * sw * 256;
        if (kTree && tile * kWBN >= pad_a) {
#pragma unroll
            for (uint32_t j = 0; j < kWaveKeys / 4; j++)
                dma_lanes(dst + j * 1024,
                          vx_bytes + extra_row(tile * kWBN + kWaveKeys * sw + 4 * j + (lane >> 4)) + v_swizzled);
        } else if ((tile + 1) * kWBN <= len_a) {
            const unsigned char* base = v_bytes + uint64_t(__builtin_amdgcn_readfirstlane(row)) * uint64_t(stride_bytes);
#pragma unroll
            for (uint32_t j = 0; j < kWaveKeys / 4; j++) dma_rows(dst + j * 1024, base + 4 * j * stride_bytes, v_lane_off);
        } else {
#pragma unroll
            for (uint32_t j = 0; j < kWaveKeys / 4; j++) {
                const uint32_t r = lane_row(tile * kWBN + kWaveKeys * sw + 4 * j + (lane >> 4));
                dma_lanes(dst + j * 1024, v_bytes + uint64_t(r) * uint64_t(stride_bytes) + v_swizzled);
            }
        }
    };

    // ---- operand addresses in LDS (bytes from s_raw).  K: key 32 sub + n is row n & 7 of the
    // transfer 4 sub + (n >> 3) (+ 8 for the second half of the row); the 16-byte piece 2 s + g
    // of the row is piece (2 s + g) & 7 of its half and sits in slot piece ^ (n & 7): one lane
    // register per value of s & 3.  Everything else that depends on the step, the sub-tile and
    // the buffer is an immediate.
    uint32_t k_lane_j[4], k_lane_hi_j[4];
#pragma unroll
    for (uint32_t j = 0; j < 4; j++) {
        k_lane_j[j] = (n >> 3) * kKChunk + (n & 7) * 128 + 16 * ((2 * j + g) ^ (n & 7));
        k_lane_hi_j[j] = k_lane_j[j] + 2 * kKTile;
    }
    // V^T through ds_read_b64_tr_b16, as in attention_tiles_kernel: 16-lane group q4, lane
    // 4 k4 + r4 inside it points at key 4 g + k4, head-dim elements 32 t + 16 (q4 & 1) + 8 (r4 & 1)
    // + 4 (r4 >> 1) .. + 3 (chunk t stored at t ^ (key & 3))
    uint32_t vt_lane[kBlocks];
    {
        const uint32_t q4 = lane >> 4, i16 = lane & 15;
        const uint32_t k4 = i16 >> 2, r4 = i16 & 3;
        const uint32_t key = 4 * g + k4;
        const uint32_t in_chunk = 16 * (q4 & 1) + 8 * (r4 & 1) + 4 * (r4 >> 1);
#pragma unroll
        for (uint32_t t = 0; t < uint32_t(kBlocks); t++)
            vt_lane[t] = kVRegion + 2 * (key * kD + (((t ^ (k4 & 3)) << 5) | in_chunk));
    }
    auto k_operand = [&](auto kb, auto sub, int s8) __attribute__((always_inline)) -> uint4v {
        constexpr int kBuf = decltype(kb)::value, kSub = decltype(sub)::value;
        const uint32_t base = kBuf < 2 ? k_lane_j[s8 & 3] : k_lane_hi_j[s8 & 3];
        const uint32_t imm = (kBuf & 1) * kKTile + (s8 >> 2) * 8 * kKChunk + kSub * 4 * kKChunk;
        return *reinterpret_cast<const uint4v*>(s_raw + base + imm);
    };
    auto v_pair = [&](const unsigned char* vp) __attribute__((always_inline)) -> uint4v {
        const uint2v lo = __builtin_bit_cast(
            uint2v, __builtin_amdgcn_ds_read_tr16_b64_v4i16((short4v __attribute__((address_space(3)))*)(vp)));
        const uint2v hi = __builtin_bit_cast(
            uint2v, __builtin_amdgcn_ds_read_tr16_b64_v4i16((short4v __attribute__((address_space(3)))*)(vp + 8 * 256)));
        return uint4v{lo.x, lo.y, hi.x, hi.y};
    };
    auto v_operand = [&](auto vb, auto sub, int i) __attribute__((always_inline)) -> uint4v {  // step i: head-dim block i % 4, key half i / 4
        constexpr int kBuf = decltype(vb)::value, kSub = decltype(sub)::value;
        return v_pair(s_raw + vt_lane[i % kBlocks] + (kBuf * kVTile + kSub * 32 * 256 + (i / kBlocks) * 16 * 256));
    };

    // keys of sub-tile j that a row may not see become minus infinity
    auto apply_mask = [&](uint32_t j, float16v (&sacc)[kRB]) __attribute__((always_inline)) {
        const uint32_t key0 = 32 * j;
        if (kTree && key0 >= pad_a) {  // tree keys: inside the tree, and an ancestor of the row (or itself)
            const uint32_t node0 = key0 - pad_a;  // a multiple of 32
#pragma unroll
            for (int rb = 0; rb < kRB; rb++) {
                const uint32_t w = node0 >> 5;
                // (the launcher may have laid several heads' rows end to end: a row's node is row mod nodes)
                const uint32_t word = w < p.mask_words ? s_rowmask[(q_row[rb] % len_b) * p.mask_words + w] : 0u;
                const int32_t room = int32_t(len_b) - int32_t(node0 + 4 * g);
                const uint32_t bits = word >> (4 * g);
#pragma unroll
                for (int r = 0; r < 16; r++) {
                    const int kc = 8 * (r >> 2) + (r & 3);
                    if (!((room > kc) && ((bits >> kc) & 1u))) sacc[rb][r] = -INFINITY;
                }
            }
            return;
        }
#pragma unroll
        for (int rb = 0; rb < kRB; rb++) {
            const uint32_t limit = causal ? min(len_a, p.start_pos + q_row[rb] + 1) : len_a;
            // element r is key 8 (r >> 2) + (r & 3) + 4 g of the sub-tile
            const int32_t room = int32_t(limit) - int32_t(key0 + 4 * g);
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int kc = 8 * (r >> 2) + (r & 3);
                if (!(room > kc)) sacc[rb][r] = -INFINITY;
            }
        }
    };
    // moves the reference of row block rb up to cover the scores `sacc`; rescales l and O
    auto rebase = [&](int rb, const float16v& sacc) __attribute__((always_inline)) {
        float mraw = -INFINITY;
#pragma unroll
        for (int r = 0; r < 16; r++) mraw = fmaxf(mraw, sacc[r]);
        const LanePair both = half_wave_pair(mraw);
        const float m_tile = fmaxf(both.lo, both.hi) * p.scale_log2;
        const float m_new = fmaxf(m_ref[rb], m_tile);
        const float alpha = fast_exp2(m_ref[rb] - m_new);
        m_ref[rb] = m_new;
        l_run[rb] *= alpha;
#pragma unroll
        for (int t = 0; t < kBlocks; t++)
#pragma unroll
            for (int r = 0; r < 16; r++) oacc[rb][t][r] *= alpha;
    };
    auto probabilities_once = [&](int rb, const float16v& sacc, half8 (&bp)[2]) __attribute__((always_inline)) -> float {
        float psum = 0.0f;
#pragma unroll
        for (int u = 0; u < 2; u++) {
            float pe[8];
#pragma unroll
            for (int j = 0; j < 8; j++) {
                pe[j] = fast_exp2(__builtin_fmaf(sacc[8 * u + j], p.scale_log2, -m_ref[rb]));
                psum += pe[j];
            }
            uint4v w;
            w.x = pack_f16x2(pe[0], pe[1]);
            w.y = pack_f16x2(pe[2], pe[3]);
            w.z = pack_f16x2(pe[4], pe[5]);
            w.w = pack_f16x2(pe[6], pe[7]);
            bp[u] = as_half8(w);
        }
        return psum;
    };
    // O^T += V^T P^T of one sub-tile, buffer known only at run time (the drain after the loop)
    auto accumulate = [&](uint32_t buf, uint32_t sub, const half8 (&bp)[kRB][2]) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < 2 * kBlocks; i++) {
            const half8 a = as_half8(v_pair(s_raw + vt_lane[i % kBlocks] + buf * kVTile + sub * 32 * 256 + (i / kBlocks) * 16 * 256));
#pragma unroll
            for (int rb = 0; rb < kRB; rb++)
                oacc[rb][i % kBlocks] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, bp[rb][i / kBlocks], oacc[rb][i % kBlocks], 0, 0, 0);
        }
    };

    // ---- one phase of the three-stage pipeline: the scores of sub-tile j + 1 (K buffer kb,
    // sub-tile sub_q) into s_out, the softmax of sub-tile j (s_in -> p_out), the second product
    // of sub-tile j - 1 (V buffer vb, sub-tile sub_v, p_prev).  One score element becomes a
    // probability after every MFMA.  side(slot), slot 0 .. kSlots - 1, is the caller's work to
    // issue in the shadow of the MFMAs.
    // There is one code path: at the ends of a wave's key range a stage that does not apply
    // runs on whatever its buffers hold and is made harmless -- scores nobody reads, a
    // softmax (softmax_live false) that leaves l alone and hands on zero probabilities, a
    // second product with zero probabilities against finite V (the buffer read before any V
    // has landed is cleared at the start).
    auto fused_phase = [&](auto kb, auto sub_q, auto vb, auto sub_v, bool masked, bool softmax_live, uint32_t j_q,
                           float16v (&s_out)[kRB], const float16v (&s_in)[kRB], half8 (&p_out)[kRB][2],
                           const half8 (&p_prev)[kRB][2], auto&& side) __attribute__((always_inline)) {
        constexpr int kRing = 3;  // LDS operands are requested two MFMAs ahead
        uint4v ring[kRing];
#pragma unroll
        for (int i = 0; i < kRing - 1; i++) ring[i] = k_operand(kb, sub_q, i);
        float16v c[kRB];
#pragma unroll
        for (int rb = 0; rb < kRB; rb++)
#pragma unroll
            for (int r = 0; r < 16; r++) c[rb][r] = 0.0f;
        float psum[kRB], tn[kRB];
        float pe[kRB][16];
        uint32_t pw[kRB][8];
#pragma unroll
        for (int rb = 0; rb < kRB; rb++) {
            psum[rb] = 0.0f;
            tn[rb] = __builtin_fmaf(s_in[rb][0], p.scale_log2, -m_ref[rb]);
        }
        // step e of row block rb: exponential of element e, scale-and-subtract of element e + 1,
        // sum (and, in pairs, conversion) of element e - 1
        auto softmax_step = [&](int rb, int e) __attribute__((always_inline)) {
            pe[rb][e] = fast_exp2(tn[rb]);
            if (e < 15) tn[rb] = __builtin_fmaf(s_in[rb][e + 1], p.scale_log2, -m_ref[rb]);
            if (e > 0) psum[rb] += pe[rb][e - 1];
            if (e > 0 && (e & 1) == 0) pw[rb][e / 2 - 1] = pack_f16x2(pe[rb][e - 2], pe[rb][e - 1]);
            asm volatile("" : "+v"(pe[rb][e]), "+v"(tn[rb]), "+v"(psum[rb]));
            if (e > 0 && (e & 1) == 0) asm volatile("" : "+v"(pw[rb][e / 2 - 1]));
        };
#pragma unroll
        for (int s8 = 0; s8 < kSteps; s8++) {
            if (s8 + kRing - 1 < kSteps) ring[(s8 + kRing - 1) % kRing] = k_operand(kb, sub_q, s8 + kRing - 1);
#pragma unroll
            for (int rb = 0; rb < kRB; rb++) {
                c[rb] = __builtin_amdgcn_mfma_f32_32x32x16_f16(as_half8(ring[s8 % kRing]), bq[rb][s8], c[rb], 0, 0, 0);
                softmax_step(rb, s8);
                side(kRB * s8 + rb);
                __builtin_amdgcn_sched_barrier(0);
                if constexpr (kQF32) {
                    c[rb] = __builtin_amdgcn_mfma_f32_32x32x16_f16(as_half8(ring[s8 % kRing]), bq_lo[rb][s8], c[rb], 0, 0, 0);
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
        }
#pragma unroll
        for (int i = 0; i < kRing - 1; i++) ring[i] = v_operand(vb, sub_v, i);
        if (masked) apply_mask(j_q, c);  // rare
#pragma unroll
        for (int i = 0; i < 2 * kBlocks; i++) {
            if (i + kRing - 1 < 2 * kBlocks) ring[(i + kRing - 1) % kRing] = v_operand(vb, sub_v, i + kRing - 1);
#pragma unroll
            for (int rb = 0; rb < kRB; rb++) {
                oacc[rb][i % kBlocks] = __builtin_amdgcn_mfma_f32_32x32x16_f16(
                    as_half8(ring[i % kRing]), p_prev[rb][i / kBlocks], oacc[rb][i % kBlocks], 0, 0, 0);
                softmax_step(rb, kSteps + i);
                side(kRB * (kSteps + i) + rb);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
#pragma unroll
        for (int rb = 0; rb < kRB; rb++) {
            psum[rb] += pe[rb][15];
            pw[rb][7] = pack_f16x2(pe[rb][14], pe[rb][15]);
            p_out[rb][0] = as_half8(uint4v{pw[rb][0], pw[rb][1], pw[rb][2], pw[rb][3]});
            p_out[rb][1] = as_half8(uint4v{pw[rb][4], pw[rb][5], pw[rb][6], pw[rb][7]});
            if (softmax_live) {
                if (__any(!(psum[rb] < kProbLimit))) {  // rare: the reference has to move, redo the sub-tile
                    rebase(rb, s_in[rb]);
                    psum[rb] = probabilities_once(rb, s_in[rb], p_out[rb]);
                }
                l_run[rb] += psum[rb];
            } else {
                p_out[rb][0] = p_out[rb][1] = as_half8(uint4v{0, 0, 0, 0});
            }
            s_out[rb] = c[rb];
        }
    };

    // the scores of sub-tile `sub` of the K tile in buffer `buf` alone (start of the pipeline)
    auto scores = [&](uint32_t buf, uint32_t sub, float16v (&sacc)[kRB]) __attribute__((always_inline)) {
        float16v c[kRB];
#pragma unroll
        for (int rb = 0; rb < kRB; rb++)
#pragma unroll
            for (int r = 0; r < 16; r++) c[rb][r] = 0.0f;
#pragma unroll
        for (int s8 = 0; s8 < kSteps; s8++) {
            const half8 a = as_half8(*reinterpret_cast<const uint4v*>(
                s_raw + k_lane_j[s8 & 3] + buf * kKTile + (s8 >> 2) * 8 * kKChunk + sub * 4 * kKChunk));
#pragma unroll
            for (int rb = 0; rb < kRB; rb++) {
                c[rb] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, bq[rb][s8], c[rb], 0, 0, 0);
                if constexpr (kQF32) c[rb] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, bq_lo[rb][s8], c[rb], 0, 0, 0);
            }
        }
#pragma unroll
        for (int rb = 0; rb < kRB; rb++) sacc[rb] = c[rb];
    };

    // ---- who stages what.  A wave computes on tiles t_begin .. first_idle - 1 and only helps to
    // stage afterwards.  Under the causal pairing the two runs of a workgroup end far apart, and a
    // wave that still computes then has its SIMD to itself and is bound by its own instruction
    // stream: from the tile on which wave w ^ kRunWaves (same SIMD, other run) has gone idle, that
    // wave stages this wave's share of every tile as well as its own, and this wave issues no
    // transfer at all.  Both sides derive the hand-over from the same numbers.
    auto first_idle_of = [&](uint32_t w) __attribute__((always_inline)) -> uint32_t {
        const bool second = w >= kRunWaves;
        const bool live = !second || early_half < late_half;
        const uint32_t half = causal ? (second ? early_half : late_half) : (second ? late_half : early_half);
        const uint32_t first_row = live ? half * kHalf + kWaveRows * (kSplit ? w % 2 : w % kRunWaves) : p.seq_q;
        uint32_t vis_end = 0;
        if (first_row < p.seq_q) {
            vis_end = len_v;
            if (causal) vis_end = min(vis_end, p.start_pos + min(first_row + kWaveRows, p.seq_q));
            vis_end = min(vis_end, n_tiles * kWBN);
        }
        const uint32_t end = max((vis_end + 31) / 32, j_begin);  // its j_end
        // (split form: the second product lags a whole tile, so a range that ends in the first
        // half of a tile needs the tile behind it as well)
        return j_begin < end ? min((end + (kSplit ? 1u : 0u)) / 2, n_tiles - 1) + 1 : t_begin;
    };
    // (kHandOver false: every wave stages its own share throughout, and the loop carries no test
    // for it; the launcher says which -- handing over pays when the runs end far apart)
    const uint32_t partner = wave ^ kRunWaves;
    const uint32_t first_idle = first_idle_of(wave);
    const uint32_t partner_first_idle = kHandOver ? first_idle_of(partner) : n_tiles;

    // What a wave carries for a share it stages: at the start of iteration `it`, the block-table
    // entry of tile it + 3 (whose K is staged in that iteration) and the row of tile it + 2 (whose
    // V is).
    struct Share {
        uint32_t sw, entry_next, v_row;
    };
    // This iteration's transfers of a share: V of tile it + 2 (piece 0) and K of tile it + 3 (piece
    // 1) into buffers vbuf, kbuf.
    const auto stage_next = [&](Share& sh, uint32_t it, uint32_t kbuf, uint32_t vbuf, int piece) __attribute__((always_inline)) {
        if (piece == 0 && it + 2 < n_tiles) stage_v(sh.sw, it + 2, vbuf, sh.v_row);
        if (piece == 1 && it + 3 < n_tiles) {
            const uint32_t row = group_row(sh.sw, it + 3, sh.entry_next);
            stage_k(sh.sw, it + 3, kbuf, row);
            sh.v_row = row;
            if ((it + 4 - t_begin) % kEntries == 0) fill_entries(sh.sw, it + 4);
            sh.entry_next = group_entry(sh.sw, it + 4);
        }
    };
    // a share taken over at iteration `it`: its two values straight from the table (the LDS
    // region of the share holds what is needed from tile it + 4 on)
    const auto take_over = [&](uint32_t sw, uint32_t it) __attribute__((always_inline)) -> Share {
        Share sh;
        sh.sw = sw;
        sh.entry_next = table_entry(sw, it + 3);
        sh.v_row = group_row(sw, min(it + 2, n_tiles - 1), table_entry(sw, it + 2));
        return sh;
    };
    // What the next iteration reads (K of it + 2, V of it + 1) was requested an iteration ago:
    // the wave waits until no more transfers are outstanding than it issued in this iteration
    // (`shares` shares' worth), then the barrier.
    constexpr int kKTransfers = 2 * (kWaveKeys / 8), kVTransfers = kWaveKeys / 4;
    static_assert(kKTransfers + kVTransfers == kTransfers);
    const auto end_of_tile = [&](uint32_t it, uint32_t shares) __attribute__((always_inline)) {
        const bool k_issued = it + 3 < n_tiles, v_issued = it + 2 < n_tiles;
        if (shares == 0 || !v_issued) wait_transfers<0>();
        else if (shares == 1 && k_issued) wait_transfers<kTransfers>();
        else if (shares == 1) wait_transfers<kVTransfers>();
        else if (k_issued) wait_transfers<2 * kTransfers>();
        else wait_transfers<2 * kVTransfers>();
        __syncthreads();
    };

    if (t_begin < n_tiles) {  // uniform over the workgroup; an empty share writes a neutral partial
        // ---- prologue: K of the first three tiles and V of the first two into their buffers
        // (tile t_begin + i lives in buffer i & 3); every wave its own share
        fill_entries(wave, t_begin);
        {
            const uint32_t last = n_tiles - 1;
#pragma unroll
            for (uint32_t i = 0; i < 3; i++) {
                const uint32_t t = t_begin + i;
                if (t > last) break;
                const uint32_t row = group_row(wave, t, group_entry(wave, t));
                stage_k(wave, t, i, row);
                if (i < 2) stage_v(wave, t, i, row);
            }
        }
        Share mine;
        mine.sw = wave;
        mine.entry_next = group_entry(wave, t_begin + 3);
        mine.v_row = group_row(wave, min(t_begin + 2, n_tiles - 1), group_entry(wave, t_begin + 2));
        // V buffer 3 is read (against zero probabilities) before any tile has landed in it
        {
            uint4v* vclear = reinterpret_cast<uint4v*>(s_raw + kVRegion + 3 * kVTile);
#pragma unroll
            for (uint32_t i = 0; i < kVTile / 16 / kWThreads; i++) vclear[tid + i * kWThreads] = uint4v{0, 0, 0, 0};
        }
        if constexpr (kTree) {
            if (build_masks) build_tree_masks();  // visible after the barrier below
        }
        wait_transfers<0>();
        __syncthreads();

        float16v s0[kRB], s1[kRB];
        half8 p_old[kRB][2], p_new[kRB][2];
#pragma unroll
        for (int rb = 0; rb < kRB; rb++) {
            p_old[rb][0] = p_old[rb][1] = p_new[rb][0] = p_new[rb][1] = as_half8(uint4v{0, 0, 0, 0});
#pragma unroll
            for (int r = 0; r < 16; r++) s0[rb][r] = s1[rb][r] = 0.0f;
        }
        uint32_t it = t_begin;
        if constexpr (kSplit) {
            // ---- the split form: this wave's sub-tile (my_sub) of every tile.  In iteration `it`,
            // one phase: the scores of tile it + 1 (K buffer B + 1), the softmax of tile it, the
            // second product of tile it - 1 (V buffer B + 3).  Scores and probabilities alternate
            // between two sets of registers.
            auto split_run = [&](auto subc) __attribute__((always_inline)) {
                constexpr int kSub = decltype(subc)::value;
                if (2 * t_begin + kSub < j_end) {
                    scores(0, kSub, s0);
                    if (2 * t_begin + kSub >= j_mask) apply_mask(2 * t_begin + kSub, s0);
                }
                auto split_iteration = [&](auto bc, uint32_t itc, const float16v (&s_in)[kRB], float16v (&s_out)[kRB],
                                           const half8 (&p_prev)[kRB][2], half8 (&p_out)[kRB][2]) __attribute__((always_inline)) {
                    constexpr int B = decltype(bc)::value;
                    const uint32_t jc = 2 * itc + kSub, jn = jc + 2;
                    const bool staging = itc < partner_first_idle;  // else the partner stages this wave's share
                    fused_phase(IC<(B + 1) & 3>{}, IC<kSub>{}, IC<(B + 3) & 3>{}, IC<kSub>{}, jn >= j_mask, jc < j_end, jn, s_out,
                                s_in, p_out, p_prev, [&](int slot) __attribute__((always_inline)) {
                                    if (slot == 9 && staging) stage_next(mine, itc, (B + 3) & 3, (B + 2) & 3, 0);
                                    if (slot == 11 && staging) stage_next(mine, itc, (B + 3) & 3, (B + 2) & 3, 1);
                                });
                    end_of_tile(itc, staging ? 1 : 0);
                };
                __builtin_amdgcn_s_waitcnt(0x0F70);  // (see the plain loop below)
                if (it < first_idle) {
                    for (;;) {
                        split_iteration(IC<0>{}, it, s0, s1, p_old, p_new);
                        if (++it >= first_idle) break;
                        split_iteration(IC<1>{}, it, s1, s0, p_new, p_old);
                        if (++it >= first_idle) break;
                        split_iteration(IC<2>{}, it, s0, s1, p_old, p_new);
                        if (++it >= first_idle) break;
                        split_iteration(IC<3>{}, it, s1, s0, p_new, p_old);
                        if (++it >= first_idle) break;
                    }
                }
            };
            if (my_sub == 0) split_run(IC<0>{});
            else split_run(IC<1>{});
        } else {
        if (j_begin < j_end) {
            scores(0, 0, s0);
            if (j_begin >= j_mask) apply_mask(j_begin, s0);
        }
        // ---- tiles on which this wave computes.  Tile `it` is in buffers B (K and V), K of
        // it + 1 in B + 1, V of it - 1 in B + 3.  Both phases always run (no branch around them:
        // a conditional second product costs the register allocator a second set of output
        // registers); the stages that do not apply at the ends of the range are harmless.
        auto iteration = [&](auto bc, uint32_t it) __attribute__((always_inline)) {
            constexpr int B = decltype(bc)::value;
            const uint32_t j = 2 * it;
            const bool staging = !kHandOver || it < partner_first_idle;  // else the partner stages this wave's share
            fused_phase(IC<B>{}, IC<1>{}, IC<(B + 3) & 3>{}, IC<1>{}, j + 1 >= j_mask, j < j_end, j + 1, s1, s0,
                        p_new, p_old, [&](int slot) __attribute__((always_inline)) {
                            // (after the 10th and 12th MFMA of the first phase: measured best by 1 %)
                            if (slot == 9 && staging) stage_next(mine, it, (B + 3) & 3, (B + 2) & 3, 0);
                            if (slot == 11 && staging) stage_next(mine, it, (B + 3) & 3, (B + 2) & 3, 1);
                        });
            fused_phase(IC<(B + 1) & 3>{}, IC<0>{}, IC<B>{}, IC<0>{}, j + 2 >= j_mask, j + 1 < j_end, j + 2, s0, s1,
                        p_old, p_new, [](int) {});
            end_of_tile(it, staging ? 1 : 0);
        };
        // Every load the compiler knows of is complete here (vmcnt(0), as the builtin so that it
        // is visible to the compiler's own wait insertion): otherwise it carries one as pending
        // into the loop and waits for the memory counter, i.e. for the transfers in flight, in
        // the middle of the first phase.
        __builtin_amdgcn_s_waitcnt(0x0F70);
        if (it < first_idle) {
            for (;;) {
                iteration(IC<0>{}, it);
                if (++it >= first_idle) break;
                iteration(IC<1>{}, it);
                if (++it >= first_idle) break;
                iteration(IC<2>{}, it);
                if (++it >= first_idle) break;
                iteration(IC<3>{}, it);
                if (++it >= first_idle) break;
            }
        }
        }  // !kSplit
        // ---- tiles this wave only helps to stage (its rows see none of their keys): its own
        // share, taken back if the partner had it, and the partner's while that wave computes
        if (it < n_tiles) {
            if constexpr (kHandOver) mine = take_over(wave, it);
            if (kHandOver && it < partner_first_idle) {
                Share theirs = take_over(partner, it);
                for (; it < min(partner_first_idle, n_tiles); ++it) {
                    const uint32_t b = (it - t_begin) & 3;
                    stage_next(mine, it, (b + 3) & 3, (b + 2) & 3, 0);
                    stage_next(theirs, it, (b + 3) & 3, (b + 2) & 3, 0);
                    stage_next(mine, it, (b + 3) & 3, (b + 2) & 3, 1);
                    stage_next(theirs, it, (b + 3) & 3, (b + 2) & 3, 1);
                    end_of_tile(it, 2);
                }
            }
            for (; it < n_tiles; ++it) {
                const uint32_t b = (it - t_begin) & 3;
                stage_next(mine, it, (b + 3) & 3, (b + 2) & 3, 0);
                stage_next(mine, it, (b + 3) & 3, (b + 2) & 3, 1);
                end_of_tile(it, 1);
            }
        }
        // the second product of the last sub-tile, when the range ends with the last tile
        if constexpr (kSplit) {
            // (the wave's sub-tile of the last tile; its probabilities are in the set the last
            // iteration wrote: p_new after an odd number of iterations)
            if (2 * (n_tiles - 1) + my_sub < j_end && j_end > j_begin) {
                if ((first_idle - t_begin) & 1) accumulate((n_tiles - 1 - t_begin) & 3, my_sub, p_new);
                else accumulate((n_tiles - 1 - t_begin) & 3, my_sub, p_old);
            }
        } else {
            if (j_end == 2 * n_tiles && j_end > j_begin) accumulate((n_tiles - 1 - t_begin) & 3, 1, p_old);
        }
    }

    // ---- split form: the odd sub-tiles' (m, l, O) of a row block join the even ones' through LDS
    // (the tile buffers: every transfer has landed and, after the barrier, nobody reads them)
    if constexpr (kSplit) {
        float* const mbuf = reinterpret_cast<float*>(s_raw);  // [row block][64 O + m + l][lane]
        constexpr uint32_t kMergeFloats = (16 * kBlocks + 2) * 64;
        const bool first_run = wave < kRunWaves;
        __syncthreads();
        if (first_run && my_sub == 1) {
            float* dst = mbuf + row_wave * kMergeFloats + lane;
#pragma unroll
            for (int t = 0; t < kBlocks; t++)
#pragma unroll
                for (int r = 0; r < 16; r++) dst[(16 * t + r) * 64] = oacc[0][t][r];
            dst[16 * kBlocks * 64] = m_ref[0];
            dst[(16 * kBlocks + 1) * 64] = l_run[0];
        }
        __syncthreads();
        if (first_run && my_sub == 0) {
            const float* src = mbuf + row_wave * kMergeFloats + lane;
            const float m2 = src[16 * kBlocks * 64], l2 = src[(16 * kBlocks + 1) * 64];
            const float m = fmaxf(m_ref[0], m2);
            const float f1 = fast_exp2(m_ref[0] - m), f2 = fast_exp2(m2 - m);
#pragma unroll
            for (int t = 0; t < kBlocks; t++)
#pragma unroll
                for (int r = 0; r < 16; r++) oacc[0][t][r] = oacc[0][t][r] * f1 + src[(16 * t + r) * 64] * f2;
            l_run[0] = l_run[0] * f1 + l2 * f2;
            m_ref[0] = m;
        }
        if (my_sub != 0) return;  // the even sub-tiles' wave writes the rows
    }

    if (!wave_active) return;
#pragma unroll
    for (int rb = 0; rb < kRB; rb++) {
        const LanePair both = half_wave_pair(l_run[rb]);
        l_run[rb] = both.lo + both.hi;
    }
#pragma unroll
    for (int rb = 0; rb < kRB; rb++) {
        if (q_row[rb] >= p.seq_q) continue;
        if (p.n_splits > 1) {
            // partial result of this key range: O unnormalised, (m_ref, l) beside it
            const size_t row = (size_t(split) * p.num_heads + head) * p.seq_q + q_row[rb];
            float* po = p.part_o + row * kD;
#pragma unroll
            for (int t = 0; t < kBlocks; t++)
#pragma unroll
                for (int ah = 0; ah < 2; ah++) {
                    float x[8];
#pragma unroll
                    for (int e = 0; e < 8; e++) x[e] = oacc[rb][t][8 * ah + e];
                    float* op = po + 32 * t + 16 * ah + 8 * g;
                    *reinterpret_cast<float4v*>(op) = float4v{x[0], x[1], x[2], x[3]};
                    *reinterpret_cast<float4v*>(op + 4) = float4v{x[4], x[5], x[6], x[7]};
                }
            if (g == 0) {
                p.part_ml[row * 2 + 0] = m_ref[rb];
                p.part_ml[row * 2 + 1] = l_run[rb];
            }
            continue;
        }
        const float inv_l = 1.0f / l_run[rb];
        const int64_t ooff = int64_t(q_row[rb]) * p.out_tok_stride + int64_t(head) * p.out_head_stride;
        // accumulator [t][4 a + b] is head-dim element 32 t + 16 (a >> 1) + 8 g + 4 (a & 1) + b
#pragma unroll
        for (int t = 0; t < kBlocks; t++)
#pragma unroll
            for (int ah = 0; ah < 2; ah++) {
                float x[8];
#pragma unroll
                for (int e = 0; e < 8; e++) x[e] = oacc[rb][t][8 * ah + e] * inv_l;
                const uint32_t d = 32 * t + 16 * ah + 8 * g;
                if constexpr (kOutF32) {
                    float* op = static_cast<float*>(p.out) + ooff + d;
                    *reinterpret_cast<float4v*>(op) = float4v{x[0], x[1], x[2], x[3]};
                    *reinterpret_cast<float4v*>(op + 4) = float4v{x[4], x[5], x[6], x[7]};
                } else {
                    uint4v w;
                    w.x = pack_f16x2(x[0], x[1]);
                    w.y = pack_f16x2(x[2], x[3]);
                    w.z = pack_f16x2(x[4], x[5]);
                    w.w = pack_f16x2(x[6], x[7]);
                    *reinterpret_cast<uint4v*>(static_cast<uint16_t*>(p.out) + ooff + d) = w;
                }
            }
        if (p.lse && g == 0)
            p.lse[size_t(head) * p.seq_q + q_row[rb]] = (m_ref[rb] + __builtin_amdgcn_logf(l_run[rb])) * kLn2;
    }
}

template <bool kQF32, bool kOutF32, bool kPaged, bool kHandOver, bool kTree = false, bool kSplit = false>
int launch_dma(const AttnParams& p, dim3 grid) {
    auto kernel = attention_tiles_dma_kernel<kQF32, kOutF32, kPaged, kHandOver, kTree, kSplit>;
    static bool configured[kMaxDevices];  // the tile buffers exceed the 64 KiB default limit
    if (int rc = raise_dynamic_lds_limit(reinterpret_cast<const void*>(kernel), kDmaLds, configured)) return rc;
    kernel<<<grid, dim3(kWThreads), kDmaLds, ctx().stream>>>(p);
    return launch_status();
}

template <bool kQF32, bool kOutF32, bool kPaged>
int launch_dma_shape(const AttnParams& p, dim3 grid) {
    // Under a causal mask the two runs of a workgroup end up to seq_q keys apart.  When that is
    // a large part of the walk (a prompt from the start, a chunk longer than its prefix), the
    // waves of the run that ends first take over the staging of the other run's shares; behind a
    // long prefix the runs end almost together and the plain loop is the faster one (chunked
    // prefill over 32k tokens: 0.6 % slower with the hand-over compiled in).
    // The same holds when all the rows of a launch fit one run (at most 128 query rows): the other
    // run's waves are idle from the start.
    // A tree launch (its rows are the tree's nodes, at most kMaxFusedNodes) always takes the
    // hand-over form: correct for any shape, and its one instantiation per layout is enough.
    // At most 64 rows: the split form (two waves per row block, each a sub-tile of every tile).
    const bool split = p.seq_q <= uint32_t(kWBM / 4);
    if (p.mask_mode == GRANITE_HIP_MASK_TREE)
        return split ? launch_dma<kQF32, kOutF32, kPaged, true, true, true>(p, grid)
                     : launch_dma<kQF32, kOutF32, kPaged, true, true, false>(p, grid);
    if (split) return launch_dma<kQF32, kOutF32, kPaged, true, false, true>(p, grid);
    const bool hand_over =
        (p.mask_mode == GRANITE_HIP_MASK_CAUSAL && p.start_pos < p.seq_q) || p.seq_q <= uint32_t(kWBM / 2);
    return hand_over ? launch_dma<kQF32, kOutF32, kPaged, true>(p, grid)
                     : launch_dma<kQF32, kOutF32, kPaged, false>(p, grid);
}

template <bool kQF32, bool kOutF32>
int launch_dma_layout(const AttnParams& p, dim3 grid) {
    return p.table != nullptr ? launch_dma_shape<kQF32, kOutF32, true>(p, grid)
                              : launch_dma_shape<kQF32, kOutF32, false>(p, grid);
}

}  // namespace

size_t tiles_dma_lds_bytes() { return kDmaLds; }

int launch_tiles_dma(const AttnParams& p, dim3 grid, bool q_f32, bool out_f32) {
    if (p.table != nullptr && p.bs_shift < 3) return GRANITE_HIP_EUNSUPPORTED;
    // the kernel's share of the key tiles per split is computed in 32 bits
    if ((uint64_t(p.cache_len) / kWBN + uint64_t(p.extra_len) / kWBN + 2) * p.n_splits >= (1ull << 32))
        return GRANITE_HIP_EUNSUPPORTED;
    if (p.mask_mode == GRANITE_HIP_MASK_TREE) {
        // the kernel builds the ancestor masks itself and numbers the tree's keys behind the cache's
        if (!p.tree_parents || !p.k_extra || !p.v_extra || p.extra_len == 0 || p.extra_len > kMaxFusedNodes ||
            p.cache_len == 0 || p.seq_q % p.extra_len != 0)
            return GRANITE_HIP_EUNSUPPORTED;
    } else if (p.extra_len != 0) {
        return GRANITE_HIP_EUNSUPPORTED;
    }
    if (q_f32) return out_f32 ? launch_dma_layout<true, true>(p, grid) : launch_dma_layout<true, false>(p, grid);
    return out_f32 ? launch_dma_layout<false, true>(p, grid) : launch_dma_layout<false, false>(p, grid);
}

}  // namespace ghip
