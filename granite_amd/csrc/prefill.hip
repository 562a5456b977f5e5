// Causal GQA flash-attention prefill, chunked prefill over a paged cache and
// tree-masked attention for gfx950 (MFMA, K/V tiles staged in LDS): the launcher of
// granite_hip_attention, the register-staged tiles kernel, the split-K merge and the tree
// mask kernel.  Launches of head size 128 with a contiguous cache or blocks of a power of two
// of at least 8 tokens, and with no extra key segment other than a tree of at most
// kMaxFusedNodes nodes behind a non-empty cache, go to the direct-to-LDS form of the tiles
// kernel instead (prefill_dma.hip), which shares the grid, the partial layout and the merge;
// everything else runs the kernel of this file.
//
// Stands in for
//   flash_attention_prefill     src/backend/metal/kernels/metal_shaders_attention.h:1447-1660
//   attention_tree_f16kv        metal_shaders_attention.h:1677-1865
// and follows the arithmetic of the CPU path they are checked against:
//   TransformerModel::attention       src/llm/transformer.mm:1779-1840
//   TransformerModel::attention_tree  src/llm/transformer.mm:2044-2126
// (fp32 scores and softmax, no epsilon, key k visible iff k <= start_pos + q;
// tree: cache keys visible, tree key j visible iff j is q or an ancestor).
//
// Structure.  One workgroup of 8 waves (two per SIMD) per (256 query rows,
// query head, key split); a wave owns 32 query rows, and a K/V tile staged in
// LDS serves all 256.  The 256 rows are two runs of 128: the halves of one
// query tile or, under a causal mask, the k-th run from the end and the k-th
// from the start, so that every workgroup of a head has the same amount of
// work.  Workgroup ids are remapped so that the
// workgroups that stream the same K/V range (same KV head, same split) land on
// the same XCD and share its L2.  Keys are walked in tiles of 64, each handled
// as two 32-key sub-tiles.  Per sub-tile every wave computes, with
// v_mfma_f32_32x32x16_f16,
//
//   S^T[key, q]  = K[key, :] . Q[q, :]          (A = K from LDS, B = Q in VGPRs)
//   softmax in the result layout: a lane owns one query row and 16 of the 32
//   keys, so max/sum are in-lane plus one exchange between the wave's halves
//   O^T[d, q]   += V^T[d, key] . P^T[key, q]    (A = V^T from LDS, B = P in VGPRs)
//
// Computing the transposed products makes the softmax output of the first
// MFMA land exactly in the B-operand layout of the second: with the keys of a
// tile in their natural order the lane that owns S^T rows (keys) 8a + 4g + b
// needs, as B operand of the second MFMA, k-index 8g + 4a' + b for key
// 16u + 8a' + 4g + b, and the A operand (V^T) simply reads its keys in that
// order.
//
// Pipeline.  The three stages of consecutive sub-tiles run in one phase
// (fused_phase): the MFMAs of the scores of sub-tile j + 1, the softmax
// arithmetic of sub-tile j and the MFMAs of the second product of sub-tile
// j - 1, with one score element turned into a probability after every MFMA.
// On this part a 32x32x16 MFMA keeps the vector ALU busy for only half of its
// 32 cycles and transcendentals run beside it, so vector work placed between
// MFMAs costs next to nothing while the same work after a burst of MFMAs costs
// its full time.
//
// Data movement.  K/V tiles go global -> registers -> LDS (issued piecewise in the shadow
// of the first phase's MFMAs); a thread moves two
// 16-byte pieces of one key row of K and of V (one row lookup per thread and
// tile).  What is loaded in one iteration is stored two iterations later (two
// register sets); block-table lookups
// are issued two iterations before the loads that use them.  K is needed a tile earlier than V, so LDS holds three K
// tiles (being finished, next, being written) and three V tiles (previous,
// current, being written), which leaves one barrier per tile.  Both are stored
// row-major as they lie in memory.  K rows have a pitch of 136 halves.  V rows
// have no padding; the four 64-byte chunks of a row are XOR-swizzled with the
// low two bits of the key instead.  The V^T operand comes out of the row-major
// tile through ds_read_b64_tr_b16: inside a 16-lane group, lane 4k + r supplies
// the address of four consecutive head-dim elements of key k and lane j
// receives element j & 3 of the four lanes {4k' + (j >> 2)}, i.e. one head-dim
// element of four consecutive keys.  With the swizzle the four key rows a
// group reads fall into different bank groups, so neither the 16-byte stores
// nor the transposing reads conflict.  The head-dim order of the A-operand
// rows is chosen so that each lane ends up with runs of 8 consecutive output
// elements.
//
// Softmax rescaling is lazy: probabilities are taken relative to a per-row
// reference maximum that is not tracked tile by tile at all.  Only when the
// probabilities of a sub-tile sum to 2^14 or more (or to infinity, as in the
// first sub-tile, whose reference is still minus infinity) is the reference
// moved to the row maximum, O and l rescaled and the sub-tile redone.  Results
// are identical up to rounding, P stays inside half range, and neither the row
// maximum nor the accumulator rescale is paid for in almost every tile.
//
// Algorithmic work: 4 * D flops per visible (query, key) pair.
#include <cstdlib>

#include "prefill_shared.h"

namespace ghip {
namespace {

constexpr int kBM = 256;       // query rows per workgroup
constexpr int kBN = 64;        // keys per tile
constexpr int kThreads = 512;  // 8 waves, two per SIMD
constexpr int kKBuffers = 3;  // K runs a tile ahead of V and is read across two iterations
constexpr int kVBuffers = 3;  // V of the previous tile is still read while the next is written
// What depends on the head size kD (128, or 64: the reference's d64 kernels,
// metal_shaders_attention.h:1447-1660): tile pitches in LDS, MFMA steps of a score
// product (16 head-dim elements each) and 32-row blocks of the output.
template <int kD>
struct Geometry {
    static_assert(kD == 64 || kD == 128, "head sizes with kernels: 64 and 128");
    static constexpr int kKPitch = kD + 8;  // halves per K row in LDS
    static constexpr int kVPitch = kD;      // halves per V row in LDS (chunks swizzled, no padding)
    static constexpr int kKTileHalves = kBN * kKPitch;
    static constexpr int kVTileHalves = kBN * kVPitch;
    static constexpr size_t kLdsBytes =
        size_t(kKBuffers * kKTileHalves + kVBuffers * kVTileHalves) * sizeof(uint16_t);
    static constexpr int kSteps = kD / 16;   // MFMAs of the scores of a sub-tile
    static constexpr int kBlocks = kD / 32;  // 32-row head-dim blocks of O^T; also 64-byte chunks of a V row
    static constexpr int kPhase = kSteps + 2 * kBlocks;  // MFMAs of a pipeline phase
};
__device__ __forceinline__ half8 as_half8(uint4v x) { return __builtin_bit_cast(half8, x); }

// Row of the K/V array that holds key `idx`: of the cache segment (through the
// block table when paged) or, with `extra`, of the extra segment (row = idx).
// In two steps, so that the table entry can stay in flight while other loads are
// issued: row_lookup() issues the table load and keeps the offset inside the
// block; row_finish() combines them where the row is needed.  Branch-free on
// purpose: a load inside a conditional makes the compiler wait for every
// outstanding load at the join, which would serialise the pipeline.
struct RowLookup {
    uint32_t entry;  // block table entry (paged cache segment)
    uint32_t add;    // offset inside the block, or the row itself where no table applies
};

template <int kRows>
__device__ __forceinline__ RowLookup row_lookup(const AttnParams& p, uint32_t idx, bool extra) {
    RowLookup r;
    if constexpr (kRows == kRowsContiguous) {
        r.entry = 0;
        r.add = idx;
    } else {
        const uint32_t t = extra ? 0u : idx;  // always a valid table position
        if constexpr (kRows == kRowsPagedPow2) {
            r.entry = uint32_t(p.table[t >> p.bs_shift]);
            r.add = extra ? idx : (t & (p.block_size - 1));
        } else {
            const uint32_t blk = t / p.block_size;
            r.entry = uint32_t(p.table[blk]);
            r.add = extra ? idx : (t - blk * p.block_size);
        }
    }
    return r;
}

template <int kRows>
__device__ __forceinline__ uint32_t row_finish(const AttnParams& p, const RowLookup& r, bool extra) {
    if constexpr (kRows == kRowsContiguous) {
        return r.add;
    } else {
        const uint32_t e = extra ? 0u : r.entry;
        if constexpr (kRows == kRowsPagedPow2) return (e << p.bs_shift) + r.add;
        return e * p.block_size + r.add;
    }
}

template <bool kQF32, bool kOutF32, int kRows, int kD>
__global__ void __launch_bounds__(kThreads, 2) attention_tiles_kernel(AttnParams p) {
    using G = Geometry<kD>;
    constexpr int kKPitch = G::kKPitch, kVPitch = G::kVPitch, kKTileHalves = G::kKTileHalves,
                  kVTileHalves = G::kVTileHalves, kSteps = G::kSteps, kBlocks = G::kBlocks, kPhase = G::kPhase;
    extern __shared__ __attribute__((aligned(16))) uint16_t s_mem[];
    uint16_t* const s_k0 = s_mem;
    uint16_t* const s_v0 = s_mem + kKBuffers * kKTileHalves;

    const uint32_t tid = threadIdx.x;
    const uint32_t lane = tid & 63;
    const uint32_t wave = tid >> 6;
    const uint32_t n = lane & 31;  // query row inside the wave / MFMA row index m
    const uint32_t g = lane >> 5;  // MFMA k-group (0/1)

    // ---- which (query tile, head, key split) this workgroup computes.  Workgroups are
    // handed to the 8 XCDs round-robin by their linear id, and every XCD has its own L2;
    // the ids are therefore remapped so that an XCD receives a contiguous run of the list
    // ordered (kv head, split, head in group, query tile): the workgroups that stream the
    // same K/V range share an L2 instead of fetching it once per XCD.
    uint32_t job = blockIdx.x;
    {
        constexpr uint32_t kXcds = 8;
        const uint32_t total = gridDim.x;
        if (total % kXcds == 0) job = (job % kXcds) * (total / kXcds) + job / kXcds;
    }
    const uint32_t members = p.group * p.q_tiles;  // workgroups per (kv head, split)
    const uint32_t gidx = job / members, member = job - gidx * members;
    const uint32_t split = gidx % p.n_splits;
    const uint32_t head = (gidx / p.n_splits) * p.group + member / p.q_tiles;
    const uint32_t kvh = head / p.group;
    // ---- the query rows.  A workgroup holds two runs of 128 rows (half tiles), one per four
    // waves, so one per SIMD pair of waves.  Normally they are the two halves of query tile
    // `slot` from the end.  Under a causal mask the work of a half tile grows with its
    // position (4 .. 32 key tiles across 2048 tokens), so the k-th workgroup of a head takes
    // the k-th half tile from the end and the k-th from the start instead: every workgroup
    // then has the same number of (wave, key tile) steps, and while only the late half tile
    // still has keys to visit its waves have their SIMDs to themselves.
    constexpr uint32_t kHalf = kBM / 2;
    const uint32_t slot = member % p.q_tiles;
    const uint32_t halves = (p.seq_q + kHalf - 1) / kHalf;
    const bool paired = p.mask_mode == GRANITE_HIP_MASK_CAUSAL;
    const uint32_t late_half = paired ? halves - 1 - slot : 2 * (p.q_tiles - 1 - slot) + 1;
    const uint32_t early_half = paired ? slot : late_half - 1;
    // (an odd count leaves the middle half tile alone in its workgroup)
    const bool second_run = wave >= kThreads / 128;
    const bool run_live = !second_run || early_half < late_half;
    const uint32_t my_half = paired ? (second_run ? early_half : late_half)
                                    : (second_run ? late_half : early_half);
    const uint32_t q0 = run_live ? my_half * kHalf + 32 * (wave & 3) : p.seq_q;
    const uint32_t q_row = q0 + n;
    const bool wave_active = q0 < p.seq_q;
    const uint32_t q_ld = min(q_row, p.seq_q - 1);

    // ---- keys this workgroup has to visit: those of its later half tile
    uint32_t len_a = p.cache_len;
    if (p.mask_mode == GRANITE_HIP_MASK_CAUSAL) {
        const uint32_t q_last = min((late_half + 1) * kHalf, p.seq_q) - 1;
        len_a = min(len_a, p.start_pos + q_last + 1);
    }
    const uint32_t len_b = p.extra_len;
    const uint32_t tiles_a = (len_a + kBN - 1) / kBN;
    const uint32_t tiles_b = (len_b + kBN - 1) / kBN;
    const uint32_t all_tiles = tiles_a + tiles_b;
    // this workgroup's share of the key tiles when the keys are split
    const uint32_t t_begin = uint32_t(uint64_t(all_tiles) * split / p.n_splits);
    const uint32_t n_tiles = uint32_t(uint64_t(all_tiles) * (split + 1) / p.n_splits);

    const uint16_t* ka_base = p.k + size_t(kvh) * p.a_head_stride;
    const uint16_t* va_base = p.v + size_t(kvh) * p.a_head_stride;
    const uint16_t* kb_base = p.k_extra ? p.k_extra + size_t(kvh) * len_b * kD : nullptr;
    const uint16_t* vb_base = p.v_extra ? p.v_extra + size_t(kvh) * len_b * kD : nullptr;

    // ---- Q^T as B operand: lane (n, g), step s holds Q[q][16 s + 8 g .. +7]
    half8 bq[kSteps];
    half8 bq_lo[kQF32 ? kSteps : 1];
    {
        const int64_t qoff = int64_t(q_ld) * p.q_tok_stride + int64_t(head) * p.q_head_stride;
#pragma unroll
        for (int s = 0; s < kSteps; s++) {
            if constexpr (kQF32) {
                const float* qp = static_cast<const float*>(p.q) + qoff + 16 * s + 8 * g;
                float4v x0 = *reinterpret_cast<const float4v*>(qp);
                float4v x1 = *reinterpret_cast<const float4v*>(qp + 4);
                float x[8] = {x0.x, x0.y, x0.z, x0.w, x1.x, x1.y, x1.z, x1.w};
                half8 hi, lo;
#pragma unroll
                for (int i = 0; i < 8; i++) {
                    _Float16 h = static_cast<_Float16>(x[i]);
                    hi[i] = h;
                    lo[i] = static_cast<_Float16>(x[i] - static_cast<float>(h));
                }
                bq[s] = hi;
                bq_lo[s] = lo;
            } else {
                const uint16_t* qp = static_cast<const uint16_t*>(p.q) + qoff + 16 * s + 8 * g;
                bq[s] = as_half8(*reinterpret_cast<const uint4v*>(qp));
            }
        }
    }

    // ---- tree mask.  Row i of the ancestor matrix has bit j set iff tree node i may attend
    // node j: itself and its ancestors (src/llm/transformer.mm:822-840).  For trees of up to
    // kMaxFusedNodes nodes every workgroup builds the matrix in LDS from the parent pointers:
    // one thread per node walks the pointers (copied to LDS first), at most num_nodes steps,
    // so a malformed array cannot hang it.  That saves a launch and keeps the mask reads out
    // of the vector-memory queue.
    __shared__ int32_t s_parent[kMaxFusedNodes];
    __shared__ uint32_t s_rowmask[kMaxFusedNodes * (kMaxFusedNodes / 32)];
    if (p.tree_parents) {  // uniform
        for (uint32_t i = tid; i < p.extra_len; i += kThreads) s_parent[i] = p.tree_parents[i];
        for (uint32_t i = tid; i < p.extra_len * p.mask_words; i += kThreads) s_rowmask[i] = 0;
        __syncthreads();
        if (tid < p.extra_len) {
            uint32_t* row = s_rowmask + tid * p.mask_words;
            row[tid >> 5] |= 1u << (tid & 31);
            int32_t cur = s_parent[tid];
            for (uint32_t step = 0; step < p.extra_len && cur >= 0 && cur < int32_t(p.extra_len); step++) {
                row[uint32_t(cur) >> 5] |= 1u << (uint32_t(cur) & 31);
                cur = s_parent[cur];
            }
        }
        __syncthreads();
    }
    const uint32_t mask_row_index = min(q_row, p.extra_len - 1) * p.mask_words;
    const uint32_t* mask_row = p.tree_mask ? p.tree_mask + mask_row_index : nullptr;

    float m_ref = kNegBig;  // reference maximum (log2 domain) the probabilities are relative to
    float l_run = 0.0f;     // lane-partial sum (the two k-groups are added at the end)
    float16v oacc[kBlocks];
#pragma unroll
    for (int t = 0; t < kBlocks; t++)
#pragma unroll
        for (int r = 0; r < 16; r++) oacc[t][r] = 0.0f;

    // ---- tile staging: this thread moves two 16-byte pieces of key ld_r, columns ld_c and
    // ld_c + 8 of the 256-byte row, of K and of V (head size 64: one piece of the 128-byte
    // row): one row lookup and one address per thread and tile, and every load instruction
    // still covers whole 128-byte lines.
    static_assert(kThreads == 8 * kBN, "two 16-byte pieces of one row per thread");
    constexpr bool kTwoPieces = kD == 128;
    const uint32_t ld_c = tid & 7;   // 16-byte column of the first piece
    const uint32_t ld_r = tid >> 3;  // key inside the tile, 0 .. 63
    // V: the 64-byte chunk (col >> 2) of row `key` is stored at chunk (col >> 2) ^ (key mod
    // chunks per row); the second piece is two chunks further
    constexpr uint32_t kSwz = kBlocks - 1;
    const uint32_t v_st = ld_r * kVPitch + ((((ld_c >> 2) ^ (ld_r & kSwz)) << 5) | ((ld_c & 3) << 3));
    const uint32_t v_st2 = ld_r * kVPitch + (((((ld_c >> 2) + 2) ^ (ld_r & kSwz)) << 5) | ((ld_c & 3) << 3));
    const uint32_t k_st = ld_r * kKPitch + 8 * ld_c;

    // two register sets: the loads of an iteration are stored two iterations later
    uint4v kreg_a[2], vreg_a[2], kreg_b[2], vreg_b[2];

    // row of key ld_r of tile `it`: the lookup, and the row once the lookup has arrived
    auto tile_lookup = [&](uint32_t it) -> RowLookup {
        it = min(it, n_tiles - 1);
        const bool seg_b = it >= tiles_a;
        const uint32_t key0 = (seg_b ? it - tiles_a : it) * kBN;
        const uint32_t last = (seg_b ? len_b : len_a) - 1;
        return row_lookup<kRows>(p, min(key0 + ld_r, last), seg_b);
    };
    auto tile_row = [&](uint32_t it, const RowLookup& r) -> uint32_t {
        return row_finish<kRows>(p, r, min(it, n_tiles - 1) >= tiles_a);
    };
    // K and V of a tile are moved separately: K runs one tile ahead of V (see the loop).
    // load_k returns the element offset of its row; the V load of the same tile, issued one
    // iteration later, starts from that offset instead of multiplying again.
    auto load_k = [&](uint32_t it, uint32_t row, uint4v (&kreg)[2]) -> int64_t {
        it = min(it, n_tiles - 1);
        const bool seg_b = it >= tiles_a;
        const uint16_t* kb = (seg_b ? kb_base : ka_base) + 8 * ld_c;
        const int64_t stride = seg_b ? int64_t(kD) : p.a_tok_stride;
        const int64_t off = int64_t(row) * stride;
        const uint4v* src = reinterpret_cast<const uint4v*>(kb + off);
        kreg[0] = src[0];
        if constexpr (kTwoPieces) kreg[1] = src[8];
        return off;
    };
    auto load_v = [&](uint32_t it, int64_t off, uint4v (&vreg)[2]) {
        it = min(it, n_tiles - 1);
        const bool seg_b = it >= tiles_a;
        const uint16_t* vb = (seg_b ? vb_base : va_base) + 8 * ld_c;
        const uint4v* src = reinterpret_cast<const uint4v*>(vb + off);
        vreg[0] = src[0];
        if constexpr (kTwoPieces) vreg[1] = src[8];
    };
    auto store_k_piece = [&](uint32_t buf, const uint4v (&kreg)[2], int piece) {
        if (piece && !kTwoPieces) return;
        uint4v* dst = reinterpret_cast<uint4v*>(s_k0 + buf * kKTileHalves + k_st);
        dst[8 * piece] = kreg[piece];
    };
    auto store_v_piece = [&](uint32_t buf, const uint4v (&vreg)[2], int piece) {
        if (piece && !kTwoPieces) return;
        uint16_t* sv = s_v0 + buf * kVTileHalves;
        *reinterpret_cast<uint4v*>(sv + (piece ? v_st2 : v_st)) = vreg[piece];
    };
    auto store_k = [&](uint32_t buf, const uint4v (&kreg)[2]) {
        store_k_piece(buf, kreg, 0);
        store_k_piece(buf, kreg, 1);
    };
    auto store_v = [&](uint32_t buf, const uint4v (&vreg)[2]) {
        store_v_piece(buf, vreg, 0);
        store_v_piece(buf, vreg, 1);
    };

    // ---- V^T operand reads.  16-lane group q = lane / 16, lane i = 4k + r inside it:
    // the lane points at key 4 g + k (plus the step's first key), head-dim elements
    // 32 t + 16 (q & 1) + 8 (r & 1) + 4 (r >> 1) .. + 3, and receives, as row n of the A
    // operand, one head-dim element of four consecutive keys.
    uint32_t vt_off[kBlocks];  // halves, per head-dim block t
    {
        const uint32_t q4 = lane >> 4, i16 = lane & 15;
        const uint32_t k4 = i16 >> 2, r4 = i16 & 3;
        const uint32_t key = 4 * g + k4;
        const uint32_t in_chunk = 16 * (q4 & 1) + 8 * (r4 & 1) + 4 * (r4 >> 1);
#pragma unroll
        for (uint32_t t = 0; t < uint32_t(kBlocks); t++)
            vt_off[t] = key * kVPitch + (((t ^ (k4 & kSwz)) << 5) | in_chunk);
    }

    // ---- per-tile pieces
    struct TileInfo {
        bool seg_b, active;
        uint32_t key0, seg_len;
    };
    auto tile_info = [&](uint32_t it) -> TileInfo {
        TileInfo ti;
        ti.seg_b = it >= tiles_a;
        ti.key0 = (ti.seg_b ? it - tiles_a : it) * kBN;
        ti.seg_len = ti.seg_b ? len_b : len_a;
        ti.active = wave_active && it < n_tiles;
        if (p.mask_mode == GRANITE_HIP_MASK_CAUSAL && !ti.seg_b) {
            const uint32_t q_last_wave = min(q0 + 32, p.seq_q) - 1;
            if (ti.key0 > p.start_pos + q_last_wave) ti.active = false;  // nothing visible to this wave
        }
        return ti;
    };
    // S^T of the 32-key sub-tile `sub` of the tile whose K is in buffer `kbuf`
    auto scores = [&](uint32_t kbuf, int sub, float16v& sacc) {
        const uint16_t* krow = s_k0 + kbuf * kKTileHalves + (32 * sub + n) * kKPitch + 8 * g;
        float16v c = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
        for (int s8 = 0; s8 < kSteps; s8++) {
            const half8 a = as_half8(*reinterpret_cast<const uint4v*>(krow + 16 * s8));
            c = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, bq[s8], c, 0, 0, 0);
            if constexpr (kQF32) c = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, bq_lo[s8], c, 0, 0, 0);
        }
        sacc = c;
    };
    // Masks of a sub-tile; returns at once on the (common) sub-tiles that need none.
    auto apply_mask = [&](const TileInfo& ti, int sub, float16v& sacc) {
        const uint32_t key0 = ti.key0 + 32 * sub;
        const bool partial = key0 + 32 > ti.seg_len;
        const bool diagonal = p.mask_mode == GRANITE_HIP_MASK_CAUSAL && !ti.seg_b &&
                              key0 + 31 > p.start_pos + q0;
        const bool tree = p.mask_mode == GRANITE_HIP_MASK_TREE && ti.seg_b;
        if (!(partial || diagonal || tree)) return false;
        uint32_t mw = 0xFFFFFFFFu;
        if (tree) {
            const uint32_t w = key0 >> 5;
            mw = w >= p.mask_words ? 0u : (p.tree_parents ? s_rowmask[mask_row_index + w] : mask_row[w]);
        }
        const uint32_t limit = diagonal ? min(ti.seg_len, p.start_pos + q_row + 1) : ti.seg_len;
        // Element r is key 8 (r >> 2) + (r & 3) + 4 g of the sub-tile: everything that
        // depends on the lane goes into `room` and the shifted mask word, the rest is
        // a compile-time constant (no per-element registers).
        const int32_t room = int32_t(limit) - int32_t(key0 + 4 * g);
        const uint32_t bits = mw >> (4 * g);
#pragma unroll
        for (int r = 0; r < 16; r++) {
            const int kc = 8 * (r >> 2) + (r & 3);
            const bool vis = (room > kc) && ((bits >> kc) & 1u);
            if (!vis) sacc[r] = -INFINITY;
        }
        return true;
    };
    // The reference maximum is not tracked tile by tile: probabilities are taken relative to
    // the current reference, and only when those of a sub-tile sum to kProbLimit or more
    // (or to infinity: the first sub-tile, whose reference is still minus infinity) is the
    // reference moved to the row maximum and the sub-tile redone.  That keeps the maximum
    // (16 comparisons, an exchange between the half waves) out of almost every sub-tile.
    // A probability below kProbLimit is far inside half range; results are the same up to
    // rounding because O, l and P always share one reference.
    // rebase(): moves the reference up to cover the scores `sacc` and rescales l and O.
    auto rebase = [&](const float16v& sacc) {
        float mraw = -INFINITY;
#pragma unroll
        for (int r = 0; r < 16; r++) mraw = fmaxf(mraw, sacc[r]);
        const LanePair both = half_wave_pair(mraw);
        const float m_tile = fmaxf(both.lo, both.hi) * p.scale_log2;
        const float m_new = fmaxf(m_ref, m_tile);
        const float alpha = fast_exp2(m_ref - m_new);
        m_ref = m_new;
        l_run *= alpha;
#pragma unroll
        for (int t = 0; t < kBlocks; t++)
#pragma unroll
            for (int r = 0; r < 16; r++) oacc[t][r] *= alpha;
    };
    // P^T = exp2(S^T * scale - m_ref) of a sub-tile as B operands of the second product;
    // adds to l.
    auto probabilities_once = [&](const float16v& sacc, half8 (&bp)[2]) -> float {
        float psum = 0.0f;
#pragma unroll
        for (int u = 0; u < 2; u++) {
            float pe[8];
#pragma unroll
            for (int j = 0; j < 8; j++) {
                pe[j] = fast_exp2(__builtin_fmaf(sacc[8 * u + j], p.scale_log2, -m_ref));
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
    auto probabilities = [&](const float16v& sacc, half8 (&bp)[2]) {
        float psum = probabilities_once(sacc, bp);
        if (__any(!(psum < kProbLimit))) {
            rebase(sacc);
            psum = probabilities_once(sacc, bp);
        }
        l_run += psum;
    };
    // O^T += V^T P^T for sub-tile `sub` of the tile whose V is in buffer `vbuf`
    auto accumulate = [&](uint32_t vbuf, int sub, const half8 (&bp)[2]) {
        const uint16_t* sv = s_v0 + vbuf * kVTileHalves + 32 * sub * kVPitch;
#pragma unroll
        for (int t = 0; t < kBlocks; t++) {
#pragma unroll
            for (int u = 0; u < 2; u++) {
                // keys 16 u + {0, 8} + 4 g + (0..3) of the sub-tile: k-index 8 g + 4 a' + b
                const uint16_t* vp = sv + vt_off[t] + 16 * u * kVPitch;
                const uint2v lo = __builtin_bit_cast(
                    uint2v, __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                                (short4v __attribute__((address_space(3)))*)(vp)));
                const uint2v hi = __builtin_bit_cast(
                    uint2v, __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                                (short4v __attribute__((address_space(3)))*)(vp + 8 * kVPitch)));
                const uint4v a16 = {lo.x, lo.y, hi.x, hi.y};
                oacc[t] = __builtin_amdgcn_mfma_f32_32x32x16_f16(as_half8(a16), bp[u], oacc[t], 0,
                                                                 0, 0);
            }
        }
    };

    // One phase of the three-stage pipeline, instruction streams interleaved by hand.  For
    // sub-tile j it runs
    //   the 8 MFMAs of the scores of sub-tile j + 1        (K operands from LDS),
    //   the softmax arithmetic of sub-tile j               (scores s_in -> probabilities p_out),
    //   the 8 MFMAs of the second product of sub-tile j - 1 (V^T operands from LDS, p_prev),
    // with one score element turned into a probability after every MFMA, so that all 16
    // MFMAs of a phase have vector work of an *earlier* sub-tile to hide: on this part a
    // 32x32x16 MFMA keeps the vector ALU to itself for only half of its 32 cycles and
    // transcendentals run beside it, so a few vector instructions between MFMAs are free
    // while the same instructions after a burst of MFMAs are not.  The scheduling barriers
    // and the empty asm statements keep the compiler from regrouping or sinking the slices.
    // side(step) is called after the vector work of every step (0 .. kPhase - 1) for work of the
    // caller's that should issue in the shadow of the MFMAs (the tile staging).
    // Operands are fetched from LDS two steps ahead.  Step e scales element e + 1, takes the
    // exponential of element e and sums / packs element e - 1.
    auto fused_phase = [&](const TileInfo& ti_q, uint32_t kbuf, int sub_q, float16v& s_out,
                           const float16v& s_in, half8 (&p_out)[2], uint32_t vbuf, int sub_v,
                           const half8 (&p_prev)[2], auto&& side) {
        const uint16_t* krow = s_k0 + kbuf * kKTileHalves + (32 * sub_q + n) * kKPitch + 8 * g;
        const uint16_t* sv = s_v0 + vbuf * kVTileHalves + 32 * sub_v * kVPitch;
        auto k_operand = [&](int s8) -> uint4v {
            return *reinterpret_cast<const uint4v*>(krow + 16 * s8);
        };
        auto v_operand = [&](int i) -> uint4v {  // step i: head-dim block i % kBlocks, key half i / kBlocks
            const uint16_t* vp = sv + vt_off[i % kBlocks] + 16 * (i / kBlocks) * kVPitch;
            const uint2v lo = __builtin_bit_cast(
                uint2v, __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                            (short4v __attribute__((address_space(3)))*)(vp)));
            const uint2v hi = __builtin_bit_cast(
                uint2v, __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                            (short4v __attribute__((address_space(3)))*)(vp + 8 * kVPitch)));
            return uint4v{lo.x, lo.y, hi.x, hi.y};
        };
        constexpr int kRing = 3;
        uint4v ring[kRing];
#pragma unroll
        for (int i = 0; i < kRing - 1; i++) ring[i] = k_operand(i);
        float16v c = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
        float psum = 0.0f;
        float pe[16];
        uint32_t pw[8];
        float tn = __builtin_fmaf(s_in[0], p.scale_log2, -m_ref);
        // the vector work of step e (0..15); element e - 1 is finished here, in pairs
        auto softmax_step = [&](int e) {
            pe[e] = fast_exp2(tn);
            if (e < 15) tn = __builtin_fmaf(s_in[e + 1], p.scale_log2, -m_ref);
            if (e > 0) psum += pe[e - 1];
            if (e > 0 && (e & 1) == 0) pw[e / 2 - 1] = pack_f16x2(pe[e - 2], pe[e - 1]);
            asm volatile("" : "+v"(pe[e]), "+v"(tn), "+v"(psum));
            if (e > 0 && (e & 1) == 0) asm volatile("" : "+v"(pw[e / 2 - 1]));
        };
        // the 16 elements are spread evenly over the phase's MFMAs (one each at head size
        // 128, two each at 64)
        constexpr int kPer = 16 / kPhase;
        auto vector_work = [&](int step) {
#pragma unroll
            for (int j = 0; j < kPer; j++) softmax_step(step * kPer + j);
            side(step);
        };
#pragma unroll
        for (int s8 = 0; s8 < kSteps; s8++) {
            if (s8 + kRing - 1 < kSteps) ring[(s8 + kRing - 1) % kRing] = k_operand(s8 + kRing - 1);
            c = __builtin_amdgcn_mfma_f32_32x32x16_f16(as_half8(ring[s8 % kRing]), bq[s8], c, 0, 0, 0);
            if constexpr (kQF32)
                c = __builtin_amdgcn_mfma_f32_32x32x16_f16(as_half8(ring[s8 % kRing]), bq_lo[s8], c, 0, 0, 0);
            vector_work(s8);
            __builtin_amdgcn_sched_barrier(0);
        }
#pragma unroll
        for (int i = 0; i < kRing - 1; i++) ring[i] = v_operand(i);
        apply_mask(ti_q, sub_q, c);  // rare
#pragma unroll
        for (int i = 0; i < 2 * kBlocks; i++) {
            if (i + kRing - 1 < 2 * kBlocks) ring[(i + kRing - 1) % kRing] = v_operand(i + kRing - 1);
            oacc[i % kBlocks] = __builtin_amdgcn_mfma_f32_32x32x16_f16(
                as_half8(ring[i % kRing]), p_prev[i / kBlocks], oacc[i % kBlocks], 0, 0, 0);
            vector_work(kSteps + i);
            __builtin_amdgcn_sched_barrier(0);
        }
        psum += pe[15];
        pw[7] = pack_f16x2(pe[14], pe[15]);
        p_out[0] = as_half8(uint4v{pw[0], pw[1], pw[2], pw[3]});
        p_out[1] = as_half8(uint4v{pw[4], pw[5], pw[6], pw[7]});
        if (__any(!(psum < kProbLimit))) {  // rare: the reference has to move, redo the sub-tile
            rebase(s_in);
            psum = probabilities_once(s_in, p_out);
        }
        l_run += psum;
        s_out = c;
    };

    if (t_begin < n_tiles) {  // uniform over the workgroup; an empty share writes a neutral partial
    // ---- prologue.  In LDS: K of the first two tiles, V of the first.  In flight: K of the
    // third and fourth tile, V of the second and third.  Row lookups: one tile further.
    // K and V of tile t_begin + j live in buffers j % 3.
    const uint32_t r0 = tile_row(t_begin, tile_lookup(t_begin));
    const uint32_t r1 = tile_row(t_begin + 1, tile_lookup(t_begin + 1));
    const uint32_t r2 = tile_row(t_begin + 2, tile_lookup(t_begin + 2));
    const uint32_t r3 = tile_row(t_begin + 3, tile_lookup(t_begin + 3));
    const int64_t o0 = load_k(t_begin, r0, kreg_a);
    load_v(t_begin, o0, vreg_a);
    const int64_t o1 = load_k(t_begin + 1, r1, kreg_b);
    store_k(0, kreg_a);
    store_v(0, vreg_a);
    store_k(1, kreg_b);
    // From here on a lookup is issued two iterations before the loads that use it, and kept
    // with the register set (a / b) that those loads fill.  The counter of outstanding loads
    // is in order: a load's address then depends on nothing younger than the loads that the
    // stores of the same iteration wait for anyway, and the K/V loads of the previous
    // iteration stay in flight.  The prologue issues its loads in the loop's order (K, V,
    // lookup; set a, then set b) so that the waits the compiler derives for the loop's first
    // pass are those of every other pass.
    // set a: K of tile t_begin + 2, V of t_begin + 1; set b: K of t_begin + 3, V of t_begin + 2
    __builtin_amdgcn_sched_barrier(0);  // (the scheduler would move the lookups to the front)
    const int64_t o2 = load_k(t_begin + 2, r2, kreg_a);
    load_v(t_begin + 1, o1, vreg_a);
    __builtin_amdgcn_sched_barrier(0);
    RowLookup look_a = tile_lookup(t_begin + 4);
    __builtin_amdgcn_sched_barrier(0);
    int64_t off_v = load_k(t_begin + 3, r3, kreg_b);  // of the tile whose V is loaded next
    load_v(t_begin + 2, o2, vreg_b);
    __builtin_amdgcn_sched_barrier(0);
    RowLookup look_b = tile_lookup(t_begin + 5);
    __builtin_amdgcn_sched_barrier(0);
    __syncthreads();

    // The loop is software pipelined three deep over 32-key sub-tiles (see fused_phase).
    // On entry to an iteration s0 holds the scores of sub-tile 0 of tile `it` and p_old the
    // probabilities of sub-tile 1 of tile it - 1, whose second product is still due.  K is
    // therefore staged one tile ahead of V, and both are kept in three buffers (K: the tile
    // being finished, the next one, the one being written; V: the previous tile, the
    // current one, the one being written), which leaves one barrier per tile.
    float16v s0, s1;
    half8 p_old[2], p_new[2];
    {
        const TileInfo first = tile_info(t_begin);
        if (first.active) {
            scores(0, 0, s0);
            apply_mask(first, 0, s0);
        }
    }
    uint32_t kb_cur = 0, kb_next = 1, kb_store = 2;  // K buffers of tiles it, it + 1, it + 2
    uint32_t vb_prev = 2, vb_cur = 0, vb_store = 1;  // V buffers of tiles it - 1, it, it + 1
    bool prev_active = false;                        // tile it - 1 was computed by this wave
    auto iteration = [&](uint32_t it, uint4v (&kreg)[2], uint4v (&vreg)[2], RowLookup& look) {
        const TileInfo cur = tile_info(it);
        const TileInfo nxt = tile_info(it + 1);
        const bool fused = prev_active && cur.active && nxt.active;  // the common case
        // Staging, on every path (indices clamp at the last tile; stores past the last tile go
        // to buffers nobody reads any more): what is stored now was requested two iterations
        // ago (the register set alternates), and the target buffers (K of tile it - 1, V of
        // tile it - 2) have been free since the last barrier.  In a fused iteration its
        // pieces are spread over the second half of the first phase, one per MFMA, so that
        // the matrix cores do not idle while the waves of a SIMD store and load together.
        auto staging = [&](int piece) {
            if (piece == 0) store_k_piece(kb_store, kreg, 0);  // K of tile it + 2
            if (piece == 1) store_k_piece(kb_store, kreg, 1);
            if (piece == 2) store_v_piece(vb_store, vreg, 0);  // V of tile it + 1
            if (piece == 3) store_v_piece(vb_store, vreg, 1);
            if (piece == 4) {
                const uint32_t row_k = tile_row(it + 4, look);
                const int64_t off_k = load_k(it + 4, row_k, kreg);
                load_v(it + 3, off_v, vreg);
                off_v = off_k;
            }
            if (piece == 5) look = tile_lookup(it + 6);
        };
        if (fused) {
            fused_phase(cur, kb_cur, 1, s1, s0, p_new, vb_prev, 1, p_old,
                        [&](int step) { staging(step - (kPhase - 8)); });
            fused_phase(nxt, kb_next, 0, s0, s1, p_old, vb_cur, 0, p_new, [](int) {});
        } else {
#pragma unroll
            for (int piece = 0; piece < 6; piece++) staging(piece);
            // the same three stages one after the other, each only where it applies
            if (prev_active) accumulate(vb_prev, 1, p_old);
            if (cur.active) {
                scores(kb_cur, 1, s1);
                probabilities(s0, p_new);
                apply_mask(cur, 1, s1);
                accumulate(vb_cur, 0, p_new);
                probabilities(s1, p_old);
            }
            if (nxt.active) {
                scores(kb_next, 0, s0);
                apply_mask(nxt, 0, s0);
            }
        }
        prev_active = cur.active;
        __syncthreads();
        const uint32_t kfreed = kb_cur;
        kb_cur = kb_next;
        kb_next = kb_store;
        kb_store = kfreed;
        const uint32_t vfreed = vb_prev;
        vb_prev = vb_cur;
        vb_cur = vb_store;
        vb_store = vfreed;
    };
    // Always in pairs: past the last tile an iteration only finishes what is pending and
    // stages into buffers nobody reads.  (Leaving the loop between the two makes the
    // compiler wait for the previous iteration's loads before every store.)
    for (uint32_t it = t_begin; it < n_tiles; it += 2) {
        iteration(it, kreg_a, vreg_a, look_a);
        iteration(it + 1, kreg_b, vreg_b, look_b);
    }
    if (prev_active) accumulate(vb_prev, 1, p_old);  // drain: sub-tile 1 of the last tile
    }

    if (!wave_active) return;
    {
        const LanePair both = half_wave_pair(l_run);
        l_run = both.lo + both.hi;
    }
    if (q_row >= p.seq_q) return;
    if (p.n_splits > 1) {
        // partial result of this key range: O unnormalised, (m_ref, l) beside it
        const size_t row = (size_t(split) * p.num_heads + head) * p.seq_q + q_row;
        float* po = p.part_o + row * kD;
#pragma unroll
        for (int t = 0; t < kBlocks; t++)
#pragma unroll
            for (int ah = 0; ah < 2; ah++) {
                float x[8];
#pragma unroll
                for (int e = 0; e < 8; e++) x[e] = oacc[t][8 * ah + e];
                float* op = po + 32 * t + 16 * ah + 8 * g;
                *reinterpret_cast<float4v*>(op) = float4v{x[0], x[1], x[2], x[3]};
                *reinterpret_cast<float4v*>(op + 4) = float4v{x[4], x[5], x[6], x[7]};
            }
        if (g == 0) {
            p.part_ml[row * 2 + 0] = m_ref;
            p.part_ml[row * 2 + 1] = l_run;
        }
        return;
    }
    const float inv_l = 1.0f / l_run;
    const int64_t ooff = int64_t(q_row) * p.out_tok_stride + int64_t(head) * p.out_head_stride;
    // Accumulator [t][4a + b] is A-operand row 8a + 4g + b of block t, which was fed
    // head-dim element 32 t + 16 (a >> 1) + 8 g + 4 (a & 1) + b: 8 consecutive elements
    // per (t, a >> 1).
#pragma unroll
    for (int t = 0; t < kBlocks; t++)
#pragma unroll
        for (int ah = 0; ah < 2; ah++) {
            float x[8];
#pragma unroll
            for (int e = 0; e < 8; e++) x[e] = oacc[t][8 * ah + e] * inv_l;
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
        p.lse[size_t(head) * p.seq_q + q_row] = (m_ref + __builtin_amdgcn_logf(l_run)) * kLn2;
}

// One thread per node: set own bit, then walk parent pointers
// (src/llm/transformer.mm:822-840); at most num_nodes steps.
__global__ void tree_mask_kernel(const int32_t* parents, uint32_t* mask, uint32_t num_nodes,
                                 uint32_t words) {
    const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= num_nodes) return;
    uint32_t* row = mask + size_t(i) * words;
    for (uint32_t w = 0; w < words; w++) row[w] = 0;
    row[i >> 5] |= 1u << (i & 31);
    int32_t cur = parents[i];
    for (uint32_t step = 0; step < num_nodes && cur >= 0 && cur < int32_t(num_nodes); step++) {
        row[uint32_t(cur) >> 5] |= 1u << (uint32_t(cur) & 31);
        cur = parents[cur];
    }
}

// Combines the split-K partials of 16 (head size 64: 32) query rows of one head: one
// thread per (row, 8 consecutive head-dim elements).
template <bool kOutF32, int kD>
__global__ void __launch_bounds__(256) attention_merge_kernel(AttnParams p, uint32_t n_splits) {
    constexpr uint32_t kLanesPerRow = kD / 8, kRowsPerGroup = 256 / kLanesPerRow;
    const uint32_t head = blockIdx.y;
    const uint32_t q_row = blockIdx.x * kRowsPerGroup + threadIdx.x / kLanesPerRow;
    const uint32_t dc = threadIdx.x % kLanesPerRow;
    if (q_row >= p.seq_q) return;
    // One pass, four splits at a time: the loads of a group depend on nothing computed
    // here, so they are in flight together, and the running maximum is folded in as the
    // groups arrive.
    float mx = kNegBig, l = 0.0f;
    float o[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    for (uint32_t s0 = 0; s0 < n_splits; s0 += 4) {
        float m[4], ls[4];
        float4v a[4], b[4];
#pragma unroll
        for (uint32_t i = 0; i < 4; i++) {
            const uint32_t sp = min(s0 + i, n_splits - 1);  // clamped: always a written row
            const size_t row = (size_t(sp) * p.num_heads + head) * p.seq_q + q_row;
            m[i] = p.part_ml[row * 2];
            ls[i] = p.part_ml[row * 2 + 1];
            const float* po = p.part_o + row * kD + 8 * dc;
            a[i] = *reinterpret_cast<const float4v*>(po);
            b[i] = *reinterpret_cast<const float4v*>(po + 4);
        }
        float m_new = mx;
#pragma unroll
        for (uint32_t i = 0; i < 4; i++) m_new = fmaxf(m_new, s0 + i < n_splits ? m[i] : kNegBig);
        const float keep = fast_exp2(mx - m_new);
        l *= keep;
#pragma unroll
        for (int e = 0; e < 8; e++) o[e] *= keep;
#pragma unroll
        for (uint32_t i = 0; i < 4; i++) {
            const float f = s0 + i < n_splits ? fast_exp2(m[i] - m_new) : 0.0f;
            l += ls[i] * f;
            o[0] += a[i].x * f; o[1] += a[i].y * f; o[2] += a[i].z * f; o[3] += a[i].w * f;
            o[4] += b[i].x * f; o[5] += b[i].y * f; o[6] += b[i].z * f; o[7] += b[i].w * f;
        }
        mx = m_new;
    }
    const float inv_l = 1.0f / l;
    const int64_t ooff =
        int64_t(q_row) * p.final_tok_stride + int64_t(head) * p.final_head_stride + 8 * dc;
    if constexpr (kOutF32) {
        float* op = static_cast<float*>(p.final_out) + ooff;
        *reinterpret_cast<float4v*>(op) =
            float4v{o[0] * inv_l, o[1] * inv_l, o[2] * inv_l, o[3] * inv_l};
        *reinterpret_cast<float4v*>(op + 4) =
            float4v{o[4] * inv_l, o[5] * inv_l, o[6] * inv_l, o[7] * inv_l};
    } else {
        uint4v w;
        w.x = pack_f16x2(o[0] * inv_l, o[1] * inv_l);
        w.y = pack_f16x2(o[2] * inv_l, o[3] * inv_l);
        w.z = pack_f16x2(o[4] * inv_l, o[5] * inv_l);
        w.w = pack_f16x2(o[6] * inv_l, o[7] * inv_l);
        *reinterpret_cast<uint4v*>(static_cast<uint16_t*>(p.final_out) + ooff) = w;
    }
    if (p.lse && dc == 0)
        p.lse[size_t(head) * p.seq_q + q_row] = (mx + __builtin_amdgcn_logf(l)) * kLn2;
}

template <bool kQF32, bool kOutF32, int kRows, int kD>
int launch_tiles(const AttnParams& p, dim3 grid) {
    auto kernel = attention_tiles_kernel<kQF32, kOutF32, kRows, kD>;
    constexpr size_t kLdsBytes = Geometry<kD>::kLdsBytes;
    static bool configured[kMaxDevices];  // the tile buffers exceed the 64 KiB default limit
    if (int rc = raise_dynamic_lds_limit(reinterpret_cast<const void*>(kernel), kLdsBytes, configured)) return rc;
    kernel<<<grid, dim3(kThreads), kLdsBytes, ctx().stream>>>(p);
    return launch_status();
}

template <bool kQF32, bool kOutF32, int kD>
int launch_tiles_rows(const AttnParams& p, dim3 grid, int rows) {
    if (rows == kRowsContiguous) return launch_tiles<kQF32, kOutF32, kRowsContiguous, kD>(p, grid);
    if (rows == kRowsPagedPow2) return launch_tiles<kQF32, kOutF32, kRowsPagedPow2, kD>(p, grid);
    return launch_tiles<kQF32, kOutF32, kRowsPagedAny, kD>(p, grid);
}

template <int kD>
int launch_tiles_types(const AttnParams& p, dim3 grid, int rows, bool qf32, bool of32) {
    if (qf32 && of32) return launch_tiles_rows<true, true, kD>(p, grid, rows);
    if (qf32 && !of32) return launch_tiles_rows<true, false, kD>(p, grid, rows);
    if (!qf32 && of32) return launch_tiles_rows<false, true, kD>(p, grid, rows);
    return launch_tiles_rows<false, false, kD>(p, grid, rows);
}

}  // namespace

int launch_tree_mask(const int32_t* parents, uint32_t* mask_words, uint32_t num_nodes) {
    if (!parents || !mask_words) return GRANITE_HIP_ENULL;
    if (num_nodes == 0) return GRANITE_HIP_OK;
    const uint32_t words = (num_nodes + 31) / 32;
    {
        KernelTimerScope timer("tree_mask");
        tree_mask_kernel<<<dim3((num_nodes + 63) / 64), dim3(64), 0, ctx().stream>>>(
            parents, mask_words, num_nodes, words);
    }
    return launch_status();
}

int launch_attention(const granite_hip_attention_args& a, const ScratchSource& scratch) {
    if (!a.q || !a.out) return GRANITE_HIP_ENULL;
    if (a.head_dim != 128 && a.head_dim != 64) return GRANITE_HIP_EUNSUPPORTED;
    const uint32_t D = a.head_dim;
    if (a.num_heads == 0 || a.num_kv_heads == 0 || a.num_heads % a.num_kv_heads != 0)
        return GRANITE_HIP_EINVAL;
    if ((a.q_dtype != GRANITE_HIP_F32 && a.q_dtype != GRANITE_HIP_F16) ||
        (a.out_dtype != GRANITE_HIP_F32 && a.out_dtype != GRANITE_HIP_F16))
        return GRANITE_HIP_EINVAL;
    if (scratch.query) *scratch.query = 0;
    if (a.seq_q == 0) return GRANITE_HIP_OK;
    if (a.cache_len + a.extra_len == 0) return GRANITE_HIP_EINVAL;
    if (a.cache_len > 0 && (!a.k_cache || !a.v_cache)) return GRANITE_HIP_ENULL;
    if (a.extra_len > 0 && (!a.k_extra || !a.v_extra)) return GRANITE_HIP_ENULL;
    if (a.block_table && a.block_size == 0) return GRANITE_HIP_EINVAL;
    if (!a.block_table && a.cache_len > 0 && a.max_seq < a.cache_len) return GRANITE_HIP_EINVAL;
    const size_t qes = a.q_dtype == GRANITE_HIP_F32 ? 4 : 2, oes = a.out_dtype == GRANITE_HIP_F32 ? 4 : 2;
    if ((a.q_tok_stride * qes) % 16 || (a.q_head_stride * qes) % 16 ||
        (reinterpret_cast<uintptr_t>(a.q) & 15) || (a.out_tok_stride * oes) % 16 ||
        (a.out_head_stride * oes) % 16 || (reinterpret_cast<uintptr_t>(a.out) & 15))
        return GRANITE_HIP_EINVAL;

    AttnParams p{};
    p.q = a.q;
    p.out = a.out;
    p.lse = a.lse;
    p.q_tok_stride = a.q_tok_stride;
    p.q_head_stride = a.q_head_stride;
    p.out_tok_stride = a.out_tok_stride;
    p.out_head_stride = a.out_head_stride;
    p.k = static_cast<const uint16_t*>(a.k_cache);
    p.v = static_cast<const uint16_t*>(a.v_cache);
    p.table = a.block_table;
    p.block_size = a.block_table ? a.block_size : 1;
    p.bs_shift = (p.block_size & (p.block_size - 1)) == 0 ? __builtin_ctz(p.block_size) : -1;
    if (a.block_table) {
        p.a_tok_stride = int64_t(a.num_kv_heads) * D;
        p.a_head_stride = D;
    } else {
        p.a_tok_stride = D;
        p.a_head_stride = int64_t(a.max_seq) * D;
    }
    p.cache_len = a.cache_len;
    p.k_extra = static_cast<const uint16_t*>(a.k_extra);
    p.v_extra = static_cast<const uint16_t*>(a.v_extra);
    p.extra_len = a.extra_len;
    p.mask_mode = a.mask_mode;
    p.start_pos = a.start_pos;
    p.seq_q = a.seq_q;
    p.num_heads = a.num_heads;
    p.group = a.num_heads / a.num_kv_heads;
    p.scale_log2 = a.scale * kLog2e;

    if (a.mask_mode == GRANITE_HIP_MASK_CAUSAL) {
        if (a.extra_len != 0) return GRANITE_HIP_EUNSUPPORTED;
    } else if (a.mask_mode == GRANITE_HIP_MASK_TREE) {
        if (!a.parents) return GRANITE_HIP_ENULL;
        if (a.extra_len == 0 || a.seq_q != a.extra_len) return GRANITE_HIP_EINVAL;
        p.mask_words = (a.extra_len + 31) / 32;
    } else if (a.mask_mode != GRANITE_HIP_MASK_NONE) {
        return GRANITE_HIP_EINVAL;
    }

    // Which kernel: the direct-to-LDS one (prefill_dma.hip) where it applies -- head size 128,
    // contiguous rows or blocks of a power of two >= 8 tokens, and no extra key segment other
    // than the tree of a tree-masked launch whose ancestor masks a workgroup builds itself,
    // behind a non-empty cache -- else the register-staged kernel of this file.
    const int rows = !a.block_table ? kRowsContiguous
                                    : (p.bs_shift >= 0 ? kRowsPagedPow2 : kRowsPagedAny);
    const bool tree_dma = a.mask_mode == GRANITE_HIP_MASK_TREE && a.cache_len > 0 && a.extra_len <= kMaxFusedNodes;
    bool dma = D == 128 && rows != kRowsPagedAny && (rows == kRowsContiguous || p.bs_shift >= 3) &&
               (tree_dma || (a.extra_len == 0 && a.mask_mode != GRANITE_HIP_MASK_TREE));
    if (const char* e = std::getenv("GRANITE_HIP_PREFILL_KERNEL")) dma = dma && e[0] != 't';  // "tiles": the register-staged kernel

    // A small tree on that kernel: the query heads of a KV group, side by side.  A tree of 64
    // nodes is two of a workgroup's eight waves; with [heads, nodes, D] dense (one head's rows
    // right behind the previous head's, in Q, in the output and therefore in the partials and
    // the log-sum-exp too) `pack` heads of a group are one head of pack x nodes rows to the
    // kernel, which only has to take a row's node (row mod nodes) for the ancestor mask.  Up to
    // 128 rows, i.e. one wave per SIMD computing and its idle partner staging for it; the
    // workgroups that this saves become key splits, so a workgroup's walk is 1 / pack as long.
    // Behind a long prefix only (8192 tokens and more: 64 nodes over 16 384 tokens 50.7 -> 41.5 us
    // a step): at 4096 tokens the step takes as long either way and the partials double.
    constexpr uint32_t kPackFromTiles = 128;
    uint32_t seq_q = a.seq_q, num_heads = a.num_heads;  // the launch's shape
    if (dma && tree_dma && (a.cache_len + kBN - 1) / kBN >= kPackFromTiles &&
        a.q_head_stride == int64_t(a.seq_q) * a.q_tok_stride &&
        a.out_head_stride == int64_t(a.seq_q) * a.out_tok_stride) {
        uint32_t pack = 1;
        while (2 * pack * a.seq_q <= uint32_t(kBM / 2) && p.group % (2 * pack) == 0) pack *= 2;
        seq_q = pack * a.seq_q;
        num_heads = a.num_heads / pack;
        p.seq_q = seq_q;
        p.num_heads = num_heads;
        p.group = p.group / pack;
        p.q_head_stride *= pack;
        p.out_head_stride *= pack;
    }

    const uint32_t q_tiles = (seq_q + kBM - 1) / kBM;
    if (q_tiles > 0x7FFFFFFFu / 2 || a.num_heads > 65535u) return GRANITE_HIP_EINVAL;

    // Split the keys over several workgroups when (query tiles x heads) alone cannot
    // put a workgroup on every CU; every split keeps at least 4 key tiles.
    uint32_t n_splits = 1;
    {
        const uint32_t cus = ctx().compute_units > 0 ? uint32_t(ctx().compute_units) : 256u;
        const uint64_t wgs = uint64_t(q_tiles) * num_heads;
        const uint32_t key_tiles = (a.cache_len + kBN - 1) / kBN + (a.extra_len + kBN - 1) / kBN;
        if (wgs < cus) {
            n_splits = uint32_t((cus + wgs - 1) / wgs);
            n_splits = min(n_splits, max(key_tiles / 4, 1u));
            n_splits = min(n_splits, 64u);
        }
        if (const char* e = std::getenv("GRANITE_HIP_ATTN_SPLITS")) n_splits = max(1, std::atoi(e));
    }
    // One scratch request for everything (growing the scratch buffer moves it): the
    // tree mask first, the split-K partials behind it.
    const bool tree = a.mask_mode == GRANITE_HIP_MASK_TREE && a.extra_len > kMaxFusedNodes;
    if (a.mask_mode == GRANITE_HIP_MASK_TREE && !tree) p.tree_parents = a.parents;
    const size_t mask_bytes =
        tree ? (size_t(a.extra_len) * p.mask_words * sizeof(uint32_t) + 255) & ~size_t(255) : 0;
    const size_t rows_total = n_splits > 1 ? size_t(n_splits) * num_heads * seq_q : 0;
    const size_t need = mask_bytes + rows_total * (D + 2) * sizeof(float);
    if (scratch.query) {
        *scratch.query = need;
        return GRANITE_HIP_OK;
    }
    if (need > 0) {
        void* ws_ptr = nullptr;
        int rc = take_scratch(scratch, need, &ws_ptr);
        if (rc != GRANITE_HIP_OK) return rc;
        char* ws = static_cast<char*>(ws_ptr);
        if (tree) {
            uint32_t* mask = reinterpret_cast<uint32_t*>(ws);
            rc = launch_tree_mask(a.parents, mask, a.extra_len);
            if (rc != GRANITE_HIP_OK) return rc;
            p.tree_mask = mask;
        }
        if (n_splits > 1) {
            p.part_o = reinterpret_cast<float*>(ws + mask_bytes);
            p.part_ml = p.part_o + rows_total * D;
            p.final_out = a.out;
            p.final_tok_stride = p.out_tok_stride;
            p.final_head_stride = p.out_head_stride;
        }
    }
    p.q_tiles = q_tiles;
    p.n_splits = n_splits;
    if (uint64_t(q_tiles) * num_heads * n_splits > 0x7FFFFFFFull) return GRANITE_HIP_EINVAL;
    dim3 grid(q_tiles * num_heads * n_splits);
    const bool qf32 = a.q_dtype == GRANITE_HIP_F32, of32 = a.out_dtype == GRANITE_HIP_F32;
    int rc;
    {
        KernelTimerScope timer("attention_tiles");
        if (dma) rc = launch_tiles_dma(p, grid, qf32, of32);
        else rc = D == 128 ? launch_tiles_types<128>(p, grid, rows, qf32, of32)
                           : launch_tiles_types<64>(p, grid, rows, qf32, of32);
    }
    if (rc != GRANITE_HIP_OK || n_splits == 1) return rc;
    {
        KernelTimerScope timer("attention_merge");
        const uint32_t rows_per_group = 256 / (D / 8);
        dim3 mgrid((seq_q + rows_per_group - 1) / rows_per_group, num_heads);
        hipStream_t st = ctx().stream;
        if (D == 128) {
            if (of32) attention_merge_kernel<true, 128><<<mgrid, dim3(256), 0, st>>>(p, n_splits);
            else attention_merge_kernel<false, 128><<<mgrid, dim3(256), 0, st>>>(p, n_splits);
        } else {
            if (of32) attention_merge_kernel<true, 64><<<mgrid, dim3(256), 0, st>>>(p, n_splits);
            else attention_merge_kernel<false, 64><<<mgrid, dim3(256), 0, st>>>(p, n_splits);
        }
    }
    return launch_status();
}

}  // namespace ghip
