// Persistent ("stream") form of the decode attention kernel.
//
// The context of every sequence is cut into 32-token tiles; all tiles of the
// batch form one flat list that is cut into equal contiguous ranges, one per
// worker, and the grid is one workgroup per compute unit (one wave per SIMD),
// so every wave streams the same number of K/V bytes and there is no per-chunk
// workgroup start-up.  (Two workgroups per CU measured slower: the older one
// wins the memory pipeline and the younger finishes 25 % later.)
//
// Two shapes of the list:
//   * rows ("kPair"), when the number of heads is a multiple of 8: the list is
//     ordered (sequence, group of 8 heads, tile) and a worker is a workgroup.
//     Its four waves walk the same tiles, each for two heads that it alternates
//     between, so a workgroup reads whole token rows (all heads of a token are
//     contiguous in the pool) at about the same time.  Which memory channels a
//     workgroup loads then does not depend on how the sequence lengths fall:
//     with one head per wave, a batch of mixed lengths ran 11 % slower than one
//     of equal lengths, and the waves' run times spread by +-15 %.
//   * flat, otherwise: the list is ordered (sequence, head, tile) and a worker
//     is a wave.
// A worker that crosses from one (sequence, head) to the next writes a partial
// (m, l, O) for the part it covered; the merge kernel combines the partials of
// a (sequence, head), whose positions follow from the same arithmetic.
//
// Partials are stored compactly.  Walking the flat list, a new piece (one worker's
// part of one (sequence, list head) segment) begins at every worker boundary and at
// every segment boundary, so the pieces are numbered without collision by
// worker + segment, segment = sequence * lists + list head: from one piece to the
// next the worker or the segment grows, and neither ever shrinks.  There are
// therefore workers + batch * lists piece slots however long the sequences may
// become, each holding the query heads of one list head.
//
// There is no separate planning launch: every workgroup scans the sequence
// lengths into tile counts and their prefix sums itself, in LDS (a few hundred
// nanoseconds for a batch of 64), and looks everything up there afterwards, so
// that none of the bookkeeping ever waits on global memory.  Workgroup 0 also
// stores the prefix sums and the per-worker share for the merge kernel.
//
// Inside a wave the pipeline is three tiles deep: the block-table rows of tile
// i+2 and the K/V rows of tile i+1 are in flight while tile i goes through the
// MFMAs (two register buffers, no LDS, no barriers).  The per-tile math and
// operand layouts are those of decode.hip.
#include <cstdlib>

#include "common.h"
#include "decode_common.h"

namespace ghip {
namespace {

// One entry of the flat list: a 32-token tile of one (sequence, list head).  A list
// head is a virtual head (kv_head * q_groups + q_group) or, in the rows shape, a group
// of 8 consecutive virtual heads.
struct Cursor {
    uint32_t b;    // sequence
    uint32_t vh;   // list head
    uint32_t t;    // tile inside the sequence
    uint32_t nt;   // tiles of sequence b
    uint32_t len;  // tokens of sequence b
};

__device__ __forceinline__ uint32_t seq_len_of(const DecodeParams& p, uint32_t b) {
    uint32_t len = p.seq_lens ? uint32_t(max(p.seq_lens[b], 0)) : p.max_tokens;
    return min(len, p.max_tokens);
}

// Next tile in (sequence, list head, tile) order (`lists` list heads); skips empty sequences.  `more`
// false leaves the cursor where it is (the caller re-reads the last tile
// instead of running off the end, so no load ever sits inside a branch).
// `lens` holds the token count of every sequence, in LDS.
__device__ __forceinline__ void advance(const DecodeParams& p, const uint32_t* lens, uint32_t lists,
                                        Cursor& c, bool more) {
    if (!more) return;
    if (++c.t < c.nt) return;
    c.t = 0;
    if (++c.vh < lists) return;
    c.vh = 0;
    do {
        ++c.b;
        c.len = c.b < p.batch ? uint32_t(__builtin_amdgcn_readfirstlane(int(lens[c.b]))) : kTile;
        c.nt = (c.len + kTile - 1) / kTile;
    } while (c.nt == 0 && c.b < p.batch);
    if (c.b >= p.batch) c.b = p.batch - 1;  // never dereferenced past the end
}

// Heads of one list entry in the rows shape: two per wave.
constexpr uint32_t kPairHeads = 2 * kWavesPerWG;

// First query head of list head `lh`: a list head is one virtual head
// (kv_head * q_groups + q_group, up to 16 query heads) or, in the rows shape, 8
// consecutive ones; the query heads of consecutive virtual heads are consecutive.
__device__ __forceinline__ uint32_t list_first_head(const DecodeParams& p, uint32_t lh, bool pair) {
    const uint32_t v0 = pair ? lh * kPairHeads : lh;
    return (v0 / p.q_groups) * p.group + (v0 % p.q_groups) * 16;
}

template <int kD>
struct TileRegs {
    half8 ka[2][kD / 32];
    uint4v vr[8];
};

// kD: head size, 128 or 64 (at 64 lanes 8..15 of a group repeat the V loads of lanes 0..7
// and the output rows they stand for are dropped, as in the chunk kernel).
template <bool kQF32, int kRows, bool kPair, int kD>
__global__ void __launch_bounds__(kWavesPerWG* kWave, 1) decode_stream_kernel(DecodeParams p) {
    constexpr int kKSteps = kD / 32;
    const uint32_t lane = threadIdx.x & 63;
    const uint32_t wave = threadIdx.x >> 6;
    const uint32_t n = lane & 15;
    const uint32_t g = lane >> 4;
    // wave-uniform by construction; saying so keeps every cursor in scalar registers
    const uint32_t worker = uint32_t(
        __builtin_amdgcn_readfirstlane(int(kPair ? blockIdx.x : blockIdx.x * kWavesPerWG + wave)));

    // ---- tile counts and their prefix sums, in LDS
    extern __shared__ uint32_t s_dyn[];
    uint32_t* s_prefix = s_dyn;             // [batch + 1]: tiles of the sequences before b
    uint32_t* s_len = s_dyn + p.batch + 1;  // [batch]: tokens of sequence b
    __shared__ uint32_t s_wave_sum[kWavesPerWG];
    const uint32_t vheads = p.num_kv_heads * p.q_groups;
    uint32_t tiles_total;
    {
        // every thread sums a run of consecutive sequences, the runs are scanned
        const uint32_t run = (p.batch + blockDim.x - 1) / blockDim.x;
        const uint32_t b0 = threadIdx.x * run;
        uint32_t mine = 0;
        for (uint32_t b = b0; b < min(b0 + run, p.batch); b++) {
            const uint32_t len = seq_len_of(p, b);
            s_len[b] = len;
            mine += (len + kTile - 1) / kTile;
        }
        uint32_t incl = mine;  // inclusive scan inside the wave
#pragma unroll
        for (uint32_t off = 1; off < kWave; off <<= 1) {
            const uint32_t up = lane_read(incl, lane >= off ? lane - off : lane);
            if (lane >= off) incl += up;
        }
        if (lane == kWave - 1) s_wave_sum[wave] = incl;
        __syncthreads();
        uint32_t before = 0, all = 0;
#pragma unroll
        for (uint32_t w = 0; w < kWavesPerWG; w++) {
            const uint32_t v = s_wave_sum[w];
            if (w < wave) before += v;
            all += v;
        }
        uint32_t at = before + incl - mine;
        for (uint32_t b = b0; b < min(b0 + run, p.batch); b++) {
            s_prefix[b] = at;
            at += (s_len[b] + kTile - 1) / kTile;
        }
        tiles_total = uint32_t(__builtin_amdgcn_readfirstlane(int(all)));
        if (threadIdx.x == 0) s_prefix[p.batch] = tiles_total;
        __syncthreads();
    }
    const uint32_t lists = kPair ? vheads / kPairHeads : vheads;  // list heads
    const uint32_t total = tiles_total * lists;
    const uint32_t per = max((total + p.workers - 1) / p.workers, p.min_per);
    if (blockIdx.x == 0) {  // for the merge kernel
        for (uint32_t i = threadIdx.x; i <= p.batch; i += blockDim.x) p.plan[kPlanHeader + i] = s_prefix[i];
        if (threadIdx.x == 0) {
            p.plan[0] = per;
            p.plan[1] = total;
            p.plan[2] = kPair ? kPairHeads : 1;
        }
    }
    auto prefix_u = [&](uint32_t i) -> uint32_t {  // wave-uniform index: stays in a scalar register
        return uint32_t(__builtin_amdgcn_readfirstlane(int(s_prefix[i])));
    };

    // ---- this worker's range of the flat tile list
    const uint32_t u0 = worker * per;
    if (u0 >= total) return;
    const uint32_t n_units = min(per, total - u0);

    // locate u0: largest b with prefix[b] * lists <= u0
    Cursor first;
    {
        uint32_t lo = 0, hi = p.batch;  // invariant: prefix[lo]*vheads <= u0 < prefix[hi]*vheads
        while (hi - lo > 1) {
            const uint32_t mid = (lo + hi) >> 1;
            if (prefix_u(mid) * lists <= u0) lo = mid; else hi = mid;
        }
        first.b = lo;
        first.nt = prefix_u(lo + 1) - prefix_u(lo);
        first.len = uint32_t(__builtin_amdgcn_readfirstlane(int(s_len[lo])));
        const uint32_t in_seq = u0 - prefix_u(lo) * lists;
        first.vh = in_seq / first.nt;
        first.t = in_seq - first.vh * first.nt;
    }

    auto rows_of = [&](const Cursor& c) -> uint32_t {
        const int32_t* table =
            kRows != kRowsContiguous ? p.tables + size_t(c.b) * p.max_blocks : nullptr;
        return tile_row<kRows>(p, table, c.t * kTile, lane, c.len);
    };
    // Virtual head a cursor stands for: in the rows shape, the wave's first (side 0) or
    // second (side 1) head of the cursor's group.
    auto head_of = [&](const Cursor& c, uint32_t side) -> uint32_t {
        return kPair ? c.vh * kPairHeads + 2 * wave + side : c.vh;
    };
    auto issue = [&](TileRegs<kD>& r, uint32_t rows, uint32_t vh) {
        const uint32_t kvh = vh / p.q_groups;
        const uint16_t* kbase = p.k + size_t(kvh) * p.head_stride + 8 * g;
        const uint16_t* vbase = p.v + size_t(kvh) * p.head_stride + 8 * (n & (kD / 8 - 1));
#pragma unroll
        for (int sub = 0; sub < 2; sub++) {
            const uint32_t row = lane_read(rows, 16 * sub + n);
            const uint16_t* kp = kbase + size_t(row) * p.tok_stride;
#pragma unroll
            for (int s = 0; s < kKSteps; s++)
                r.ka[sub][s] = as_half8(*reinterpret_cast<const uint4v*>(kp + 32 * s));
        }
#pragma unroll
        for (int j = 0; j < 8; j++) {
            const uint32_t row = lane_read(rows, tau(g, j));
            // every byte of V is used once: a streaming load measured 9 % faster (for K,
            // whose lines are covered by four instructions, it made no difference)
            r.vr[j] = __builtin_nontemporal_load(
                reinterpret_cast<const uint4v*>(vbase + size_t(row) * p.tok_stride));
        }
    };

    // Running state of one (sequence, virtual head): Q as B operands (with fp32 Q, an fp16
    // head and an fp16 remainder), the maximum, the sum and O.
    struct HeadState {
        half8 bq[kKSteps];
        half8 bq_lo[kQF32 ? kKSteps : 1];
        float m_run, l_run;
        float4v acc[8];
    };
    auto clear = [&](HeadState& h) {
        h.m_run = kNegBig;
        h.l_run = 0.0f;
#pragma unroll
        for (int t = 0; t < 8; t++) h.acc[t] = float4v{0, 0, 0, 0};
    };
    auto load_q = [&](uint32_t b, uint32_t vh, HeadState& h) {
        const uint32_t kvh = vh / p.q_groups, qg = vh % p.q_groups;
        const uint32_t q_in_group = qg * 16 + n;
        const bool q_valid = q_in_group < p.group;
        const uint32_t qh = kvh * p.group + (q_valid ? q_in_group : 0);
        const size_t off = (size_t(b) * p.num_heads + qh) * kD + 8 * g;
#pragma unroll
        for (int s = 0; s < kKSteps; s++) {
            if constexpr (kQF32) {
                const float* qp = static_cast<const float*>(p.q) + off + 32 * s;
                float4v x0 = *reinterpret_cast<const float4v*>(qp);
                float4v x1 = *reinterpret_cast<const float4v*>(qp + 4);
                float x[8] = {x0.x, x0.y, x0.z, x0.w, x1.x, x1.y, x1.z, x1.w};
                half8 hi, lo;
#pragma unroll
                for (int i = 0; i < 8; i++) {
                    const float xv = q_valid ? x[i] : 0.0f;
                    _Float16 hv = static_cast<_Float16>(xv);
                    hi[i] = hv;
                    lo[i] = static_cast<_Float16>(xv - static_cast<float>(hv));
                }
                h.bq[s] = hi;
                h.bq_lo[s] = lo;
            } else {
                uint4v w = *reinterpret_cast<const uint4v*>(static_cast<const uint16_t*>(p.q) +
                                                            off + 32 * s);
                if (!q_valid) w = uint4v{0, 0, 0, 0};
                h.bq[s] = as_half8(w);
            }
        }
    };

    auto compute = [&](const TileRegs<kD>& r, const Cursor& c, HeadState& h) {
        const uint32_t tok0 = c.t * kTile;
        float4v c0 = {0, 0, 0, 0}, c1 = {0, 0, 0, 0};
#pragma unroll
        for (int s = 0; s < kKSteps; s++) {
            c0 = __builtin_amdgcn_mfma_f32_16x16x32_f16(r.ka[0][s], h.bq[s], c0, 0, 0, 0);
            c1 = __builtin_amdgcn_mfma_f32_16x16x32_f16(r.ka[1][s], h.bq[s], c1, 0, 0, 0);
            if constexpr (kQF32) {
                c0 = __builtin_amdgcn_mfma_f32_16x16x32_f16(r.ka[0][s], h.bq_lo[s], c0, 0, 0, 0);
                c1 = __builtin_amdgcn_mfma_f32_16x16x32_f16(r.ka[1][s], h.bq_lo[s], c1, 0, 0, 0);
            }
        }
        float s[8];
#pragma unroll
        for (int i = 0; i < 4; i++) {
            s[i] = c0[i] * p.scale_log2;
            s[4 + i] = c1[i] * p.scale_log2;
        }
        if (tok0 + kTile > c.len) {  // ragged last tile of a sequence
#pragma unroll
            for (int i = 0; i < 4; i++) {
                if (tok0 + 4 * g + i >= c.len) s[i] = -INFINITY;
                if (tok0 + 16 + 4 * g + i >= c.len) s[4 + i] = -INFINITY;
            }
        }
        float mloc = fmaxf(fmaxf(fmaxf(s[0], s[1]), fmaxf(s[2], s[3])),
                           fmaxf(fmaxf(s[4], s[5]), fmaxf(s[6], s[7])));
        mloc = fmaxf(mloc, wave_shfl_xor(mloc, 16));
        mloc = fmaxf(mloc, wave_shfl_xor(mloc, 32));
        const float m_new = fmaxf(h.m_run, mloc);
        const float alpha = fast_exp2(h.m_run - m_new);
        h.m_run = m_new;
        float psum = 0.0f, pj[8];
#pragma unroll
        for (int j = 0; j < 8; j++) {
            pj[j] = fast_exp2(s[j] - m_new);
            psum += pj[j];
        }
        h.l_run = h.l_run * alpha + psum;
        uint4v bpw;
        bpw.x = pack_f16x2(pj[0], pj[1]);
        bpw.y = pack_f16x2(pj[2], pj[3]);
        bpw.z = pack_f16x2(pj[4], pj[5]);
        bpw.w = pack_f16x2(pj[6], pj[7]);
        const half8 bp = as_half8(bpw);
#pragma unroll
        for (int t = 0; t < 8; t++) {
            const uint32_t sel = (t & 1) ? 0x07060302u : 0x05040100u;
            uint4v aw;
            aw.x = __builtin_amdgcn_perm(r.vr[1][t >> 1], r.vr[0][t >> 1], sel);
            aw.y = __builtin_amdgcn_perm(r.vr[3][t >> 1], r.vr[2][t >> 1], sel);
            aw.z = __builtin_amdgcn_perm(r.vr[5][t >> 1], r.vr[4][t >> 1], sel);
            aw.w = __builtin_amdgcn_perm(r.vr[7][t >> 1], r.vr[6][t >> 1], sel);
            float4v cin = h.acc[t] * alpha;
            h.acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(as_half8(aw), bp, cin, 0, 0, 0);
        }
    };

    // Writes the partial of virtual head `vh` for the (sequence, list head) the cursor is
    // in and clears the state.
    auto flush = [&](const Cursor& c, uint32_t vh, HeadState& h) {
        float l = h.l_run;
        l += wave_shfl_xor(l, 16);
        l += wave_shfl_xor(l, 32);
        const uint32_t kvh = vh / p.q_groups, qg = vh % p.q_groups;
        const uint32_t q_in_group = qg * 16 + n;
        if (q_in_group < p.group && 32 * g < uint32_t(kD)) {  // (lanes whose rows d = 32 g + .. exist)
            // piece slot = worker + segment; inside it, the query head counted from the
            // first one of the list head
            const uint32_t piece = worker + c.b * lists + c.vh;
            const uint32_t local = kvh * p.group + q_in_group - list_first_head(p, c.vh, kPair);
            const size_t at = size_t(piece) * p.part_cap + local;
            float* po = p.part_o + at * kD + 32 * g;
#pragma unroll
            for (int i = 0; i < 8; i++) {
                float4v w;
#pragma unroll
                for (int k = 0; k < 4; k++) {
                    const int e = 4 * i + k;  // d = 32g + e  <->  acc[e % 8][e / 8]
                    w[k] = h.acc[e & 7][e >> 3];
                }
                *reinterpret_cast<float4v*>(po + 4 * i) = w;
            }
            if (g == 0) {
                p.part_ml[at * 2 + 0] = h.m_run;
                p.part_ml[at * 2 + 1] = l;
            }
        }
        clear(h);
    };

    // ---- three-stage pipeline over the worker's tiles
    Cursor cc = first;  // tile being computed
    Cursor cl = first;  // tile whose K/V rows are requested next
    Cursor cr = first;  // tile whose block-table rows are requested next
    TileRegs<kD> ra, rb;

    if constexpr (kPair) {
        // Buffer A always holds the wave's first head of a tile, buffer B its second; both
        // use the same rows, so there is one block-table lookup per tile.
        HeadState ha, hb;
        clear(ha);
        clear(hb);
        uint32_t rows_t = rows_of(cr);  // of the tile whose K/V is requested next
        advance(p, s_len, lists, cr, 1 < n_units);
        uint32_t rows_n = rows_of(cr);  // of the tile after it
        advance(p, s_len, lists, cr, 2 < n_units);
        issue(ra, rows_t, head_of(cl, 0));
        load_q(cc.b, head_of(cc, 0), ha);
        load_q(cc.b, head_of(cc, 1), hb);

        for (uint32_t i = 0; i < n_units; i++) {
            issue(rb, rows_t, head_of(cl, 1));
            advance(p, s_len, lists, cl, i + 1 < n_units);
            compute(ra, cc, ha);

            rows_t = rows_n;
            rows_n = rows_of(cr);
            advance(p, s_len, lists, cr, i + 3 < n_units);
            issue(ra, rows_t, head_of(cl, 0));  // tile i + 1 (tile i again at the very end)
            compute(rb, cc, hb);

            const bool last = i + 1 >= n_units;
            const bool seg_end = last || cc.t + 1 == cc.nt;
            const Cursor done = cc;
            advance(p, s_len, lists, cc, !last);
            if (seg_end) {
                flush(done, head_of(done, 0), ha);
                flush(done, head_of(done, 1), hb);
                if (!last) {
                    load_q(cc.b, head_of(cc, 0), ha);
                    load_q(cc.b, head_of(cc, 1), hb);
                }
            }
        }
    } else {
        HeadState h;
        clear(h);
        uint32_t rows_a = rows_of(cr);
        advance(p, s_len, lists, cr, 1 < n_units);
        uint32_t rows_b = rows_of(cr);
        advance(p, s_len, lists, cr, 2 < n_units);
        issue(ra, rows_a, cl.vh);
        advance(p, s_len, lists, cl, 1 < n_units);
        load_q(cc.b, cc.vh, h);

        for (uint32_t i = 0; i < n_units; i += 2) {
            // tile i+1 (or tile i again at the very end) into buffer B
            issue(rb, rows_b, cl.vh);
            advance(p, s_len, lists, cl, i + 2 < n_units);
            rows_a = rows_of(cr);
            advance(p, s_len, lists, cr, i + 3 < n_units);

            compute(ra, cc, h);
            {
                const bool last = i + 1 >= n_units;
                const bool seg_end = last || cc.t + 1 == cc.nt;
                const Cursor done = cc;
                advance(p, s_len, lists, cc, !last);
                if (seg_end) {
                    flush(done, done.vh, h);
                    if (!last) load_q(cc.b, cc.vh, h);
                }
                if (last) break;
            }

            issue(ra, rows_a, cl.vh);
            advance(p, s_len, lists, cl, i + 3 < n_units);
            rows_b = rows_of(cr);
            advance(p, s_len, lists, cr, i + 4 < n_units);

            compute(rb, cc, h);
            {
                const bool last = i + 2 >= n_units;
                const bool seg_end = last || cc.t + 1 == cc.nt;
                const Cursor done = cc;
                advance(p, s_len, lists, cc, !last);
                if (seg_end) {
                    flush(done, done.vh, h);
                    if (!last) load_q(cc.b, cc.vh, h);
                }
            }
        }
    }
}

// Merges the partials of one (sequence, query head): the workers that touched
// its list head are consecutive, first = u_start / per, last = (u_end - 1) / per.
__global__ void __launch_bounds__(kHeadDim) decode_stream_merge_kernel(DecodeParams p) {  // head_dim threads
    const uint32_t qh = blockIdx.x;
    const uint32_t b = blockIdx.y;
    const uint32_t* prefix = p.plan + kPlanHeader;
    const uint32_t nt = prefix[b + 1] - prefix[b];
    if (nt == 0) return;  // empty sequence: output untouched
    const uint32_t per = p.plan[0];
    const uint32_t vheads = p.num_kv_heads * p.q_groups;
    const uint32_t kvh = qh / p.group, qg = (qh % p.group) / 16;
    const uint32_t heads_per_list = p.plan[2];  // 1 (flat list) or 8 (rows)
    const uint32_t lists = vheads / heads_per_list;
    const uint32_t vh = (kvh * p.q_groups + qg) / heads_per_list;
    const uint32_t u_start = prefix[b] * lists + vh * nt;
    const uint32_t first_worker = u_start / per;
    const uint32_t n_parts = (u_start + nt - 1) / per - first_worker + 1;
    const size_t head = size_t(b) * p.num_heads + qh;
    // piece c of this segment sits in slot first_worker + c + segment (see the stream kernel)
    const size_t at0 = size_t(first_worker + b * lists + vh) * p.part_cap +
                       (qh - list_first_head(p, vh, heads_per_list > 1));
    const float* ml = p.part_ml + at0 * 2;
    const uint32_t D = p.head_dim;
    const float* po = p.part_o + at0 * D;
    const size_t step = p.part_cap;  // slots of consecutive pieces are part_cap heads apart
    const uint32_t d = threadIdx.x;

    // One pass, four pieces at a time: the loads of a group do not depend on anything
    // computed here, so they are all in flight together (two dependent rounds of memory
    // latency in all: the plan, then the pieces), and the running maximum is folded in
    // as the groups arrive.
    float mx = kNegBig, o = 0.0f, l = 0.0f;
    for (uint32_t c0 = 0; c0 < n_parts; c0 += 4) {
        float m[4], ls[4], os[4];
#pragma unroll
        for (uint32_t i = 0; i < 4; i++) {
            const size_t c = min(c0 + i, n_parts - 1);  // clamped: always a written slot
            m[i] = ml[2 * c * step];
            ls[i] = ml[2 * c * step + 1];
            os[i] = po[c * step * D + d];
        }
        float m_new = mx;
#pragma unroll
        for (uint32_t i = 0; i < 4; i++) m_new = fmaxf(m_new, c0 + i < n_parts ? m[i] : kNegBig);
        const float keep = fast_exp2(mx - m_new);
        o *= keep;
        l *= keep;
#pragma unroll
        for (uint32_t i = 0; i < 4; i++) {
            const float f = c0 + i < n_parts ? fast_exp2(m[i] - m_new) : 0.0f;
            l += ls[i] * f;
            o += os[i] * f;
        }
        mx = m_new;
    }
    p.out[head * D + d] = o / l;
    if (p.lse && d == 0) p.lse[head] = (mx + __builtin_amdgcn_logf(l)) * kLn2;
}

}  // namespace

bool decode_stream_supports(uint32_t batch) { return batch + 1 <= kStreamMaxPrefix; }

int launch_decode_stream(DecodeParams p, bool q_f32, int rows, const ScratchSource& scratch) {
    if (!decode_stream_supports(p.batch)) return GRANITE_HIP_EINVAL;
    // One workgroup per CU, one wave per SIMD.  A worker is a workgroup when the heads come
    // in groups of 8 (the rows shape), else a wave.
    const uint32_t cus = ctx().compute_units > 0 ? uint32_t(ctx().compute_units) : 256u;
    const uint32_t wgs = cus;
    const uint32_t vheads = p.num_kv_heads * p.q_groups;
    const bool pair = vheads % kPairHeads == 0;
    const uint32_t workers = pair ? wgs : wgs * kWavesPerWG;
    // Smallest range a worker may get: it keeps a short batch from being cut into ranges
    // of a tile or two, and is never above chunk_tokens.
    const uint32_t max_tiles = (p.max_tokens + kTile - 1) / kTile;
    const uint32_t min_per = min(max(p.chunk_tokens / kTile, 1u), max((max_tiles + 31) / 32, 1u));

    // Partial results: one slot per piece (worker + segment), each with room for the query
    // heads of a list head.
    const uint32_t lists = pair ? vheads / kPairHeads : vheads;
    p.part_cap = (pair ? kPairHeads : 1u) * min(p.group, 16u);
    const size_t slots = (size_t(workers) + size_t(p.batch) * lists) * p.part_cap;
    const size_t plan_words = kPlanHeader + size_t(p.batch) + 1;
    const size_t plan_bytes = (plan_words * sizeof(uint32_t) + 255) & ~size_t(255);
    const size_t need = plan_bytes + slots * (p.head_dim + 2) * sizeof(float);
    void* ws_ptr = nullptr;
    int rc = take_scratch(scratch, need, &ws_ptr);
    if (rc != GRANITE_HIP_OK || scratch.query) return rc;
    char* ws = static_cast<char*>(ws_ptr);
    p.plan = reinterpret_cast<uint32_t*>(ws);
    p.part_o = reinterpret_cast<float*>(ws + plan_bytes);
    p.part_ml = p.part_o + slots * p.head_dim;

    p.workers = workers;
    p.min_per = min_per;
    const size_t lds_bytes = (2 * size_t(p.batch) + 1) * sizeof(uint32_t);

    hipStream_t st = ctx().stream;
    {
        KernelTimerScope timer("decode_stream");
        dim3 grid(wgs), block(kWavesPerWG * kWave);
        const bool d128 = p.head_dim == 128;
#define GHIP_STREAM_CASE(QF32, ROWS)                                                       \
    if (q_f32 == QF32 && rows == ROWS) {                                                   \
        if (pair && d128)                                                                  \
            decode_stream_kernel<QF32, ROWS, true, 128><<<grid, block, lds_bytes, st>>>(p);  \
        else if (pair)                                                                     \
            decode_stream_kernel<QF32, ROWS, true, 64><<<grid, block, lds_bytes, st>>>(p);   \
        else if (d128)                                                                     \
            decode_stream_kernel<QF32, ROWS, false, 128><<<grid, block, lds_bytes, st>>>(p); \
        else                                                                               \
            decode_stream_kernel<QF32, ROWS, false, 64><<<grid, block, lds_bytes, st>>>(p);  \
    }
        GHIP_STREAM_CASE(true, kRowsContiguous)
        GHIP_STREAM_CASE(true, kRowsPagedPow2)
        GHIP_STREAM_CASE(true, kRowsPagedAny)
        GHIP_STREAM_CASE(false, kRowsContiguous)
        GHIP_STREAM_CASE(false, kRowsPagedPow2)
        GHIP_STREAM_CASE(false, kRowsPagedAny)
#undef GHIP_STREAM_CASE
    }
    rc = launch_status();
    if (rc != GRANITE_HIP_OK) return rc;
    {
        KernelTimerScope timer("decode_merge");
        decode_stream_merge_kernel<<<dim3(p.num_heads, p.batch), dim3(p.head_dim), 0, st>>>(p);
    }
    return launch_status();
}

}  // namespace ghip
