// Paged / contiguous KV decode attention for gfx950: split-K over the context,
// MFMA tiles fed straight from global memory, log-sum-exp merge.
//
// Stands in for the reference decode kernels
//   flash_attention_decode_d128            metal_shaders_attention.h:2982-3177
//   paged_flash_attention_decode_d128      metal_shaders_attention.h:3660-3847
//   batched_paged_attention_decode         metal_shaders_attention.h:2186-2304
// with the arithmetic of the CPU path (src/llm/transformer.mm:1779-1840): fp32
// scores, softmax without epsilon, GQA head h reads KV head h / G.
//
// Work split.  grid = (chunks, kv_heads * q_groups, sequences).  A workgroup
// of 4 waves owns one (sequence, KV head, chunk of `chunk_tokens` tokens) and
// all G query heads of that KV head, so every K/V byte is fetched once.  Each
// wave walks 32-token tiles of the chunk (tile index = wave, wave+4, ...):
//
//   S^T[tok, q]  = K[tok, :] . Q[q, :]        8 x v_mfma_f32_16x16x32_f16
//   online softmax in the MFMA result layout  (a lane owns ONE query head and
//                                              8 tokens: no cross-lane traffic
//                                              except two shuffles for the max)
//   O^T[d, q]   += V^T[d, tok] . P^T[tok, q]  8 x v_mfma_f32_16x16x32_f16
//
// Operand layouts are chosen so that nothing goes through LDS:
//   * K rows are the MFMA A operand as they lie in memory: lane (m = lane%16,
//     g = lane/16) loads 16 bytes of token m at d = 32*step + 8*g.
//   * the token order inside the PV contraction is permuted (tau below) so the
//     probabilities a lane holds after the first MFMA are exactly the B
//     operand of the second;
//   * V rows are loaded 16 bytes per lane (token tau(g, j), d = 8m..8m+7) and
//     turned into the A operand by an 8x8 in-register transpose made of
//     v_perm_b32; output row m of d-tile t stands for d = 8m + t, which makes
//     each lane end up with 32 consecutive output floats.
// The four waves' (m, l, O) are merged through LDS, written as one partial per
// (sequence, query head, chunk), and a second kernel merges the chunks.
//
// Algorithmic HBM bytes per token of context: 2 (K,V) * num_kv_heads * 128 * 2.
#include <cstdlib>
#include <string>

#include "common.h"
#include "decode_common.h"

namespace ghip {
namespace {

// kD is the head size: 128, or 64 (the reference's d64 decode kernels,
// metal_shaders_attention.h:2769-2977, 3202-3422).  At 64 a K row gives two MFMA steps
// instead of four, and only rows 0..7 of the V^T operand (d = 8 m + t < 64) are real: lanes
// 8..15 of a group repeat the loads of lanes 0..7 and their output rows are dropped.
template <bool kQF32, int kRows, int kD>
__global__ void __launch_bounds__(kWavesPerWG * kWave, 2) decode_splitk_kernel(DecodeParams p) {
    constexpr int kKSteps = kD / 32;
    // Workgroups go to the 8 XCDs round-robin by linear id, and only the first
    // n_chunks of every (sequence, head) row of the grid carry work.  Rotating
    // the chunk index per row spreads the live chunks evenly over the XCDs;
    // without it XCD 0 always gets the odd chunk and finishes last.
    const uint32_t chunk = (blockIdx.x + blockIdx.y + 3 * blockIdx.z) % gridDim.x;
    const uint32_t kvh = blockIdx.y / p.q_groups;
    const uint32_t qg = blockIdx.y % p.q_groups;
    const uint32_t b = blockIdx.z;

    uint32_t len = p.seq_lens ? uint32_t(max(p.seq_lens[b], 0)) : p.max_tokens;
    len = min(len, p.max_tokens);
    const uint32_t chunk_start = chunk * p.chunk_tokens;
    if (chunk_start >= len) return;
    const uint32_t chunk_end = min(len, chunk_start + p.chunk_tokens);
    const uint32_t n_tiles = (chunk_end - chunk_start + kTile - 1) / kTile;

    const uint32_t lane = threadIdx.x & 63;
    const uint32_t wave = threadIdx.x >> 6;
    const uint32_t n = lane & 15;  // MFMA column: query head within the group / row index m
    const uint32_t g = lane >> 4;  // MFMA k-group

    const uint32_t q_in_group = qg * 16 + n;  // query head index inside the GQA group
    const bool q_valid = q_in_group < p.group;
    const uint32_t qh = kvh * p.group + (q_valid ? q_in_group : 0);

    const int32_t* table =
        kRows != kRowsContiguous ? p.tables + size_t(b) * p.max_blocks : nullptr;
    const uint16_t* kbase = p.k + size_t(kvh) * p.head_stride + 8 * g;
    const uint16_t* vbase = p.v + size_t(kvh) * p.head_stride + 8 * (n & (kD / 8 - 1));

    // first tile's rows: issued before anything else so the latency overlaps the Q load
    uint32_t row_cur =
        tile_row<kRows>(p, table, chunk_start + min(wave, n_tiles - 1) * kTile, lane, len);

    // ---- Q as MFMA B operand: lane (n, g), step s holds Q[qh][32s + 8g .. +7]
    half8 bq[kKSteps];
    half8 bq_lo[kQF32 ? kKSteps : 1];
    {
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
                    _Float16 h = static_cast<_Float16>(xv);
                    hi[i] = h;
                    lo[i] = static_cast<_Float16>(xv - static_cast<float>(h));
                }
                bq[s] = hi;
                bq_lo[s] = lo;
            } else {
                uint4v w = *reinterpret_cast<const uint4v*>(static_cast<const uint16_t*>(p.q) +
                                                            off + 32 * s);
                if (!q_valid) w = uint4v{0, 0, 0, 0};
                bq[s] = as_half8(w);
            }
        }
    }

    float m_run = kNegBig;  // running max (log2 domain), identical in the 4 lanes of a column
    float l_run = 0.0f;     // running sum, lane-partial (summed over g at the end)
    float4v acc[8];
#pragma unroll
    for (int t = 0; t < 8; t++) acc[t] = float4v{0, 0, 0, 0};

    for (uint32_t tile = wave; tile < n_tiles; tile += kWavesPerWG) {
        const uint32_t tok0 = chunk_start + tile * kTile;

        // rows of the tile after this one (its table read is in flight during this tile)
        const uint32_t next = min(tile + kWavesPerWG, n_tiles - 1);
        const uint32_t row_nxt = tile_row<kRows>(p, table, chunk_start + next * kTile, lane, len);

        // ---- K tile: two 16-token sub-tiles, 4 k-steps each
        half8 ka[2][kKSteps];
#pragma unroll
        for (int sub = 0; sub < 2; sub++) {
            const uint32_t row = lane_read(row_cur, 16 * sub + n);
            const uint16_t* kp = kbase + size_t(row) * p.tok_stride;
#pragma unroll
            for (int s = 0; s < kKSteps; s++)
                ka[sub][s] = as_half8(*reinterpret_cast<const uint4v*>(kp + 32 * s));
        }
        // ---- V tile: 8 token rows per lane, 16 bytes each
        uint4v vr[8];
#pragma unroll
        for (int j = 0; j < 8; j++) {
            const uint32_t row = lane_read(row_cur, tau(g, j));
            vr[j] = *reinterpret_cast<const uint4v*>(vbase + size_t(row) * p.tok_stride);
        }

        // ---- S^T = K Q^T
        float4v c0 = {0, 0, 0, 0}, c1 = {0, 0, 0, 0};
#pragma unroll
        for (int s = 0; s < kKSteps; s++) {
            c0 = __builtin_amdgcn_mfma_f32_16x16x32_f16(ka[0][s], bq[s], c0, 0, 0, 0);
            c1 = __builtin_amdgcn_mfma_f32_16x16x32_f16(ka[1][s], bq[s], c1, 0, 0, 0);
            if constexpr (kQF32) {
                c0 = __builtin_amdgcn_mfma_f32_16x16x32_f16(ka[0][s], bq_lo[s], c0, 0, 0, 0);
                c1 = __builtin_amdgcn_mfma_f32_16x16x32_f16(ka[1][s], bq_lo[s], c1, 0, 0, 0);
            }
        }

        // ---- online softmax; lane (n, g) holds tokens 4g+r and 16+4g+r of column n
        float s[8];
#pragma unroll
        for (int r = 0; r < 4; r++) {
            s[r] = c0[r] * p.scale_log2;
            s[4 + r] = c1[r] * p.scale_log2;
        }
        if (tok0 + kTile > chunk_end) {  // only the last tile of a sequence is ragged
#pragma unroll
            for (int r = 0; r < 4; r++) {
                if (tok0 + 4 * g + r >= chunk_end) s[r] = -INFINITY;
                if (tok0 + 16 + 4 * g + r >= chunk_end) s[4 + r] = -INFINITY;
            }
        }
        float mloc = fmaxf(fmaxf(fmaxf(s[0], s[1]), fmaxf(s[2], s[3])),
                           fmaxf(fmaxf(s[4], s[5]), fmaxf(s[6], s[7])));
        mloc = fmaxf(mloc, wave_shfl_xor(mloc, 16));
        mloc = fmaxf(mloc, wave_shfl_xor(mloc, 32));
        const float m_new = fmaxf(m_run, mloc);
        const float alpha = fast_exp2(m_run - m_new);
        m_run = m_new;
        float psum = 0.0f;
        float pj[8];
#pragma unroll
        for (int j = 0; j < 8; j++) {
            pj[j] = fast_exp2(s[j] - m_new);
            psum += pj[j];
        }
        l_run = l_run * alpha + psum;
        uint4v bpw;
        bpw.x = pack_f16x2(pj[0], pj[1]);
        bpw.y = pack_f16x2(pj[2], pj[3]);
        bpw.z = pack_f16x2(pj[4], pj[5]);
        bpw.w = pack_f16x2(pj[6], pj[7]);
        const half8 bp = as_half8(bpw);

        // ---- O^T += V^T P^T : 8 d-tiles, A operand by in-register transpose
#pragma unroll
        for (int t = 0; t < 8; t++) {
            const uint32_t sel = (t & 1) ? 0x07060302u : 0x05040100u;
            uint4v aw;
            aw.x = __builtin_amdgcn_perm(vr[1][t >> 1], vr[0][t >> 1], sel);
            aw.y = __builtin_amdgcn_perm(vr[3][t >> 1], vr[2][t >> 1], sel);
            aw.z = __builtin_amdgcn_perm(vr[5][t >> 1], vr[4][t >> 1], sel);
            aw.w = __builtin_amdgcn_perm(vr[7][t >> 1], vr[6][t >> 1], sel);
            float4v cin = acc[t] * alpha;
            acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(as_half8(aw), bp, cin, 0, 0, 0);
        }
        row_cur = row_nxt;
    }

    // ---- reduce the lane-partial sums over the 4 k-groups
    l_run += wave_shfl_xor(l_run, 16);
    l_run += wave_shfl_xor(l_run, 32);

    // ---- merge the 4 waves through LDS
    constexpr int kRowPad = kD + 4;
    __shared__ float s_o[kWavesPerWG][16][kRowPad];
    __shared__ float s_m[kWavesPerWG][16];
    __shared__ float s_l[kWavesPerWG][16];
    if (g == 0) {
        s_m[wave][n] = m_run;
        s_l[wave][n] = l_run;
    }
    if (32 * g < uint32_t(kD)) {  // output rows 4 g + r of d-tile t are d = 32 g + 8 r + t
#pragma unroll
        for (int t = 0; t < 8; t++)
#pragma unroll
            for (int r = 0; r < 4; r++) s_o[wave][n][32 * g + 8 * r + t] = acc[t][r];
    }
    __syncthreads();

    const uint32_t rows = min(p.group - qg * 16, 16u);
    for (uint32_t i = threadIdx.x; i < rows * kD; i += blockDim.x) {
        const uint32_t row = i / kD, d = i % kD;
        float mx = s_m[0][row];
#pragma unroll
        for (int w = 1; w < kWavesPerWG; w++) mx = fmaxf(mx, s_m[w][row]);
        float o = 0.0f, l = 0.0f;
#pragma unroll
        for (int w = 0; w < kWavesPerWG; w++) {
            const float f = fast_exp2(s_m[w][row] - mx);
            o += s_o[w][row][d] * f;
            l += s_l[w][row] * f;
        }
        const size_t head = size_t(b) * p.num_heads + kvh * p.group + qg * 16 + row;
        if (p.max_chunks == 1) {
            // the only chunk of its (sequence, head): this is the result, no merge launch
            p.out[head * kD + d] = o / l;
            if (p.lse && d == 0) p.lse[head] = (mx + __builtin_amdgcn_logf(l)) * kLn2;
            continue;
        }
        const size_t slot = head * p.max_chunks + chunk;
        p.part_o[slot * kD + d] = o;
        if (d == 0) {
            p.part_ml[slot * 2 + 0] = mx;
            p.part_ml[slot * 2 + 1] = l;
        }
    }
}

// Merges the per-chunk partials of one (sequence, query head):
//   M = max_c m_c,  L = sum_c l_c 2^(m_c - M),  out = sum_c O_c 2^(m_c - M) / L,
//   lse = (M + log2 L) ln 2.
__global__ void __launch_bounds__(kHeadDim) decode_merge_kernel(DecodeParams p) {  // head_dim threads
    const uint32_t qh = blockIdx.x;
    const uint32_t b = blockIdx.y;
    uint32_t len = p.seq_lens ? uint32_t(max(p.seq_lens[b], 0)) : p.max_tokens;
    len = min(len, p.max_tokens);
    if (len == 0) return;  // untouched, as the reference kernel does for empty sequences
    const uint32_t n_chunks = (len + p.chunk_tokens - 1) / p.chunk_tokens;
    const size_t head = size_t(b) * p.num_heads + qh;
    const float* ml = p.part_ml + head * p.max_chunks * 2;
    const uint32_t D = p.head_dim;
    const float* po = p.part_o + head * p.max_chunks * D;
    const uint32_t d = threadIdx.x;

    float mx = kNegBig;
    for (uint32_t c = 0; c < n_chunks; c++) mx = fmaxf(mx, ml[2 * c]);
    float o = 0.0f, l = 0.0f;
    for (uint32_t c = 0; c < n_chunks; c++) {
        const float f = fast_exp2(ml[2 * c] - mx);
        l += ml[2 * c + 1] * f;
        o += po[size_t(c) * D + d] * f;
    }
    p.out[head * D + d] = o / l;
    if (p.lse && d == 0) p.lse[head] = (mx + __builtin_amdgcn_logf(l)) * kLn2;
}

}  // namespace

// Split-K chunk used when the caller passes 0.  GRANITE_HIP_DECODE_CHUNK (a
// multiple of 32) overrides it for tuning runs.
static uint32_t default_chunk_tokens() {
    static const uint32_t value = [] {
        const char* env = std::getenv("GRANITE_HIP_DECODE_CHUNK");
        if (env) {
            const long v = std::strtol(env, nullptr, 10);
            if (v >= kTile && v % kTile == 0 && v <= (1 << 20)) return static_cast<uint32_t>(v);
        }
        return 256u;
    }();
    return value;
}

// GRANITE_HIP_DECODE_MODE=chunk selects the one-workgroup-per-chunk kernel,
// anything else the persistent one.
static bool use_stream_kernel() {
    static const bool value = [] {
        const char* env = std::getenv("GRANITE_HIP_DECODE_MODE");
        return !(env && std::string(env) == "chunk");
    }();
    return value;
}

int launch_decode(const granite_hip_decode_args& a, const ScratchSource& scratch) {
    if (!a.q || !a.k_cache || !a.v_cache || !a.out) return GRANITE_HIP_ENULL;
    if (a.head_dim != 128 && a.head_dim != 64) return GRANITE_HIP_EUNSUPPORTED;
    const uint32_t D = a.head_dim;
    if (a.num_heads == 0 || a.num_kv_heads == 0 || a.num_heads % a.num_kv_heads != 0)
        return GRANITE_HIP_EINVAL;
    if (a.q_dtype != GRANITE_HIP_F32 && a.q_dtype != GRANITE_HIP_F16) return GRANITE_HIP_EINVAL;
    if (scratch.query) *scratch.query = 0;
    if (a.batch_size == 0) return GRANITE_HIP_OK;

    DecodeParams p{};
    p.q = a.q;
    p.k = static_cast<const uint16_t*>(a.k_cache);
    p.v = static_cast<const uint16_t*>(a.v_cache);
    p.tables = a.block_tables;
    p.seq_lens = a.seq_lens;
    p.out = static_cast<float*>(a.out);
    p.lse = a.lse;
    p.batch = a.batch_size;
    p.head_dim = D;
    p.num_heads = a.num_heads;
    p.num_kv_heads = a.num_kv_heads;
    p.group = a.num_heads / a.num_kv_heads;
    p.q_groups = (p.group + 15) / 16;
    if (a.block_tables) {
        if (a.block_size == 0 || a.max_blocks_per_seq == 0) return GRANITE_HIP_EINVAL;
        p.block_size = a.block_size;
        p.max_blocks = a.max_blocks_per_seq;
        p.bs_shift = (a.block_size & (a.block_size - 1)) == 0 ? __builtin_ctz(a.block_size) : -1;
        p.tok_stride = int64_t(a.num_kv_heads) * D;
        p.head_stride = D;
        const uint64_t mt = uint64_t(a.block_size) * a.max_blocks_per_seq;
        if (mt >= (1ull << 31)) return GRANITE_HIP_EINVAL;
        p.max_tokens = static_cast<uint32_t>(mt);
    } else {
        if (a.batch_size != 1 || a.max_seq == 0) return GRANITE_HIP_EINVAL;
        p.block_size = 1;
        p.max_blocks = 0;
        p.bs_shift = 0;
        p.tok_stride = D;
        p.head_stride = int64_t(a.max_seq) * D;
        p.max_tokens = a.max_seq;
    }
    if (!a.seq_lens) {
        if (a.fixed_seq_len == 0 || a.fixed_seq_len > p.max_tokens) return GRANITE_HIP_EINVAL;
        p.max_tokens = a.fixed_seq_len;
    }
    p.chunk_tokens = a.chunk_tokens ? a.chunk_tokens : default_chunk_tokens();
    if (p.chunk_tokens % kTile != 0) return GRANITE_HIP_EINVAL;
    // Short contexts (at most kDirectTokens, six tiles per wave): one workgroup per
    // (sequence, KV head) takes the whole context and writes the result itself.  One launch
    // instead of two, which is what such a call's time consists of (contiguous decode over
    // 512 tokens: 15 -> 9 us).
    constexpr uint32_t kDirectTokens = 768;
    const bool direct = !a.chunk_tokens && p.max_tokens <= kDirectTokens && use_stream_kernel();
    if (direct) p.chunk_tokens = (p.max_tokens + kTile - 1) / kTile * kTile;
    p.max_chunks = (p.max_tokens + p.chunk_tokens - 1) / p.chunk_tokens;
    p.scale_log2 = a.scale * kLog2e;

    const bool qf32 = a.q_dtype == GRANITE_HIP_F32;
    const int rows = !a.block_tables ? kRowsContiguous
                                     : (p.bs_shift >= 0 ? kRowsPagedPow2 : kRowsPagedAny);
    if (use_stream_kernel() && !direct) {
        const uint64_t units = uint64_t(p.batch) * ((p.max_tokens + kTile - 1) / kTile) *
                               p.num_kv_heads * p.q_groups;
        if (units < (1ull << 31) && decode_stream_supports(p.batch))
            return launch_decode_stream(p, qf32, rows, scratch);
    }

    if (p.max_chunks > 65535u * 32 || p.batch > 65535u) return GRANITE_HIP_EINVAL;
    int rc = GRANITE_HIP_OK;
    if (p.max_chunks > 1) {
        const size_t slots = size_t(p.batch) * p.num_heads * p.max_chunks;
        const size_t need = slots * (D + 2) * sizeof(float);
        void* ws = nullptr;
        rc = take_scratch(scratch, need, &ws);
        if (rc != GRANITE_HIP_OK || scratch.query) return rc;
        p.part_o = static_cast<float*>(ws);
        p.part_ml = p.part_o + slots * D;
    } else if (scratch.query) {
        return GRANITE_HIP_OK;  // one chunk per sequence: the kernel writes the result itself
    }

    dim3 grid(p.max_chunks, p.num_kv_heads * p.q_groups, p.batch);
    dim3 block(kWavesPerWG * kWave);
    hipStream_t st = ctx().stream;
    {
        KernelTimerScope timer("decode_splitk");
#define GHIP_DECODE_CASE(QF32, ROWS)                                        \
    if (qf32 == QF32 && rows == ROWS) {                                     \
        if (D == 128) decode_splitk_kernel<QF32, ROWS, 128><<<grid, block, 0, st>>>(p); \
        else decode_splitk_kernel<QF32, ROWS, 64><<<grid, block, 0, st>>>(p);           \
    }
        GHIP_DECODE_CASE(true, kRowsContiguous)
        GHIP_DECODE_CASE(true, kRowsPagedPow2)
        GHIP_DECODE_CASE(true, kRowsPagedAny)
        GHIP_DECODE_CASE(false, kRowsContiguous)
        GHIP_DECODE_CASE(false, kRowsPagedPow2)
        GHIP_DECODE_CASE(false, kRowsPagedAny)
#undef GHIP_DECODE_CASE
    }
    rc = launch_status();
    if (rc != GRANITE_HIP_OK || p.max_chunks == 1) return rc;
    {
        KernelTimerScope timer("decode_merge");
        decode_merge_kernel<<<dim3(p.num_heads, p.batch), dim3(D), 0, st>>>(p);
    }
    return launch_status();
}

}  // namespace ghip
