// Projections either side of attention on Q4_K weights: the fused Q/K/V matvec and the
// plain matvec (output projection) for gfx950.
//
// Stands in for
//   fused_qkv_matvec_q4k   src/backend/metal/kernels/metal_shaders_quant.h:167-295
//   matvec_q4k             metal_shaders_quant.h:59-163
// (MetalCompute::fused_qkv_matvec_q4k / matvec_q4k, include/granite/metal_compute.h:683-694,
// 73-79).  A Q4_K super-block holds 256 weights in 144 bytes: d and dmin (half), 12 bytes of
// packed 6-bit scales and minima for 8 sub-blocks of 32, and 128 bytes of 4-bit values; a
// weight is d * scale * q - dmin * min (src/model/gguf.cpp:952-1020).
//
// The work is one pass over the weights (4.5 bits each), so the kernel is built to keep
// 16-byte loads in flight, not around arithmetic.  A wave owns kRowsPerWave output rows.  Its
// 64 lanes cover 8 super-blocks at a time, 8 lanes per block; a lane takes one 16-byte piece
// of a block's nibbles (16 weights from the low nibbles and, 32 positions further on, 16
// from the high ones) and the block's 16-byte header, so every load instruction of the wave
// covers 8 x 144 contiguous bytes of a row.  The inputs reach the lanes through LDS: the
// workgroup loads the columns of a trip once (issued ahead of the weights' loads, so that
// they are staged while the weights are on their way) and a lane reads the 32 it needs,
// which serve all its rows.  As in the reference kernel the minima are applied to the sum of the
// inputs of a sub-block instead of to every weight, and a nibble is converted with one
// byte-to-float instruction (the high nibbles stay multiplied by 16, which the scale takes
// back).  Lanes are combined with shuffles at the end; results are float.
//
// A batch of tokens (a batched decode step) goes through the matrix cores instead
// (matmul_q4k_tokens_kernel): 32 tokens are the rows of the MFMA's A operand, 32 weight rows
// its columns; a workgroup takes one such tile of tokens, or two through every unpacked weight.  What makes that cheap for a 4-bit format: the B operand is not a
// dequantised weight but the integer scale * q (at most 63 * 15 = 945), written as the raw
// bits of a half -- a denormal, i.e. exactly scale * q * 2^-24, which the matrix cores keep --
// so a nibble costs a mask, a byte shuffle and a 24-bit multiply shared between two weights,
// and nothing is rounded; d * 2^24 is applied once per super-block to the accumulator.  The
// minima go through one more MFMA per super-block, the integer minima against the sums of
// the inputs of the sub-blocks.  A token's inputs of a chunk are first divided by the power of
// two that brings the largest of them into [1, 2) (exact; undone when the chunk's result is
// added), then split into a half and a half remainder (two MFMAs per step): 22 significant
// bits of the largest input and the same absolute resolution for the others, whatever the
// magnitude of the inputs, and no sub-block sum can leave the half range.  A workgroup stages its 512 input columns in
// LDS once (both halves, and the sub-block sums) for its 8 waves x 32 weight rows; the chunks
// of K are combined by a second small kernel.
#include "common.h"

namespace ghip {
namespace {

constexpr uint32_t kQK = 256;          // weights per super-block
constexpr uint32_t kBlockBytes = 144;  // bytes per super-block
constexpr int kRowsPerWave = 2;
constexpr int kWavesPerGroup = 4;
constexpr int kMaxBatch = 2;  // input vectors the vector kernel takes; larger batches go to the matrix cores

struct MatvecParams {
    const float* x;       // [batch, K], rows x_stride floats apart
    int64_t x_stride;
    // up to three weight matrices share a launch; rows are numbered through all of them
    const uint8_t* w[3];  // [n[i], K / 256] super-blocks
    float* y[3];          // [batch, n[i]], rows y_stride[i] floats apart
    int64_t y_stride[3];
    uint32_t n[3];
    uint32_t row_end[3];  // running totals of n[]
    uint32_t blocks_per_row;
    uint32_t batch;
};

__device__ __forceinline__ float ubyte_to_float(uint32_t word, int byte) {
    // one v_cvt_f32_ubyte{0..3} per byte
    return float((word >> (8 * byte)) & 0xFFu);
}

// `word` as the compiler must take it: a value it knows nothing about.  The nibble masks go
// through this before their bytes are converted, because from a byte of (w & 0x0F0F0F0F) the
// compiler otherwise makes a four-bit field extract followed by a conversion, two
// instructions where v_cvt_f32_ubyteN on the masked word is one.  No instruction is emitted.
__device__ __forceinline__ uint32_t opaque(uint32_t word) {
    asm("" : "+v"(word));
    return word;
}

// Byte k (0..11) of the 12 scale bytes held in three words.
__device__ __forceinline__ uint32_t scale_byte(const uint4v& head, uint32_t k) {
    const uint32_t word = k < 4 ? head.y : (k < 8 ? head.z : head.w);
    return (word >> (8 * (k & 3))) & 0xFFu;
}

// Scale and minimum of sub-block j (0..7) of a super-block (gguf.cpp:963-971).
__device__ __forceinline__ void scale_min(const uint4v& head, uint32_t j, float& sc, float& mn) {
    uint32_t s, m;
    if (j < 4) {
        s = scale_byte(head, j) & 63u;
        m = scale_byte(head, j + 4) & 63u;
    } else {
        s = (scale_byte(head, j + 4) & 0xFu) | ((scale_byte(head, j - 4) >> 6) << 4);
        m = (scale_byte(head, j + 4) >> 4) | ((scale_byte(head, j) >> 6) << 4);
    }
    sc = float(s);
    mn = float(m);
}

template <int kBatch>
__global__ void __launch_bounds__(kWavesPerGroup* kWave) matvec_q4k_kernel(MatvecParams p) {
    const uint32_t lane = threadIdx.x & 63;
    const uint32_t wave = threadIdx.x >> 6;
    const uint32_t piece = lane & 7;    // 16-byte piece of the block's 128 nibble bytes
    const uint32_t blk_lane = lane >> 3;  // block inside the group of 8 the wave covers
    const uint32_t row0 = (blockIdx.x * kWavesPerGroup + wave) * kRowsPerWave;
    const uint32_t rows_total = p.row_end[2];
    // (a wave past the last row stays for the barriers: its loads are clamped, its stores masked)

    // where each of the wave's rows lives
    const uint8_t* wrow[kRowsPerWave];
    float* yrow[kRowsPerWave];
    int64_t ystride[kRowsPerWave];
#pragma unroll
    for (int r = 0; r < kRowsPerWave; r++) {
        const uint32_t row = min(row0 + r, rows_total - 1);  // clamped: loads stay in bounds
        const int seg = row < p.row_end[0] ? 0 : (row < p.row_end[1] ? 1 : 2);
        const uint32_t local = row - (seg == 0 ? 0 : p.row_end[seg - 1]);
        wrow[r] = p.w[seg] + size_t(local) * p.blocks_per_row * kBlockBytes;
        yrow[r] = p.y[seg] + local;
        ystride[r] = p.y_stride[seg];
    }

    // the lane's weights inside a block: group of 64 `grp`, 16 of its first 32 positions
    // (low nibbles, sub-block 2 grp) and the 16 that lie 32 further on (high nibbles,
    // sub-block 2 grp + 1)
    const uint32_t grp = piece >> 1;
    const uint32_t col = 64 * grp + 16 * (piece & 1);

    float acc[kRowsPerWave][kBatch];
#pragma unroll
    for (int r = 0; r < kRowsPerWave; r++)
#pragma unroll
        for (int b = 0; b < kBatch; b++) acc[r][b] = 0.0f;

    // kGroups groups of 8 super-blocks per trip, all their loads issued before any arithmetic
    // (one input vector: two groups, which is the whole row of a 4096-wide layer).  The inputs
    // of a trip's columns reach the lanes through LDS: the workgroup loads the slice once, 16
    // bytes per thread and load, instead of every wave loading all of it (which was three
    // times the bytes of the weights through the vector cache).  Their loads are issued ahead
    // of the weights' -- loads return in issue order, so the slice (from the last-level cache)
    // is in LDS while the weights are still on their way.  Two buffers, so that one barrier
    // per trip is enough.
    constexpr int kGroups = kBatch == 1 ? 2 : 1;
    constexpr uint32_t kSlice = 8 * kGroups * kQK;                    // columns per trip
    constexpr uint32_t kSlicePad = kSlice + kSlice / 16 + kSlice / 16;  // floats per staged slice
    constexpr int kSliceLoads = int(kSlice / 4 / (kWavesPerGroup * kWave));  // float4 per thread and input vector
    static_assert(kSlice % (4 * kWavesPerGroup * kWave) == 0, "a slice is whole rounds of the workgroup's 16-byte loads");
    // float idx of a slice sits at idx + 4 (idx / 64) + 16 (idx / 256): the 16 lanes that a
    // 16-byte LDS read serves at a time (two blocks x eight pieces) then fall on 16 different
    // groups of four banks
    auto staged = [](uint32_t idx) { return idx + 4 * (idx / 64) + 16 * (idx / 256); };
    __shared__ __attribute__((aligned(16))) float s_x[2][kBatch * kSlicePad];
    const uint32_t K = p.blocks_per_row * kQK;
    uint32_t buf = 0;
    for (uint32_t ib0 = 0; ib0 < p.blocks_per_row; ib0 += 8 * kGroups, buf ^= 1) {
        bool live[kGroups];
        uint4v head[kGroups][kRowsPerWave], nib[kGroups][kRowsPerWave];
        float4v xlo[kGroups][kBatch][4], xhi[kGroups][kBatch][4];
        // the trip's slice of the inputs (columns past K repeat the last four: their blocks are not live)
        float4v slice[kBatch][kSliceLoads];
#pragma unroll
        for (int b = 0; b < kBatch; b++) {
            // (an input vector past the batch repeats the last one; its results are not stored)
            const float* xb = p.x + int64_t(min(uint32_t(b), p.batch - 1)) * p.x_stride;
#pragma unroll
            for (int j = 0; j < kSliceLoads; j++) {
                const uint32_t idx = 4 * (threadIdx.x + kWavesPerGroup * kWave * j);
                slice[b][j] = *reinterpret_cast<const float4v*>(xb + min(ib0 * kQK + idx, K - 4));
            }
        }
        // the weights of all rows: these are the loads that go to memory
#pragma unroll
        for (int gi = 0; gi < kGroups; gi++) {
            const uint32_t ib = ib0 + 8 * gi + blk_lane;
            live[gi] = ib < p.blocks_per_row;
            const uint32_t ibc = live[gi] ? ib : p.blocks_per_row - 1;
#pragma unroll
            for (int r = 0; r < kRowsPerWave; r++) {
                const uint8_t* blk = wrow[r] + size_t(ibc) * kBlockBytes;
                head[gi][r] = __builtin_nontemporal_load(reinterpret_cast<const uint4v*>(blk));
                nib[gi][r] = __builtin_nontemporal_load(reinterpret_cast<const uint4v*>(blk + 16 + 16 * piece));
            }
        }
#pragma unroll
        for (int b = 0; b < kBatch; b++)
#pragma unroll
            for (int j = 0; j < kSliceLoads; j++) {
                const uint32_t idx = 4 * (threadIdx.x + kWavesPerGroup * kWave * j);
                *reinterpret_cast<float4v*>(&s_x[buf][b * kSlicePad + staged(idx)]) = slice[b][j];
            }
        __syncthreads();
        // the lane's inputs: 16 + 16 floats per input vector and group
#pragma unroll
        for (int gi = 0; gi < kGroups; gi++)
#pragma unroll
            for (int b = 0; b < kBatch; b++) {
                const float* xp = &s_x[buf][b * kSlicePad + staged((8 * gi + blk_lane) * kQK + col)];
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    xlo[gi][b][i] = *reinterpret_cast<const float4v*>(xp + 4 * i);
                    xhi[gi][b][i] = *reinterpret_cast<const float4v*>(xp + 32 + 4 * i);
                }
            }
#pragma unroll
        for (int gi = 0; gi < kGroups; gi++) {
            // sums of the inputs of the two sub-blocks, for the minima
            float sum_l[kBatch], sum_h[kBatch];
#pragma unroll
            for (int b = 0; b < kBatch; b++) {
                sum_l[b] = 0.0f;
                sum_h[b] = 0.0f;
#pragma unroll
                for (int i = 0; i < 4; i++)
#pragma unroll
                    for (int e = 0; e < 4; e++) {
                        sum_l[b] += xlo[gi][b][i][e];
                        sum_h[b] += xhi[gi][b][i][e];
                    }
            }
#pragma unroll
            for (int r = 0; r < kRowsPerWave; r++) {
                const half2v dd = __builtin_bit_cast(half2v, head[gi][r].x);
                const float d = live[gi] ? float(dd.x) : 0.0f;
                const float dmin = live[gi] ? float(dd.y) : 0.0f;
                float sc_l, mn_l, sc_h, mn_h;
                scale_min(head[gi][r], 2 * grp, sc_l, mn_l);
                scale_min(head[gi][r], 2 * grp + 1, sc_h, mn_h);
                float dot_l[kBatch], dot_h[kBatch];
#pragma unroll
                for (int b = 0; b < kBatch; b++) dot_l[b] = dot_h[b] = 0.0f;
#pragma unroll
                for (int wd = 0; wd < 4; wd++) {
                    const uint32_t lo = opaque(nib[gi][r][wd] & 0x0F0F0F0Fu);
                    const uint32_t hi = opaque(nib[gi][r][wd] & 0xF0F0F0F0u);  // 16 x the high nibbles
#pragma unroll
                    for (int e = 0; e < 4; e++) {
                        const float ql = ubyte_to_float(lo, e);
                        const float qh = ubyte_to_float(hi, e);
#pragma unroll
                        for (int b = 0; b < kBatch; b++) {
                            dot_l[b] = __builtin_fmaf(xlo[gi][b][wd][e], ql, dot_l[b]);
                            dot_h[b] = __builtin_fmaf(xhi[gi][b][wd][e], qh, dot_h[b]);
                        }
                    }
                }
                const float wl = d * sc_l, wh = d * sc_h * 0.0625f;
                const float ml = dmin * mn_l, mh = dmin * mn_h;
#pragma unroll
                for (int b = 0; b < kBatch; b++)
                    acc[r][b] += (wl * dot_l[b] + wh * dot_h[b]) - (ml * sum_l[b] + mh * sum_h[b]);
            }
        }
    }

    // combine the 64 lanes; lane 0 stores
#pragma unroll
    for (int r = 0; r < kRowsPerWave; r++)
#pragma unroll
        for (int b = 0; b < kBatch; b++) {
            float v = acc[r][b];
#pragma unroll
            for (int off = 32; off >= 1; off >>= 1) v += wave_shfl_xor(v, off);
            if (lane == 0 && row0 + r < rows_total && uint32_t(b) < p.batch)
                yrow[r][int64_t(b) * ystride[r]] = v;
        }
}


// ---- a batch of tokens on the matrix cores ---------------------------------------------------

constexpr int kTokTile = 32;          // tokens of one MFMA's A operand; a workgroup takes one or two such tiles
constexpr int kTokWaves = 8;          // waves per workgroup, 32 weight rows each
constexpr int kTokRows = 32 * kTokWaves;
constexpr int kChunkK = 512;          // input columns a workgroup stages: two super-blocks
constexpr int kChunkBlocks = kChunkK / int(kQK);
constexpr int kXPitch = kChunkK + 8;  // halves per token row in LDS (16-byte reads without bank conflicts)
constexpr int kSubPerChunk = kChunkK / 32;
constexpr size_t tok_lds_bytes(int tiles) {
    return size_t(tiles) *
           (size_t(2 * kTokTile * kXPitch + 2 * kTokTile * kSubPerChunk) * sizeof(uint16_t) + kTokTile * sizeof(float));
}

struct MatmulTokParams {
    MatvecParams m;   // x, weights and row numbering as for the matvec; m.batch = all tokens
    float* partial;   // [chunks, tokens, rows_total]
    uint32_t chunks;  // ceil(K / kChunkK)
    uint32_t tokens;  // workgroups along the tokens * tokens per workgroup
};

__device__ __forceinline__ uint32_t bytes_to_u16_pair(uint32_t bytes, bool upper) {
    // bytes [b0 b1 b2 b3] -> b0 | b1 << 16 (or b2 | b3 << 16): one v_perm_b32
    return __builtin_amdgcn_perm(0u, bytes, upper ? 0x0c030c02u : 0x0c010c00u);
}

// kTiles tiles of kTokTile tokens per workgroup: the weights are unpacked once and meet every
// tile's inputs, so a second tile costs its staging and its MFMAs only.
template <int kTiles>
__global__ void __launch_bounds__(kTokWaves* kWave, 1) matmul_q4k_tokens_kernel(MatmulTokParams q) {
    const MatvecParams& p = q.m;
    constexpr int kTokens = kTiles * kTokTile;  // tokens per workgroup
    extern __shared__ __attribute__((aligned(16))) uint16_t s_tok[];
    uint16_t* const s_xh = s_tok;                          // [kTokens][kXPitch] half of x
    uint16_t* const s_xl = s_xh + kTokens * kXPitch;       // remainder of x
    uint16_t* const s_sh = s_xl + kTokens * kXPitch;       // [kTokens][kSubPerChunk] sub-block sums
    uint16_t* const s_sl = s_sh + kTokens * kSubPerChunk;  // and their remainders
    float* const s_unit = reinterpret_cast<float*>(s_sl + kTokens * kSubPerChunk);  // [kTokens] power of two a token's inputs were divided by
    const uint32_t tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const uint32_t n = lane & 31, g = lane >> 5;
    const uint32_t chunk = blockIdx.y;
    const uint32_t tok0 = blockIdx.z * kTokens;           // first token of this workgroup
    const uint32_t tile_batch = min(p.batch - tok0, uint32_t(kTokens));
    const uint32_t k0 = chunk * kChunkK;
    const uint32_t K = p.blocks_per_row * kQK;

    // ---- this lane's weight row
    const uint32_t rows_total = p.row_end[2];
    const uint32_t row = blockIdx.x * kTokRows + wave * 32 + n;
    const uint32_t rowc = min(row, rows_total - 1);  // clamped: loads stay in bounds, stores are masked
    const int seg = rowc < p.row_end[0] ? 0 : (rowc < p.row_end[1] ? 1 : 2);
    const uint32_t local = rowc - (seg == 0 ? 0 : p.row_end[seg - 1]);
    const uint8_t* wrow = p.w[seg] + size_t(local) * p.blocks_per_row * kBlockBytes;

    // ---- all loads first, the inputs ahead of the weights: loads return in the order they were
    // issued, so the inputs (from the last-level cache) can be converted while the weights are
    // still on their way from HBM
    // 16 threads per token; thread j of them takes the 16-byte pieces j, j + 16, ... of the
    // token's 512 columns, so that a load instruction covers 256 contiguous bytes per token
    // (with the pieces of a sub-block in one thread it touched 16 lines per token for 16 bytes
    // each, and the vector cache took four times as long over the same bytes)
    float4v raw[kTiles][8];
#pragma unroll
    for (int t = 0; t < kTiles; t++) {
        const uint32_t b = t * kTokTile + tid / kSubPerChunk, j = tid % kSubPerChunk;
        const float* xb = p.x + int64_t(tok0 + min(b, tile_batch - 1)) * p.x_stride;
#pragma unroll
        for (int i = 0; i < 8; i++)
            raw[t][i] = *reinterpret_cast<const float4v*>(xb + min(k0 + 4 * (j + 16 * i), K - 4));
    }
    uint4v head[kChunkBlocks], nib[kChunkBlocks][4];
    bool live_block[kChunkBlocks];
#pragma unroll
    for (int sb = 0; sb < kChunkBlocks; sb++) {
        const uint32_t ib = chunk * kChunkBlocks + sb;
        live_block[sb] = ib < p.blocks_per_row;
        const uint8_t* blk = wrow + size_t(min(ib, p.blocks_per_row - 1)) * kBlockBytes;
        head[sb] = __builtin_nontemporal_load(reinterpret_cast<const uint4v*>(blk));
#pragma unroll
        for (int G = 0; G < 4; G++)
            nib[sb][G] = __builtin_nontemporal_load(reinterpret_cast<const uint4v*>(blk + 16 + 32 * G + 16 * g));
    }

    // ---- stage the chunk's inputs.  A token's inputs of this chunk are first scaled by a power
    // of two (exact) that brings the largest of them into [1, 2), so that the split into a half
    // and a half remainder keeps 22 significant bits of the largest inputs whatever their
    // magnitude -- inputs beyond the half range and inputs far below its normal range alike --
    // and a sub-block's sum of 32 inputs stays below 64.  The factor is taken out again when
    // the chunk's products are added to y.
    static_assert(kSubPerChunk == 16 && kChunkK == 512, "16 threads per token, eight 16-byte pieces each");
#pragma unroll
    for (int t = 0; t < kTiles; t++) {
        const uint32_t b = t * kTokTile + tid / kSubPerChunk, j = tid % kSubPerChunk;
        const bool live_token = b < tile_batch;
        float amax = 0.0f;
#pragma unroll
        for (int i = 0; i < 8; i++) {
            const float4v v = raw[t][i];
            if (live_token && k0 + 4 * (j + 16 * i) < K)
                amax = fmaxf(fmaxf(amax, fmaxf(fabsf(v.x), fabsf(v.y))), fmaxf(fabsf(v.z), fabsf(v.w)));
        }
#pragma unroll
        for (int m = 1; m < kSubPerChunk; m <<= 1) amax = fmaxf(amax, __shfl_xor(amax, m, kWave));
        // 2^floor(log2 amax), kept inside [2^-126, 2^126] so that it and its inverse are normal floats
        const uint32_t ebits = min(max(__float_as_uint(amax) & 0x7F800000u, 0x00800000u), 0x7E800000u);
        const float unit = amax > 0.0f ? __uint_as_float(ebits) : 1.0f;
        const float scale = 1.0f / unit;
        if (j == 0) s_unit[b] = unit;
#pragma unroll
        for (int i = 0; i < 8; i++) {
            const uint32_t col = 4 * (j + 16 * i);  // first of the piece's four columns
            const bool live = live_token && k0 + col < K;
            const float4v r = raw[t][i];
            const float v[4] = {r.x, r.y, r.z, r.w};
            uint32_t hi[2], lo[2];
            float sum = 0.0f;
#pragma unroll
            for (int e = 0; e < 2; e++) {
                const float x0 = live ? v[2 * e] * scale : 0.0f, x1 = live ? v[2 * e + 1] * scale : 0.0f;
                sum += x0 + x1;
                const _Float16 h0 = static_cast<_Float16>(x0), h1 = static_cast<_Float16>(x1);
                half2v hh, ll;
                hh.x = h0;
                hh.y = h1;
                ll.x = static_cast<_Float16>(x0 - static_cast<float>(h0));
                ll.y = static_cast<_Float16>(x1 - static_cast<float>(h1));
                hi[e] = __builtin_bit_cast(uint32_t, hh);
                lo[e] = __builtin_bit_cast(uint32_t, ll);
            }
            *reinterpret_cast<uint2v*>(s_xh + b * kXPitch + col) = uint2v{hi[0], hi[1]};
            *reinterpret_cast<uint2v*>(s_xl + b * kXPitch + col) = uint2v{lo[0], lo[1]};
            // the eight pieces of sub-block 2 i + j / 8 lie in eight neighbouring threads
#pragma unroll
            for (int m = 1; m < 8; m <<= 1) sum += __shfl_xor(sum, m, kWave);
            if ((j & 7) == 0) {
                const _Float16 sh = static_cast<_Float16>(sum);
                s_sh[b * kSubPerChunk + 2 * i + (j >> 3)] = __builtin_bit_cast(uint16_t, sh);
                s_sl[b * kSubPerChunk + 2 * i + (j >> 3)] =
                    __builtin_bit_cast(uint16_t, static_cast<_Float16>(sum - static_cast<float>(sh)));
            }
        }
    }
    __syncthreads();

    float y[kTiles][16], unit[kTiles][16];  // register r of tile t is token 32 t + 8 (r / 4) + 4 g + r % 4
#pragma unroll
    for (int t = 0; t < kTiles; t++)
#pragma unroll
        for (int r = 0; r < 16; r++) {
            y[t][r] = 0.0f;
            unit[t][r] = s_unit[t * kTokTile + 8 * (r >> 2) + 4 * g + (r & 3)];
        }
#pragma unroll
    for (int sb = 0; sb < kChunkBlocks; sb++) {
        // integer scales and minima of the 8 sub-blocks (gguf.cpp:963-971)
        uint32_t sc[8], mn[8];
#pragma unroll
        for (uint32_t j = 0; j < 8; j++) {
            if (j < 4) {
                sc[j] = scale_byte(head[sb], j) & 63u;
                mn[j] = scale_byte(head[sb], j + 4) & 63u;
            } else {
                sc[j] = (scale_byte(head[sb], j + 4) & 0xFu) | ((scale_byte(head[sb], j - 4) >> 6) << 4);
                mn[j] = (scale_byte(head[sb], j + 4) >> 4) | ((scale_byte(head[sb], j) >> 6) << 4);
            }
        }
        float16v acc[kTiles];
#pragma unroll
        for (int t = 0; t < kTiles; t++) acc[t] = float16v{0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
        for (int G = 0; G < 4; G++) {
            // the lane's 16 bytes of group G: low nibbles are inputs 64 G + 16 g + 0..15 (scale 2 G),
            // high nibbles the inputs 32 further on (scale 2 G + 1)
#pragma unroll
            for (int part = 0; part < 4; part++) {  // 8 inputs each: low 0..7, low 8..15, high 0..7, high 8..15
                const bool high = part >= 2;
                const uint32_t w0 = nib[sb][G][2 * (part & 1)], w1 = nib[sb][G][2 * (part & 1) + 1];
                const uint32_t q0 = (high ? (w0 >> 4) : w0) & 0x0F0F0F0Fu;
                const uint32_t q1 = (high ? (w1 >> 4) : w1) & 0x0F0F0F0Fu;
                const uint32_t scale = sc[2 * G + (high ? 1 : 0)];
                uint4v bw;  // scale * q as raw half bits: scale * q * 2^-24 exactly
                bw.x = __umul24(bytes_to_u16_pair(q0, false), scale);
                bw.y = __umul24(bytes_to_u16_pair(q0, true), scale);
                bw.z = __umul24(bytes_to_u16_pair(q1, false), scale);
                bw.w = __umul24(bytes_to_u16_pair(q1, true), scale);
                const uint32_t kk = sb * kQK + 64 * G + (high ? 32 : 0) + 16 * g + 8 * (part & 1);
                const half8 bb = __builtin_bit_cast(half8, bw);
#pragma unroll
                for (int t = 0; t < kTiles; t++) {
                    const uint32_t at = (t * kTokTile + n) * kXPitch + kk;
                    const half8 ah = __builtin_bit_cast(half8, *reinterpret_cast<const uint4v*>(s_xh + at));
                    const half8 al = __builtin_bit_cast(half8, *reinterpret_cast<const uint4v*>(s_xl + at));
                    acc[t] = __builtin_amdgcn_mfma_f32_32x32x16_f16(ah, bb, acc[t], 0, 0, 0);
                    acc[t] = __builtin_amdgcn_mfma_f32_32x32x16_f16(al, bb, acc[t], 0, 0, 0);
                }
            }
        }
        // minima: sum_j min_j * (sum of the inputs of sub-block j), j on the contraction axis
        uint4v bm = {mn[0] | (mn[1] << 16), mn[2] | (mn[3] << 16), mn[4] | (mn[5] << 16), mn[6] | (mn[7] << 16)};
        if (g == 1) bm = uint4v{0, 0, 0, 0};  // only 8 of the 16 contraction slots are used
        const half2v dd = __builtin_bit_cast(half2v, head[sb].x);
        const float d = live_block[sb] ? float(dd.x) * 16777216.0f : 0.0f;      // the integers were worth 2^-24
        const float dmin = live_block[sb] ? float(dd.y) * 16777216.0f : 0.0f;
#pragma unroll
        for (int t = 0; t < kTiles; t++) {
            float16v accm = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
            uint4v sh = *reinterpret_cast<const uint4v*>(s_sh + (t * kTokTile + n) * kSubPerChunk + 8 * sb);
            uint4v sl = *reinterpret_cast<const uint4v*>(s_sl + (t * kTokTile + n) * kSubPerChunk + 8 * sb);
            if (g == 1) {
                sh = uint4v{0, 0, 0, 0};
                sl = uint4v{0, 0, 0, 0};
            }
            accm = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(half8, sh), __builtin_bit_cast(half8, bm), accm, 0, 0, 0);
            accm = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(half8, sl), __builtin_bit_cast(half8, bm), accm, 0, 0, 0);
#pragma unroll
            for (int r = 0; r < 16; r++) y[t][r] += (d * acc[t][r] - dmin * accm[r]) * unit[t][r];
        }
    }

    // ---- this chunk's part of y: register r of tile t is token 32 t + 8 (r / 4) + 4 g + r % 4, the
    // lane's column its row
    if (row < rows_total) {
#pragma unroll
        for (int t = 0; t < kTiles; t++)
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const uint32_t b = t * kTokTile + 8 * (r >> 2) + 4 * g + (r & 3);
                if (b < tile_batch) q.partial[(size_t(chunk) * q.tokens + tok0 + b) * rows_total + row] = y[t][r];
            }
    }
}

// y[token][row] = sum over the chunks of K; one thread per (row, token)
__global__ void __launch_bounds__(256) matmul_q4k_tokens_merge_kernel(MatmulTokParams q) {
    const MatvecParams& p = q.m;
    const uint32_t rows_total = p.row_end[2];
    const uint32_t row = blockIdx.x * 256 + threadIdx.x;
    const uint32_t b = blockIdx.y;
    if (row >= rows_total) return;
    float sum = 0.0f;
    for (uint32_t c0 = 0; c0 < q.chunks; c0 += 8) {  // eight loads in flight, summed in chunk order
        float part[8];
#pragma unroll
        for (uint32_t i = 0; i < 8; i++)
            part[i] = q.partial[(size_t(min(c0 + i, q.chunks - 1)) * q.tokens + b) * rows_total + row];
#pragma unroll
        for (uint32_t i = 0; i < 8; i++) sum += c0 + i < q.chunks ? part[i] : 0.0f;
    }
    const int seg = row < p.row_end[0] ? 0 : (row < p.row_end[1] ? 1 : 2);
    const uint32_t local = row - (seg == 0 ? 0 : p.row_end[seg - 1]);
    p.y[seg][int64_t(b) * p.y_stride[seg] + local] = sum;
}

// Tokens per launch of the matrix-core kernel, and the token count a launch's chunk sums are
// laid out for: whole workgroups of one tile (up to kTokTile tokens) or of two.
constexpr uint32_t kMaxLaunchTokens = 8 * kTokTile;
inline uint32_t padded_tokens(uint32_t batch) {
    const uint32_t per_group = batch > uint32_t(kTokTile) ? 2 * kTokTile : kTokTile;
    return (batch + per_group - 1) / per_group * per_group;
}

inline bool aligned16(const void* ptr) { return (reinterpret_cast<uintptr_t>(ptr) & 15u) == 0; }

}  // namespace

// Scratch bytes a projection of `batch` tokens onto `rows` weight rows needs (the chunk sums
// of the matrix-core path; none for the vector kernel).
size_t matvec_q4k_scratch_bytes(uint32_t K, uint64_t rows, uint32_t batch) {
    if (batch <= uint32_t(kMaxBatch) || K == 0) return 0;
    return size_t((K + kChunkK - 1) / kChunkK) * padded_tokens(min(batch, kMaxLaunchTokens)) * rows * sizeof(float);
}

int launch_matvec_q4k(const void* x, int64_t x_stride, const void* const w[3], void* const y[3],
                      const int64_t y_stride[3], const uint32_t n[3], uint32_t K, uint32_t batch) {
    if (!x) return GRANITE_HIP_ENULL;
    if (K == 0 || K % kQK != 0) return GRANITE_HIP_EINVAL;
    if (!aligned16(x) || (x_stride * 4) % 16 != 0) return GRANITE_HIP_EINVAL;
    uint64_t rows = 0;
    MatvecParams p{};
    for (int i = 0; i < 3; i++) {
        if (n[i] > 0) {
            if (!w[i] || !y[i]) return GRANITE_HIP_ENULL;
            if (!aligned16(w[i])) return GRANITE_HIP_EINVAL;
            if (batch > 1 && y_stride[i] < int64_t(n[i])) return GRANITE_HIP_EINVAL;
        }
        p.w[i] = static_cast<const uint8_t*>(w[i]);
        p.y[i] = static_cast<float*>(y[i]);
        p.y_stride[i] = y_stride[i];
        p.n[i] = n[i];
        rows += n[i];
        p.row_end[i] = static_cast<uint32_t>(rows);
    }
    if (batch > 1 && x_stride < int64_t(K)) return GRANITE_HIP_EINVAL;
    if (rows == 0 || batch == 0) return GRANITE_HIP_OK;
    if (rows > 0x7FFFFFFFull) return GRANITE_HIP_EINVAL;
    p.blocks_per_row = K / kQK;
    const uint32_t rows_per_group = kRowsPerWave * kWavesPerGroup;
    const dim3 grid(uint32_t((rows + rows_per_group - 1) / rows_per_group)), block(kWavesPerGroup * kWave);
    hipStream_t st = ctx().stream;
    if (batch > uint32_t(kMaxBatch)) {
        // a batch of tokens: the matrix cores.  Up to kMaxLaunchTokens tokens per launch, in
        // workgroups of two tiles of kTokTile tokens (of one tile when there are no more than
        // kTokTile); the workgroups along the tokens (grid.z) each stream the weights once, from
        // the last-level cache after the first when the matrices fit it.
        MatmulTokParams q{};
        q.chunks = (K + kChunkK - 1) / kChunkK;
        static bool configured1[kMaxDevices], configured2[kMaxDevices];  // the staged inputs exceed the 64 KiB default limit
        if (int rc = raise_dynamic_lds_limit(reinterpret_cast<const void*>(matmul_q4k_tokens_kernel<1>), tok_lds_bytes(1),
                                             configured1))
            return rc;
        if (int rc = raise_dynamic_lds_limit(reinterpret_cast<const void*>(matmul_q4k_tokens_kernel<2>), tok_lds_bytes(2),
                                             configured2))
            return rc;
        for (uint32_t b0 = 0; b0 < batch; b0 += kMaxLaunchTokens) {
            const uint32_t nb = min(batch - b0, kMaxLaunchTokens);
            const uint32_t per_group = nb > uint32_t(kTokTile) ? 2 * kTokTile : kTokTile;
            q.tokens = padded_tokens(nb);
            int rc = ensure_workspace(matvec_q4k_scratch_bytes(K, rows, nb));
            if (rc != GRANITE_HIP_OK) return rc;
            q.partial = static_cast<float*>(ctx().workspace);
            q.m = p;
            q.m.x = static_cast<const float*>(x) + int64_t(b0) * x_stride;
            q.m.x_stride = x_stride;
            for (int i = 0; i < 3; i++)
                if (q.m.y[i]) q.m.y[i] += int64_t(b0) * q.m.y_stride[i];
            q.m.batch = nb;
            {
                KernelTimerScope timer("matmul_q4k_tokens");
                const dim3 tgrid(uint32_t((rows + kTokRows - 1) / kTokRows), q.chunks, q.tokens / per_group);
                if (per_group == uint32_t(kTokTile))
                    matmul_q4k_tokens_kernel<1><<<tgrid, dim3(kTokWaves * kWave), tok_lds_bytes(1), st>>>(q);
                else
                    matmul_q4k_tokens_kernel<2><<<tgrid, dim3(kTokWaves * kWave), tok_lds_bytes(2), st>>>(q);
            }
            rc = launch_status();
            if (rc != GRANITE_HIP_OK) return rc;
            {
                KernelTimerScope timer("matmul_q4k_merge");
                matmul_q4k_tokens_merge_kernel<<<dim3(uint32_t((rows + 255) / 256), nb), dim3(256), 0, st>>>(q);
            }
            rc = launch_status();
            if (rc != GRANITE_HIP_OK) return rc;
        }
        return GRANITE_HIP_OK;
    }
    // up to kMaxBatch input vectors: the vector kernel, one launch
    {
        MatvecParams q = p;
        q.x = static_cast<const float*>(x);
        q.x_stride = batch > 1 ? x_stride : 0;
        q.batch = batch;
        KernelTimerScope timer("matvec_q4k");
        if (batch == 1) matvec_q4k_kernel<1><<<grid, block, 0, st>>>(q);
        else matvec_q4k_kernel<2><<<grid, block, 0, st>>>(q);
        int rc = launch_status();
        if (rc != GRANITE_HIP_OK) return rc;
    }
    return GRANITE_HIP_OK;
}

}  // namespace ghip
