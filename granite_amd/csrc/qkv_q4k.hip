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
// covers 8 x 144 contiguous bytes of a row.  The 32 inputs a lane needs are loaded once and
// serve all its rows.  As in the reference kernel the minima are applied to the sum of the
// inputs of a sub-block instead of to every weight, and a nibble is converted with one
// byte-to-float instruction (the high nibbles stay multiplied by 16, which the scale takes
// back).  Lanes are combined with shuffles at the end; results are float.
#include "common.h"

namespace ghip {
namespace {

constexpr uint32_t kQK = 256;          // weights per super-block
constexpr uint32_t kBlockBytes = 144;  // bytes per super-block
constexpr int kRowsPerWave = 2;
constexpr int kWavesPerGroup = 4;
constexpr int kMaxBatch = 4;  // input vectors one launch multiplies every weight with

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
    // compiles to v_cvt_f32_ubyte{0..3}: one instruction per byte
    return float((word >> (8 * byte)) & 0xFFu);
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
    if (row0 >= rows_total) return;

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
    // (one input vector: two groups, which is the whole row of a 4096-wide layer)
    constexpr int kGroups = kBatch == 1 ? 2 : 1;
    for (uint32_t ib0 = 0; ib0 < p.blocks_per_row; ib0 += 8 * kGroups) {
        bool live[kGroups];
        uint4v head[kGroups][kRowsPerWave], nib[kGroups][kRowsPerWave];
        float4v xlo[kGroups][kBatch][4], xhi[kGroups][kBatch][4];
#pragma unroll
        for (int gi = 0; gi < kGroups; gi++) {
            const uint32_t ib = ib0 + 8 * gi + blk_lane;
            live[gi] = ib < p.blocks_per_row;
            const uint32_t ibc = live[gi] ? ib : p.blocks_per_row - 1;
            // weights of all rows first: these are the loads that go to memory
#pragma unroll
            for (int r = 0; r < kRowsPerWave; r++) {
                const uint8_t* blk = wrow[r] + size_t(ibc) * kBlockBytes;
                head[gi][r] = __builtin_nontemporal_load(reinterpret_cast<const uint4v*>(blk));
                nib[gi][r] = __builtin_nontemporal_load(reinterpret_cast<const uint4v*>(blk + 16 + 16 * piece));
            }
            // the inputs: 16 + 16 floats per input vector
#pragma unroll
            for (int b = 0; b < kBatch; b++) {
                // (an input vector past the batch repeats the last one; its results are not stored)
                const float* xp = p.x + int64_t(min(uint32_t(b), p.batch - 1)) * p.x_stride + size_t(ibc) * kQK + col;
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    xlo[gi][b][i] = *reinterpret_cast<const float4v*>(xp + 4 * i);
                    xhi[gi][b][i] = *reinterpret_cast<const float4v*>(xp + 32 + 4 * i);
                }
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
                    const uint32_t lo = nib[gi][r][wd] & 0x0F0F0F0Fu;
                    const uint32_t hi = nib[gi][r][wd] & 0xF0F0F0F0u;  // 16 x the high nibbles
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

inline bool aligned16(const void* ptr) { return (reinterpret_cast<uintptr_t>(ptr) & 15u) == 0; }

}  // namespace

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
    // every launch multiplies the weights with up to kMaxBatch input vectors; a larger batch
    // streams the weights again per group of kMaxBatch (from the last-level cache when the
    // matrices fit it)
    for (uint32_t b0 = 0; b0 < batch; b0 += kMaxBatch) {
        const uint32_t nb = min(batch - b0, uint32_t(kMaxBatch));
        MatvecParams q = p;
        q.x = static_cast<const float*>(x) + int64_t(b0) * x_stride;
        q.x_stride = nb > 1 ? x_stride : 0;
        for (int i = 0; i < 3; i++)
            if (q.y[i]) q.y[i] += int64_t(b0) * q.y_stride[i];
        q.batch = nb;
        KernelTimerScope timer("matvec_q4k");
        if (nb == 1) matvec_q4k_kernel<1><<<grid, block, 0, st>>>(q);
        else if (nb == 2) matvec_q4k_kernel<2><<<grid, block, 0, st>>>(q);
        else matvec_q4k_kernel<4><<<grid, block, 0, st>>>(q);  // 3: the fourth vector repeats the third
        int rc = launch_status();
        if (rc != GRANITE_HIP_OK) return rc;
    }
    return GRANITE_HIP_OK;
}

}  // namespace ghip
