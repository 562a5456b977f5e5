// Matrix-core rate under load: a measurement aid, not part of the attention path.
//
// Every wave keeps four A and four B operands of v_mfma_f32_32x32x16_f16 (or
// v_mfma_f32_16x16x32_f16) in registers and issues MFMAs on them back to back, so nothing
// but the matrix cores and the register file is busy.  With all-zero operands the part
// holds its peak clock; with operands that look like data it is held back by its power
// limit, and the rate it then reaches, not the published peak, is what a kernel that also
// has to feed the matrix cores can be compared with.  The operands are the caller's: 16
// halves per lane, lane i of the grid reading halves [16 i, 16 i + 16) modulo the buffer.
#include "common.h"

namespace ghip {
namespace {

constexpr int kCalWaves = 8;  // two waves per SIMD, as the attention kernel runs

template <bool kWide>
__global__ void __launch_bounds__(kCalWaves* kWave)
    mfma_rate_kernel(const uint4v* __restrict__ operands, uint32_t n_vec, uint32_t iterations,
                     float* sink) {
    const uint32_t lane_id = blockIdx.x * blockDim.x + threadIdx.x;
    half8 a[4], b[4];
#pragma unroll
    for (uint32_t i = 0; i < 4; i++) {
        a[i] = __builtin_bit_cast(half8, operands[(lane_id * 8 + i) % n_vec]);
        b[i] = __builtin_bit_cast(half8, operands[(lane_id * 8 + 4 + i) % n_vec]);
    }
    // All operands in registers and the workgroup's waves in step before the loop: waves
    // that enter it at scattered times have been measured up to 30 % slower for its whole
    // length, and differently from launch to launch.
#pragma unroll
    for (int i = 0; i < 4; i++) asm volatile("" : "+v"(a[i]), "+v"(b[i]));
    __syncthreads();
    float total = 0.0f;
    if constexpr (kWide) {  // 16 MFMAs of 32x32x16 per pass
        float16v c[4];
#pragma unroll
        for (int i = 0; i < 4; i++)
#pragma unroll
            for (int r = 0; r < 16; r++) c[i][r] = 0.0f;
        for (uint32_t it = 0; it < iterations; it++) {
#pragma unroll
            for (int i = 0; i < 4; i++)
#pragma unroll
                for (int j = 0; j < 4; j++)
                    c[i] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[j], b[(i + j) & 3], c[i], 0, 0, 0);
        }
#pragma unroll
        for (int i = 0; i < 4; i++)
#pragma unroll
            for (int r = 0; r < 16; r++) total += c[i][r];
    } else {  // 32 MFMAs of 16x16x32 per pass: the same number of flops
        float4v c[8];
#pragma unroll
        for (int i = 0; i < 8; i++) c[i] = float4v{0.0f, 0.0f, 0.0f, 0.0f};
        for (uint32_t it = 0; it < iterations; it++) {
#pragma unroll
            for (int j = 0; j < 4; j++)
#pragma unroll
                for (int i = 0; i < 8; i++)
                    c[i] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[j], b[(i + j) & 3], c[i], 0, 0, 0);
        }
#pragma unroll
        for (int i = 0; i < 8; i++) total += c[i].x + c[i].y + c[i].z + c[i].w;
    }
    if (total == 1.2345e-30f) sink[0] = total;  // keeps the loop alive; practically never taken
}

}  // namespace

int launch_mfma_rate(const void* operands, uint64_t n_halves, uint32_t iterations, int shape,
                     double* flops) {
    if (!operands) return GRANITE_HIP_ENULL;
    if (n_halves < 8 || n_halves % 8 != 0 || n_halves / 8 > 0xFFFFFFFFull) return GRANITE_HIP_EINVAL;
    if (iterations == 0 || iterations > (1u << 20)) return GRANITE_HIP_EINVAL;
    if (shape != 16 && shape != 32) return GRANITE_HIP_EINVAL;
    if (int rc = ensure_workspace(sizeof(float)); rc != GRANITE_HIP_OK) return rc;
    float* sink = static_cast<float*>(ctx().workspace);
    const uint32_t workgroups = 2 * uint32_t(ctx().compute_units);  // two rounds of one per CU
    const dim3 grid(workgroups), block(kCalWaves * kWave);
    {
        KernelTimerScope timer("mfma_rate");
        if (shape == 32)
            mfma_rate_kernel<true><<<grid, block, 0, ctx().stream>>>(
                static_cast<const uint4v*>(operands), uint32_t(n_halves / 8), iterations, sink);
        else
            mfma_rate_kernel<false><<<grid, block, 0, ctx().stream>>>(
                static_cast<const uint4v*>(operands), uint32_t(n_halves / 8), iterations, sink);
    }
    if (flops)  // 16 MFMAs of 2 * 32 * 32 * 16 flops per pass and wave
        *flops = double(workgroups) * kCalWaves * double(iterations) * 16.0 * 2.0 * 32 * 32 * 16;
    return launch_status();
}

}  // namespace ghip
