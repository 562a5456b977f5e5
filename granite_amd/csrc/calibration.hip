// Matrix-core rate under load: a measurement aid in a library of its own
// (libgranite_hip_calibration.so), not part of the attention path.
//
// Every wave keeps four A and four B operands of v_mfma_f32_32x32x16_f16 (or
// v_mfma_f32_16x16x32_f16) in registers and issues MFMAs on them back to back.  With
// all-zero operands the part holds its peak clock; with operands that look like data it is
// held back by its power limit.  The mix form adds, after every MFMA, what an attention
// inner loop issues beside it -- a few float FMAs, an exponential, a 16-byte LDS read per
// lane whose data feeds a later MFMA -- and so measures what the instruction mix itself
// leaves of the matrix cores, with no staging, no barriers and no loop bookkeeping.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "granite_hip_calibration.h"

namespace {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef float float4v __attribute__((ext_vector_type(4)));
typedef float float16v __attribute__((ext_vector_type(16)));
typedef uint32_t uint4v __attribute__((ext_vector_type(4)));

constexpr int kWave = 64;
constexpr uint32_t kLdsHalves = 16384;          // 32 KiB of operands in LDS for the mix form
constexpr size_t kLdsBytes = 100 * 1024;        // and enough LDS to keep one workgroup per CU

#define CAL_CHECK(expr)                                    \
    do {                                                   \
        hipError_t _e = (expr);                            \
        if (_e != hipSuccess) return static_cast<int>(_e); \
    } while (0)

// kWide: 32x32x16 (16 MFMAs a pass) or 16x16x32 (32 MFMAs a pass, the same flops).
template <bool kWide, int kFma, int kExp, int kLds>
__global__ void __launch_bounds__(512, 1)
    mfma_rate_kernel(const uint4v* __restrict__ operands, uint32_t n_vec, uint32_t iterations,
                     float* sink) {
    extern __shared__ __attribute__((aligned(16))) uint4v s_operands[];
    const uint32_t lane_id = blockIdx.x * blockDim.x + threadIdx.x;
    const uint32_t lane = threadIdx.x & 63;
    if constexpr (kLds > 0) {
        for (uint32_t i = threadIdx.x; i < kLdsHalves / 8; i += blockDim.x) s_operands[i] = operands[i % n_vec];
    }
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
    if constexpr (kWide) {
        float16v c[4];
#pragma unroll
        for (int i = 0; i < 4; i++)
#pragma unroll
            for (int r = 0; r < 16; r++) c[i][r] = 0.0f;
        float x[8], e[4];
#pragma unroll
        for (int i = 0; i < 8; i++) x[i] = float(a[i & 3][i]) * 0.01f;
#pragma unroll
        for (int i = 0; i < 4; i++) e[i] = 0.1f * float(i + 1);
        uint4v ld[4];
#pragma unroll
        for (int i = 0; i < 4; i++) ld[i] = __builtin_bit_cast(uint4v, a[i]);
        const uint4v* lp = s_operands + lane;  // 64 lanes x 16 bytes: every bank once
        for (uint32_t it = 0; it < iterations; it++) {
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const half8 aa = kLds > 0 ? __builtin_bit_cast(half8, ld[r & 3]) : a[r & 3];
                c[r & 3] = __builtin_amdgcn_mfma_f32_32x32x16_f16(aa, b[(r + (r >> 2)) & 3], c[r & 3], 0, 0, 0);
#pragma unroll
                for (int j = 0; j < kLds; j++) ld[(r + 2) & 3] = lp[64 * ((r + j + it) & 15)];  // used two MFMAs on
#pragma unroll
                for (int j = 0; j < kFma; j++) x[(r + j) & 7] = __builtin_fmaf(x[(r + j) & 7], 0.999f, 0.001f);
#pragma unroll
                for (int j = 0; j < kExp; j++) e[(r + j) & 3] = __builtin_amdgcn_exp2f(e[(r + j) & 3] * 0.5f);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
#pragma unroll
        for (int i = 0; i < 4; i++)
#pragma unroll
            for (int r = 0; r < 16; r++) total += c[i][r];
#pragma unroll
        for (int i = 0; i < 8; i++) total += x[i];
#pragma unroll
        for (int i = 0; i < 4; i++) total += e[i] + __builtin_bit_cast(float, ld[i].x);
    } else {
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

template <bool kWide, int kFma, int kExp, int kLds>
int run(const uint4v* operands, uint32_t n_vec, uint32_t iterations, uint32_t workgroups, uint32_t threads,
        float* sink, float* milliseconds) {
    auto kernel = mfma_rate_kernel<kWide, kFma, kExp, kLds>;
    CAL_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                  hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(kLdsBytes)));
    hipEvent_t start, stop;
    CAL_CHECK(hipEventCreate(&start));
    CAL_CHECK(hipEventCreate(&stop));
    for (int warm = 0; warm < 3; warm++) kernel<<<workgroups, threads, kLdsBytes>>>(operands, n_vec, iterations, sink);
    CAL_CHECK(hipDeviceSynchronize());
    CAL_CHECK(hipEventRecord(start));
    kernel<<<workgroups, threads, kLdsBytes>>>(operands, n_vec, iterations, sink);
    CAL_CHECK(hipEventRecord(stop));
    CAL_CHECK(hipEventSynchronize(stop));
    CAL_CHECK(hipEventElapsedTime(milliseconds, start, stop));
    (void)hipEventDestroy(start);
    (void)hipEventDestroy(stop);
    return static_cast<int>(hipGetLastError());
}

}  // namespace

extern "C" int granite_hip_cal_mfma_rate(int device, const void* operands_f16, uint64_t n_halves,
                                         uint32_t iterations, int shape, int waves_per_simd,
                                         int fma_per_mfma, int exp_per_mfma, int lds_reads_per_mfma,
                                         double* flops, float* milliseconds) {
    if (!operands_f16 || !flops || !milliseconds) return -1;
    if (n_halves < kLdsHalves || n_halves % 8 != 0 || n_halves / 8 > 0xFFFFFFFFull) return -1;
    if (iterations == 0 || iterations > (1u << 20)) return -1;
    if (waves_per_simd != 1 && waves_per_simd != 2) return -1;
    CAL_CHECK(hipSetDevice(device));
    hipDeviceProp_t prop;
    CAL_CHECK(hipGetDeviceProperties(&prop, device));
    const uint32_t workgroups = uint32_t(prop.multiProcessorCount);
    const uint32_t threads = 4 * kWave * uint32_t(waves_per_simd);
    float* sink = nullptr;
    CAL_CHECK(hipMalloc(&sink, 256));
    const auto* ops = static_cast<const uint4v*>(operands_f16);
    const uint32_t n_vec = uint32_t(n_halves / 8);
    const int mix = fma_per_mfma * 100 + exp_per_mfma * 10 + lds_reads_per_mfma;
    int rc = -1;
    if (shape == 16 && mix == 0) rc = run<false, 0, 0, 0>(ops, n_vec, iterations, workgroups, threads, sink, milliseconds);
    if (shape == 32 && mix == 0) rc = run<true, 0, 0, 0>(ops, n_vec, iterations, workgroups, threads, sink, milliseconds);
    if (shape == 32 && mix == 400) rc = run<true, 4, 0, 0>(ops, n_vec, iterations, workgroups, threads, sink, milliseconds);
    if (shape == 32 && mix == 800) rc = run<true, 8, 0, 0>(ops, n_vec, iterations, workgroups, threads, sink, milliseconds);
    if (shape == 32 && mix == 10) rc = run<true, 0, 1, 0>(ops, n_vec, iterations, workgroups, threads, sink, milliseconds);
    if (shape == 32 && mix == 310) rc = run<true, 3, 1, 0>(ops, n_vec, iterations, workgroups, threads, sink, milliseconds);
    if (shape == 32 && mix == 1) rc = run<true, 0, 0, 1>(ops, n_vec, iterations, workgroups, threads, sink, milliseconds);
    if (shape == 32 && mix == 311) rc = run<true, 3, 1, 1>(ops, n_vec, iterations, workgroups, threads, sink, milliseconds);
    (void)hipFree(sink);
    // 16 MFMAs of 2 * 32 * 32 * 16 flops (or 32 of half that) per pass and wave
    *flops = double(workgroups) * (threads / kWave) * double(iterations) * 16.0 * 2.0 * 32 * 32 * 16;
    return rc;
}
