// Matrix-core rate under load: a measurement aid in a library of its own
// (libgranite_hip_calibration.so), not part of the attention path.
//
// Every wave keeps four A and four B operands of v_mfma_f32_32x32x16_f16 (or
// v_mfma_f32_16x16x32_f16) in registers and issues MFMAs on them back to back.  With
// all-zero operands the part holds its peak clock; with operands that look like data it is
// held back by its power limit.  The mix form adds, after every MFMA, what an attention
// inner loop issues beside it -- a few float FMAs, an exponential, a 16-byte LDS read per
// lane whose data feeds a later MFMA -- and so measures what the instruction mix itself
// leaves of the matrix cores, with no staging, no barriers and no loop bookkeeping.  The mix
// is given per pair of MFMAs, so that half an instruction per MFMA (an LDS operand that feeds
// two MFMAs) can be expressed, and may include scalar instructions.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "granite_hip_calibration.h"

namespace {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef float float4v __attribute__((ext_vector_type(4)));
typedef float float16v __attribute__((ext_vector_type(16)));
typedef uint32_t uint4v __attribute__((ext_vector_type(4)));
typedef uint32_t uint2v __attribute__((ext_vector_type(2)));

constexpr int kWave = 64;
constexpr uint32_t kLdsHalves = 16384;          // 32 KiB of operands in LDS for the mix form
constexpr size_t kLdsBytes = 100 * 1024;        // and enough LDS to keep one workgroup per CU

#define CAL_CHECK(expr)                                    \
    do {                                                   \
        hipError_t _e = (expr);                            \
        if (_e != hipSuccess) return static_cast<int>(_e); \
    } while (0)

// kWide: 32x32x16 (16 MFMAs a pass) or 16x16x32 (32 MFMAs a pass, the same flops).
// kFma, kExp, kLds, kSalu: instructions per PAIR of MFMAs; the first MFMA of a pair is followed
// by the larger half of each.
// kZeros only names the instantiation (all-zero operands), so that a kernel trace tells the two
// kinds of run apart; the code is the same.
template <bool kWide, int kFma, int kExp, int kLds, int kSalu, bool kZeros>
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
        // LDS operands: an odd count per pair makes the second MFMA's operand two 8-byte reads
        // (as a V^T operand is), the first one's a 16-byte read (as a K operand is); every byte
        // read feeds an MFMA.  Offsets are immediates; the base is re-declared every pass so
        // that the reads stay in the loop.
        uint32_t lds_base = lane * 16;  // 64 lanes x 16 bytes: every bank once
        const unsigned char* const lds_bytes = reinterpret_cast<const unsigned char*>(s_operands);
        uint32_t scalar = iterations;
        for (uint32_t it = 0; it < iterations; it++) {
            asm volatile("" : "+v"(lds_base));
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const bool second = r & 1;  // of the pair
                const half8 aa = kLds > 0 ? __builtin_bit_cast(half8, ld[r & 3]) : a[r & 3];
                c[r & 3] = __builtin_amdgcn_mfma_f32_32x32x16_f16(aa, b[(r + (r >> 2)) & 3], c[r & 3], 0, 0, 0);
                const int reads = second ? kLds / 2 : (kLds + 1) / 2;  // issued now, used two MFMAs on
                if (reads == 1) {
                    ld[(r + 2) & 3] = *reinterpret_cast<const uint4v*>(lds_bytes + lds_base + 1024 * (r & 15));
                } else if (reads == 2) {
                    const uint2v lo = *reinterpret_cast<const uint2v*>(lds_bytes + lds_base + 1024 * (r & 15));
                    const uint2v hi = *reinterpret_cast<const uint2v*>(lds_bytes + lds_base + 1024 * ((r + 5) & 15) + 8);
                    ld[(r + 2) & 3] = uint4v{lo.x, lo.y, hi.x, hi.y};
                }
#pragma unroll
                for (int j = 0; j < (second ? kFma / 2 : (kFma + 1) / 2); j++)
                    x[(r + j) & 7] = __builtin_fmaf(x[(r + j) & 7], 0.999f, 0.001f);
#pragma unroll
                for (int j = 0; j < (second ? kExp / 2 : (kExp + 1) / 2); j++)
                    e[(r + j) & 3] = __builtin_amdgcn_exp2f(-e[(r + j) & 3]);  // stays in [0.5, 1]
#pragma unroll
                for (int j = 0; j < (second ? kSalu / 2 : (kSalu + 1) / 2); j++)
                    asm volatile("s_add_u32 %0, %0, 3" : "+s"(scalar));
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        total += float(scalar & 1);
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

template <bool kWide, int kFma, int kExp, int kLds, int kSalu, bool kZeros = false>
int run(const uint4v* operands, uint32_t n_vec, uint32_t iterations, uint32_t workgroups, uint32_t threads,
        float* sink, float* milliseconds) {
    auto kernel = mfma_rate_kernel<kWide, kFma, kExp, kLds, kSalu, kZeros>;
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

extern "C" int granite_hip_cal_mfma_mix(int device, const void* operands_f16, uint64_t n_halves,
                                        uint32_t iterations, int shape, int waves_per_simd,
                                        int fma_per_pair, int exp_per_pair, int lds_reads_per_pair,
                                        int salu_per_pair, double* flops, float* milliseconds) {
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
    const int mix = fma_per_pair * 1000 + exp_per_pair * 100 + lds_reads_per_pair * 10 + salu_per_pair;
    // all-zero operands get an instantiation of their own (same code, another name in a trace)
    bool zeros = true;
    {
        uint32_t head[1024];
        CAL_CHECK(hipMemcpy(head, operands_f16, sizeof(head), hipMemcpyDeviceToHost));
        for (uint32_t w : head) zeros = zeros && w == 0;
    }
    int rc = -1;
#define GHIP_CAL_MIX(f, e, l, sa)                                                                          \
    if (shape == 32 && mix == (f) * 1000 + (e) * 100 + (l) * 10 + (sa))                                    \
        rc = run<true, f, e, l, sa>(ops, n_vec, iterations, workgroups, threads, sink, milliseconds);
    if (shape == 16 && mix == 0)
        rc = zeros ? run<false, 0, 0, 0, 0, true>(ops, n_vec, iterations, workgroups, threads, sink, milliseconds)
                   : run<false, 0, 0, 0, 0>(ops, n_vec, iterations, workgroups, threads, sink, milliseconds);
    if (shape == 32 && mix == 0 && zeros)
        rc = run<true, 0, 0, 0, 0, true>(ops, n_vec, iterations, workgroups, threads, sink, milliseconds);
    else
    GHIP_CAL_MIX(0, 0, 0, 0)
    GHIP_CAL_MIX(8, 0, 0, 0)   // 4 float FMAs per MFMA
    GHIP_CAL_MIX(16, 0, 0, 0)  // 8
    GHIP_CAL_MIX(0, 2, 0, 0)   // 1 exponential
    GHIP_CAL_MIX(6, 2, 0, 0)   // 3 FMAs + 1 exponential
    GHIP_CAL_MIX(0, 0, 2, 0)   // 1 LDS read
    GHIP_CAL_MIX(6, 2, 2, 0)   // 3 FMAs + 1 exponential + 1 LDS read
    GHIP_CAL_MIX(6, 2, 1, 0)   // ... + half an LDS read (an operand feeding two MFMAs)
    GHIP_CAL_MIX(6, 2, 3, 0)   // 3 FMAs + 1 exponential + 1.5 LDS reads (a K operand, a V^T operand as two)
    GHIP_CAL_MIX(6, 2, 3, 4)   // what attention_tiles_dma_kernel issues: 3 + 1 vector, 1.5 LDS, 2 scalar
    GHIP_CAL_MIX(8, 2, 3, 6)   // what attention_tiles_kernel issues: 4 + 1 vector, 1.5 LDS, 3 scalar
    GHIP_CAL_MIX(7, 2, 1, 2)   // a 64-rows-per-wave form: 3.5 + 1 vector, 0.5 LDS, 1 scalar
#undef GHIP_CAL_MIX
    (void)hipFree(sink);
    // 16 MFMAs of 2 * 32 * 32 * 16 flops (or 32 of half that) per pass and wave
    *flops = double(workgroups) * (threads / kWave) * double(iterations) * 16.0 * 2.0 * 32 * 32 * 16;
    return rc;
}

extern "C" int granite_hip_cal_mfma_rate(int device, const void* operands_f16, uint64_t n_halves,
                                         uint32_t iterations, int shape, int waves_per_simd,
                                         int fma_per_mfma, int exp_per_mfma, int lds_reads_per_mfma,
                                         double* flops, float* milliseconds) {
    return granite_hip_cal_mfma_mix(device, operands_f16, n_halves, iterations, shape, waves_per_simd,
                                    2 * fma_per_mfma, 2 * exp_per_mfma, 2 * lds_reads_per_mfma, 0, flops,
                                    milliseconds);
}
