// Shared declarations of the gfx950 attention library: launch-side context,
// error helpers and the small device utilities every kernel file uses.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "granite_hip.h"

namespace ghip {

constexpr int kHeadDim = 128;  // the largest head size the attention kernels are instantiated for (64 is the other)
constexpr int kWave = 64;      // CDNA wavefront

// Process-wide launch context (one in-order stream, one scratch buffer).
struct Context {
    bool initialized = false;
    int device = 0;
    hipStream_t own_stream = nullptr;
    hipStream_t stream = nullptr;  // the stream launches go to
    void* workspace = nullptr;     // split-K partials, tree masks
    size_t workspace_bytes = 0;
    int compute_units = 0;
};

Context& ctx();

// Grows the scratch buffer to at least `bytes`.  Growing waits for the whole
// device first (launches on any stream may still use the old buffer), frees
// and allocates; callers that must not stall reserve once up front
// (granite_hip_reserve_workspace) or bring their own scratch.
int ensure_workspace(size_t bytes);

// Where a launch takes its scratch memory (split-K partials, plans, tree masks) from.
//   default            the library workspace, grown when too small
//   fixed != nullptr   that buffer and nothing else: no allocation, no synchronisation;
//                      a launch that needs more fails with GRANITE_HIP_ESCRATCH
//   query != nullptr   nothing is launched; *query receives the bytes the launch needs
struct ScratchSource {
    void* fixed = nullptr;
    size_t fixed_bytes = 0;
    size_t* query = nullptr;
};

// Resolves `need` bytes against `src`.  Returns GRANITE_HIP_OK with *ws set (nullptr for a
// query, in which case the caller returns at once), or an error code.
int take_scratch(const ScratchSource& src, size_t need, void** ws);

#define GHIP_CHECK(expr)                               \
    do {                                               \
        hipError_t _e = (expr);                        \
        if (_e != hipSuccess) return static_cast<int>(_e); \
    } while (0)

#define GHIP_REQUIRE_INIT()                                   \
    do {                                                      \
        if (!::ghip::ctx().initialized) return GRANITE_HIP_ENOTINIT; \
    } while (0)

// Per-kernel GPU timing (MetalCompute::enable_kernel_timing analogue,
// src/backend/metal/metal_compute.mm:1021-1108).  When enabled, every launch is
// bracketed by two events on the launch stream; the pairs are resolved into a
// name -> (milliseconds, dispatches) table when the statistics are read.
struct KernelTimerScope {
    explicit KernelTimerScope(const char* name);
    ~KernelTimerScope();
    KernelTimerScope(const KernelTimerScope&) = delete;
    KernelTimerScope& operator=(const KernelTimerScope&) = delete;

  private:
    const char* name_;
    hipEvent_t start_ = nullptr;
};

// While one of these lives, KernelTimerScope records nothing (and so creates no events).
struct TimingSuppressed {
    TimingSuppressed();
    ~TimingSuppressed();
    TimingSuppressed(const TimingSuppressed&) = delete;
    TimingSuppressed& operator=(const TimingSuppressed&) = delete;

  private:
    bool was_;
};

// Kernels whose dynamic LDS exceeds the 64 KiB default need their limit raised once per
// device (the attribute belongs to the function on one device).  `done` is the caller's
// static flag array, one per kernel instantiation.
constexpr int kMaxDevices = 64;
inline int raise_dynamic_lds_limit(const void* kernel, size_t bytes, bool (&done)[kMaxDevices]) {
    const int dev = ctx().device;
    if (dev < 0 || dev >= kMaxDevices) return GRANITE_HIP_EINVAL;
    if (!done[dev]) {
        GHIP_CHECK(hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(bytes)));
        done[dev] = true;
    }
    return GRANITE_HIP_OK;
}

inline int launch_status() {
    hipError_t e = hipGetLastError();
    return e == hipSuccess ? GRANITE_HIP_OK : static_cast<int>(e);
}

// ---- launchers implemented in the kernel files -------------------------
int launch_kv_append_contig(void* cache_k, void* cache_v, const void* new_k, const void* new_v,
                            int src_dtype, int64_t src_tok_stride, int64_t src_head_stride,
                            uint32_t num_kv_heads, uint32_t head_dim, uint32_t current_len,
                            uint32_t new_len, uint32_t max_seq_len, int rounding,
                            const int32_t* src_index = nullptr, uint32_t src_tokens = 0);
int launch_kv_append_paged(const void* new_k, const void* new_v, int src_dtype,
                           int64_t src_tok_stride, int64_t src_head_stride, void* k_cache,
                           void* v_cache, const int32_t* block_table, uint32_t num_kv_heads,
                           uint32_t head_dim, uint32_t start_pos, uint32_t new_len,
                           uint32_t block_size, int rounding, const int32_t* src_index = nullptr,
                           uint32_t src_tokens = 0);
int launch_kv_gather_paged(void* dst_k, void* dst_v, const void* k_cache, const void* v_cache,
                           const int32_t* block_table, uint32_t num_kv_heads, uint32_t head_dim,
                           uint32_t len, uint32_t block_size, uint32_t max_seq_len);
int launch_copy_rows(void* dst, int64_t dst_row_bytes, const void* src, int64_t src_row_bytes, uint64_t rows,
                     uint32_t copy_bytes, uint32_t fill_bytes);
int launch_decode(const granite_hip_decode_args& a, const ScratchSource& scratch = {});
int launch_attention(const granite_hip_attention_args& a, const ScratchSource& scratch = {});
int launch_tree_mask(const int32_t* parents, uint32_t* mask_words, uint32_t num_nodes);
int launch_rope_append(const granite_hip_rope_args& a);
size_t matvec_q4k_scratch_bytes(uint32_t K, uint64_t rows, uint32_t batch);
int launch_matvec_q4k(const void* x, int64_t x_stride, const void* const w[3], void* const y[3],
                      const int64_t y_stride[3], const uint32_t n[3], uint32_t K, uint32_t batch);

// ---- device helpers ------------------------------------------------------
#if defined(__HIPCC__)

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half4 __attribute__((ext_vector_type(4)));
typedef _Float16 half2v __attribute__((ext_vector_type(2)));
typedef float float2v __attribute__((ext_vector_type(2)));
typedef float float4v __attribute__((ext_vector_type(4)));
typedef float float16v __attribute__((ext_vector_type(16)));
typedef uint32_t uint4v __attribute__((ext_vector_type(4)));
typedef uint32_t uint2v __attribute__((ext_vector_type(2)));
typedef short short4v __attribute__((ext_vector_type(4)));
typedef short short8v __attribute__((ext_vector_type(8)));

// Granite's truncating float->half (src/llm/math_ops.cpp:45-54), bit for bit.
__device__ __forceinline__ uint16_t f32_to_f16_truncate(float f) {
    uint32_t bits = __float_as_uint(f);
    uint32_t sign = (bits >> 16) & 0x8000u;
    int32_t e = static_cast<int32_t>((bits >> 23) & 0xFFu) - 127 + 15;
    uint32_t mant = (bits >> 13) & 0x3FFu;
    if (e <= 0) return static_cast<uint16_t>(sign);
    if (e >= 31) return static_cast<uint16_t>(sign | 0x7C00u);
    return static_cast<uint16_t>(sign | (static_cast<uint32_t>(e) << 10) | mant);
}

// Round-to-nearest-even float->half, what Metal's half(x) does.
__device__ __forceinline__ uint16_t f32_to_f16_nearest(float f) {
    _Float16 h = static_cast<_Float16>(f);
    return __builtin_bit_cast(uint16_t, h);
}

__device__ __forceinline__ uint32_t pack_f16x2(float lo, float hi) {
    half2v v;
    v.x = static_cast<_Float16>(lo);
    v.y = static_cast<_Float16>(hi);
    return __builtin_bit_cast(uint32_t, v);
}

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

__device__ __forceinline__ float wave_shfl_xor(float v, int mask) {
    return __shfl_xor(v, mask, kWave);
}

// The values of lanes l and l ^ 32 side by side, through v_permlane32_swap (one vector
// instruction, no LDS round trip): .lo is the value held by the lane's copy in lanes
// 0..31, .hi that of its copy in lanes 32..63; both lanes see the same pair.  Written as
// inline assembly because the compiler builtin loses the second result when both
// operands carry the same value.  The s_nop covers the two wait states the instruction
// needs after a vector write to its operands.
struct LanePair {
    float lo, hi;
};
__device__ __forceinline__ LanePair half_wave_pair(float v) {
    float a = v, b = v;
    asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1" : "+v"(a), "+v"(b));
    return LanePair{a, b};
}

#endif  // __HIPCC__

}  // namespace ghip
