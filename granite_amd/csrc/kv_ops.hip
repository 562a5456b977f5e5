// KV-cache append and gather kernels (byte/bit work, HBM bound).
//
// Replaces, on gfx950:
//   kv_cache_append_f16      src/backend/metal/kernels/metal_shaders_attention.h:102-125
//   paged_kv_cache_append    metal_shaders_attention.h:2142-2176
//   KVCache::append          src/llm/kv_cache.cpp:55-107 (half source, bit copy)
//   the per-call cache gather of src/llm/transformer.mm:1750-1763
//
// One thread moves 8 consecutive elements of one (token, head) row: a 16-byte
// store (and one 16-byte or two 16-byte loads), consecutive threads cover a
// row, so every 256-byte destination row is written by 16 adjacent lanes.
// K and V go in one launch (blockIdx.y selects).
#include <algorithm>

#include "common.h"

namespace ghip {
namespace {

constexpr int kVec = 8;

template <bool kNearest>
__device__ __forceinline__ uint16_t cvt(float f) {
    return kNearest ? f32_to_f16_nearest(f) : f32_to_f16_truncate(f);
}

template <typename SrcT, bool kNearest>
__device__ __forceinline__ uint4v load8_as_half(const SrcT* p);

template <>
__device__ __forceinline__ uint4v load8_as_half<uint16_t, false>(const uint16_t* p) {
    return *reinterpret_cast<const uint4v*>(p);
}
template <>
__device__ __forceinline__ uint4v load8_as_half<uint16_t, true>(const uint16_t* p) {
    return *reinterpret_cast<const uint4v*>(p);
}
template <>
__device__ __forceinline__ uint4v load8_as_half<float, false>(const float* p) {
    float4v a = *reinterpret_cast<const float4v*>(p);
    float4v b = *reinterpret_cast<const float4v*>(p + 4);
    uint4v r;
    r.x = cvt<false>(a.x) | (uint32_t(cvt<false>(a.y)) << 16);
    r.y = cvt<false>(a.z) | (uint32_t(cvt<false>(a.w)) << 16);
    r.z = cvt<false>(b.x) | (uint32_t(cvt<false>(b.y)) << 16);
    r.w = cvt<false>(b.z) | (uint32_t(cvt<false>(b.w)) << 16);
    return r;
}
template <>
__device__ __forceinline__ uint4v load8_as_half<float, true>(const float* p) {
    float4v a = *reinterpret_cast<const float4v*>(p);
    float4v b = *reinterpret_cast<const float4v*>(p + 4);
    uint4v r;
    r.x = cvt<true>(a.x) | (uint32_t(cvt<true>(a.y)) << 16);
    r.y = cvt<true>(a.z) | (uint32_t(cvt<true>(a.w)) << 16);
    r.z = cvt<true>(b.x) | (uint32_t(cvt<true>(b.y)) << 16);
    r.w = cvt<true>(b.z) | (uint32_t(cvt<true>(b.w)) << 16);
    return r;
}

struct AppendParams {
    const void* src[2];
    uint16_t* dst[2];
    const int32_t* table;  // nullptr: contiguous cache
    const int32_t* src_index;  // nullptr, or: new token s is source token src_index[s] (out of
                               // [0, src_tokens): the token is skipped)
    uint32_t src_tokens;
    int64_t src_tok_stride, src_head_stride;
    uint32_t num_kv_heads, head_dim, first_pos, new_len;
    uint32_t max_seq;     // contiguous
    uint32_t block_size;  // paged
};

// Destination element offset of (logical position pos, head h).
__device__ __forceinline__ size_t dst_row_offset(const AppendParams& p, uint32_t pos, uint32_t h) {
    if (p.table) {
        size_t row = size_t(p.table[pos / p.block_size]) * p.block_size + pos % p.block_size;
        return (row * p.num_kv_heads + h) * p.head_dim;
    }
    return (size_t(h) * p.max_seq + pos) * p.head_dim;
}

template <typename SrcT, bool kNearest>
__global__ void __launch_bounds__(256) kv_append_vec_kernel(AppendParams p) {
    const uint32_t vec_per_row = p.head_dim / kVec;
    const uint32_t total = p.new_len * p.num_kv_heads * vec_per_row;
    const int which = blockIdx.y;
    const SrcT* src = static_cast<const SrcT*>(p.src[which]);
    uint16_t* dst = p.dst[which];
    for (uint32_t i = blockIdx.x * blockDim.x + threadIdx.x; i < total;
         i += gridDim.x * blockDim.x) {
        uint32_t v = i % vec_per_row;
        uint32_t rest = i / vec_per_row;
        uint32_t s, h;
        if (p.table) {  // pool rows hold all heads of a token side by side
            h = rest % p.num_kv_heads;
            s = rest / p.num_kv_heads;
        } else {  // cache rows of one head are contiguous over tokens
            s = rest % p.new_len;
            h = rest / p.new_len;
        }
        uint32_t s_src = s;
        if (p.src_index) {
            const int32_t picked = p.src_index[s];
            if (picked < 0 || uint32_t(picked) >= p.src_tokens) continue;
            s_src = uint32_t(picked);
        }
        const SrcT* sp = src + int64_t(s_src) * p.src_tok_stride + int64_t(h) * p.src_head_stride +
                         v * kVec;
        uint4v val = load8_as_half<SrcT, kNearest>(sp);
        *reinterpret_cast<uint4v*>(dst + dst_row_offset(p, p.first_pos + s, h) + v * kVec) = val;
    }
}

// Element-at-a-time form for sources that are not 16-byte aligned or head
// sizes that are not a multiple of 8.
template <typename SrcT, bool kNearest>
__global__ void __launch_bounds__(256) kv_append_scalar_kernel(AppendParams p) {
    const uint32_t total = p.new_len * p.num_kv_heads * p.head_dim;
    const int which = blockIdx.y;
    const SrcT* src = static_cast<const SrcT*>(p.src[which]);
    uint16_t* dst = p.dst[which];
    for (uint32_t i = blockIdx.x * blockDim.x + threadIdx.x; i < total;
         i += gridDim.x * blockDim.x) {
        uint32_t d = i % p.head_dim;
        uint32_t rest = i / p.head_dim;
        uint32_t h = rest % p.num_kv_heads;
        uint32_t s = rest / p.num_kv_heads;
        uint32_t s_src = s;
        if (p.src_index) {
            const int32_t picked = p.src_index[s];
            if (picked < 0 || uint32_t(picked) >= p.src_tokens) continue;
            s_src = uint32_t(picked);
        }
        SrcT x = src[int64_t(s_src) * p.src_tok_stride + int64_t(h) * p.src_head_stride + d];
        uint16_t hbits;
        if constexpr (sizeof(SrcT) == 2) {
            hbits = x;
        } else {
            hbits = cvt<kNearest>(x);
        }
        dst[dst_row_offset(p, p.first_pos + s, h) + d] = hbits;
    }
}

struct GatherParams {
    const uint16_t* src[2];
    uint16_t* dst[2];
    const int32_t* table;
    uint32_t num_kv_heads, head_dim, len, block_size, max_seq;
};

__global__ void __launch_bounds__(256) kv_gather_kernel(GatherParams p) {
    const uint32_t vec_per_row = p.head_dim / kVec;
    const uint32_t total = p.len * p.num_kv_heads * vec_per_row;
    const int which = blockIdx.y;
    for (uint32_t i = blockIdx.x * blockDim.x + threadIdx.x; i < total;
         i += gridDim.x * blockDim.x) {
        uint32_t v = i % vec_per_row;
        uint32_t rest = i / vec_per_row;
        uint32_t h = rest % p.num_kv_heads;
        uint32_t s = rest / p.num_kv_heads;
        size_t row = size_t(p.table[s / p.block_size]) * p.block_size + s % p.block_size;
        const uint16_t* sp = p.src[which] + (row * p.num_kv_heads + h) * p.head_dim + v * kVec;
        uint16_t* dp = p.dst[which] + (size_t(h) * p.max_seq + s) * p.head_dim + v * kVec;
        // the pool rows are read once (streaming load: 12 % faster on a 256 MiB gather); the
        // gathered cache stays cacheable for whoever reads it next
        *reinterpret_cast<uint4v*>(dp) =
            __builtin_nontemporal_load(reinterpret_cast<const uint4v*>(sp));
    }
}

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

template <typename SrcT>
int launch_append_typed(const AppendParams& p, int rounding) {
    const size_t esz = sizeof(SrcT);
    const bool vec = p.head_dim % kVec == 0 && aligned16(p.src[0]) && aligned16(p.src[1]) &&
                     aligned16(p.dst[0]) && aligned16(p.dst[1]) &&
                     (p.src_tok_stride * esz) % 16 == 0 && (p.src_head_stride * esz) % 16 == 0;
    const uint64_t elems = uint64_t(p.new_len) * p.num_kv_heads * p.head_dim;
    if (elems >= (1ull << 32)) return GRANITE_HIP_EINVAL;
    const uint64_t work = vec ? elems / kVec : elems;
    uint32_t blocks = static_cast<uint32_t>((work + 255) / 256);
    if (blocks > 65535u * 4) blocks = 65535u * 4;
    dim3 grid(blocks, 2), block(256);
    hipStream_t st = ctx().stream;
    KernelTimerScope timer("kv_append");
    if (vec) {
        if (rounding == GRANITE_HIP_ROUND_NEAREST)
            kv_append_vec_kernel<SrcT, true><<<grid, block, 0, st>>>(p);
        else
            kv_append_vec_kernel<SrcT, false><<<grid, block, 0, st>>>(p);
    } else {
        if (rounding == GRANITE_HIP_ROUND_NEAREST)
            kv_append_scalar_kernel<SrcT, true><<<grid, block, 0, st>>>(p);
        else
            kv_append_scalar_kernel<SrcT, false><<<grid, block, 0, st>>>(p);
    }
    return launch_status();
}

int launch_append(const AppendParams& p, int src_dtype, int rounding) {
    if (!p.src[0] || !p.src[1] || !p.dst[0] || !p.dst[1]) return GRANITE_HIP_ENULL;
    if (p.num_kv_heads == 0 || p.head_dim == 0) return GRANITE_HIP_EINVAL;
    if (rounding != GRANITE_HIP_ROUND_TRUNCATE && rounding != GRANITE_HIP_ROUND_NEAREST)
        return GRANITE_HIP_EINVAL;
    if (p.new_len == 0) return GRANITE_HIP_OK;
    if (src_dtype == GRANITE_HIP_F32) return launch_append_typed<float>(p, rounding);
    if (src_dtype == GRANITE_HIP_F16) return launch_append_typed<uint16_t>(p, rounding);
    return GRANITE_HIP_EINVAL;
}

}  // namespace

int launch_kv_append_contig(void* cache_k, void* cache_v, const void* new_k, const void* new_v,
                            int src_dtype, int64_t src_tok_stride, int64_t src_head_stride,
                            uint32_t num_kv_heads, uint32_t head_dim, uint32_t current_len,
                            uint32_t new_len, uint32_t max_seq_len, int rounding,
                            const int32_t* src_index, uint32_t src_tokens) {
    if (uint64_t(current_len) + new_len > max_seq_len) return GRANITE_HIP_EOVERFLOW;
    AppendParams p{};
    p.src_index = src_index;
    p.src_tokens = src_tokens;
    p.src[0] = new_k;
    p.src[1] = new_v;
    p.dst[0] = static_cast<uint16_t*>(cache_k);
    p.dst[1] = static_cast<uint16_t*>(cache_v);
    p.table = nullptr;
    p.src_tok_stride = src_tok_stride;
    p.src_head_stride = src_head_stride;
    p.num_kv_heads = num_kv_heads;
    p.head_dim = head_dim;
    p.first_pos = current_len;
    p.new_len = new_len;
    p.max_seq = max_seq_len;
    p.block_size = 1;
    return launch_append(p, src_dtype, rounding);
}

int launch_kv_append_paged(const void* new_k, const void* new_v, int src_dtype,
                           int64_t src_tok_stride, int64_t src_head_stride, void* k_cache,
                           void* v_cache, const int32_t* block_table, uint32_t num_kv_heads,
                           uint32_t head_dim, uint32_t start_pos, uint32_t new_len,
                           uint32_t block_size, int rounding, const int32_t* src_index,
                           uint32_t src_tokens) {
    if (!block_table) return GRANITE_HIP_ENULL;
    if (block_size == 0) return GRANITE_HIP_EINVAL;
    AppendParams p{};
    p.src_index = src_index;
    p.src_tokens = src_tokens;
    p.src[0] = new_k;
    p.src[1] = new_v;
    p.dst[0] = static_cast<uint16_t*>(k_cache);
    p.dst[1] = static_cast<uint16_t*>(v_cache);
    p.table = block_table;
    p.src_tok_stride = src_tok_stride;
    p.src_head_stride = src_head_stride;
    p.num_kv_heads = num_kv_heads;
    p.head_dim = head_dim;
    p.first_pos = start_pos;
    p.new_len = new_len;
    p.max_seq = 0;
    p.block_size = block_size;
    return launch_append(p, src_dtype, rounding);
}

int launch_kv_gather_paged(void* dst_k, void* dst_v, const void* k_cache, const void* v_cache,
                           const int32_t* block_table, uint32_t num_kv_heads, uint32_t head_dim,
                           uint32_t len, uint32_t block_size, uint32_t max_seq_len) {
    if (!dst_k || !dst_v || !k_cache || !v_cache || !block_table) return GRANITE_HIP_ENULL;
    if (block_size == 0 || num_kv_heads == 0 || head_dim == 0 || head_dim % kVec != 0)
        return GRANITE_HIP_EINVAL;
    if (len > max_seq_len) return GRANITE_HIP_EOVERFLOW;
    if (len == 0) return GRANITE_HIP_OK;
    if (!aligned16(dst_k) || !aligned16(dst_v) || !aligned16(k_cache) || !aligned16(v_cache))
        return GRANITE_HIP_EINVAL;
    GatherParams p{};
    p.src[0] = static_cast<const uint16_t*>(k_cache);
    p.src[1] = static_cast<const uint16_t*>(v_cache);
    p.dst[0] = static_cast<uint16_t*>(dst_k);
    p.dst[1] = static_cast<uint16_t*>(dst_v);
    p.table = block_table;
    p.num_kv_heads = num_kv_heads;
    p.head_dim = head_dim;
    p.len = len;
    p.block_size = block_size;
    p.max_seq = max_seq_len;
    const uint64_t work = uint64_t(len) * num_kv_heads * (head_dim / kVec);
    if (work >= (1ull << 32)) return GRANITE_HIP_EINVAL;
    uint32_t blocks = static_cast<uint32_t>((work + 255) / 256);
    if (blocks > 65535u * 4) blocks = 65535u * 4;
    {
        KernelTimerScope timer("kv_gather");
        kv_gather_kernel<<<dim3(blocks, 2), dim3(256), 0, ctx().stream>>>(p);
    }
    return launch_status();
}

// Rows of 2-byte elements copied between two pitches, the tail of every destination row filled
// with zeros: pads [rows, d] to [rows, d_padded] (or slices the other way, with no fill).
__global__ void __launch_bounds__(256) copy_rows_kernel(uint16_t* dst, int64_t dst_pitch, const uint16_t* src,
                                                        int64_t src_pitch, uint64_t rows, uint32_t copy_elems,
                                                        uint32_t fill_elems) {
    const uint64_t total = rows * fill_elems;
    for (uint64_t i = uint64_t(blockIdx.x) * blockDim.x + threadIdx.x; i < total; i += uint64_t(gridDim.x) * blockDim.x) {
        const uint64_t r = i / fill_elems;
        const uint32_t c = uint32_t(i - r * fill_elems);
        dst[r * dst_pitch + c] = c < copy_elems ? src[r * src_pitch + c] : uint16_t(0);
    }
}

int launch_copy_rows(void* dst, int64_t dst_row_bytes, const void* src, int64_t src_row_bytes, uint64_t rows,
                     uint32_t copy_bytes, uint32_t fill_bytes) {
    if (!dst || !src) return GRANITE_HIP_ENULL;
    if (rows == 0 || fill_bytes == 0) return GRANITE_HIP_OK;
    if (copy_bytes > fill_bytes || (copy_bytes | fill_bytes) % 2 || dst_row_bytes % 2 || src_row_bytes % 2 ||
        dst_row_bytes < int64_t(fill_bytes) || src_row_bytes < int64_t(copy_bytes) ||
        (reinterpret_cast<uintptr_t>(dst) | reinterpret_cast<uintptr_t>(src)) % 2)
        return GRANITE_HIP_EINVAL;
    const uint64_t work = rows * (fill_bytes / 2);
    const uint32_t blocks = static_cast<uint32_t>(std::min<uint64_t>((work + 255) / 256, 65535u * 4));
    {
        KernelTimerScope timer("copy_rows");
        copy_rows_kernel<<<dim3(blocks), dim3(256), 0, ctx().stream>>>(
            static_cast<uint16_t*>(dst), dst_row_bytes / 2, static_cast<const uint16_t*>(src), src_row_bytes / 2, rows,
            copy_bytes / 2, fill_bytes / 2);
    }
    return launch_status();
}

}  // namespace ghip
