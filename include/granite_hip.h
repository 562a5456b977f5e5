/*
 * granite_hip.h -- C ABI of the MI355X (gfx950) attention backend for Granite.
 *
 * One shared library, libgranite_hip.so, exports everything below.  The
 * signatures use plain pointers and integers only, so the library can be
 * bound from C++ (the HipCompute / HipBackend classes of the host layer),
 * from ctypes, or from any other FFI.  Each entry point names the interface
 * of the reference that it stands in for (paths relative to the reference
 * tree).
 *
 * Conventions
 *   - every function returns 0 on success, a GRANITE_HIP_E* code (negative)
 *     for a rejected argument, or a positive hipError_t value;
 *     granite_hip_error_string() renders either;
 *   - all device pointers come from granite_hip_malloc() (or any other HIP
 *     allocation on the same device);
 *   - launches are enqueued on the library's single in-order stream and
 *     return immediately; results are valid after granite_hip_sync(), exactly
 *     like MetalCompute::sync() (src/backend/metal/metal_compute.mm:150-207);
 *   - "half" means IEEE binary16 stored as uint16_t;
 *   - head_dim must be 128 or 64 for the attention entry points, the two sizes
 *     the reference has decode and paged kernels for
 *     (metal_shaders_attention.h:2769-3177, 3202-3847; GRANITE_HIP_EUNSUPPORTED
 *     otherwise, as the reference rejects other sizes, metal_compute.mm:2556-2559);
 *     the KV append/gather entry points accept any head_dim that is a multiple
 *     of 8.
 *
 * Layouts (D = head_dim, G = num_heads / num_kv_heads)
 *   contiguous cache   [num_kv_heads, max_seq, D] half   (src/llm/kv_cache.cpp:20-25)
 *   paged pool         [num_blocks*block_size, num_kv_heads, D] half
 *                      (src/llm/paged_kv_cache.cpp:44-49); logical token p of a
 *                      sequence lives in row block_table[p / bs] * bs + p % bs
 */
#ifndef GRANITE_HIP_H
#define GRANITE_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- error codes ------------------------------------------------------- */
#define GRANITE_HIP_OK 0
#define GRANITE_HIP_EINVAL (-1)      /* ErrorCode::InvalidArgument */
#define GRANITE_HIP_ENOTINIT (-2)    /* ErrorCode::BackendNotInitialized */
#define GRANITE_HIP_ENOMEM (-3)      /* ErrorCode::AllocationFailed */
#define GRANITE_HIP_EUNSUPPORTED (-4)/* ErrorCode::NotImplemented */
#define GRANITE_HIP_ENULL (-5)       /* ErrorCode::NullPointer */
#define GRANITE_HIP_EOVERFLOW (-6)   /* KV cache overflow (kv_cache.cpp:61-65) */
#define GRANITE_HIP_ESCRATCH (-7)    /* the scratch buffer given is too small for this launch */

/* element types of Q / output tensors */
#define GRANITE_HIP_F32 0
#define GRANITE_HIP_F16 1

/* float -> half conversion used by the append entry points */
#define GRANITE_HIP_ROUND_TRUNCATE 0 /* Granite's CPU fp32_to_fp16 (src/llm/math_ops.cpp:45-54) */
#define GRANITE_HIP_ROUND_NEAREST 1  /* Granite's GPU kernels, half(x) (metal_shaders_attention.h:124) */

/* memory kinds, same order as granite::MemoryType (include/granite/types.h:131-135) */
#define GRANITE_HIP_MEM_DEVICE 0
#define GRANITE_HIP_MEM_SHARED 1  /* pinned host memory, device-visible */
#define GRANITE_HIP_MEM_MANAGED 2 /* device memory + host mirror handled by the C++ backend */

/* mask modes of granite_hip_attention() */
#define GRANITE_HIP_MASK_NONE 0   /* every key visible */
#define GRANITE_HIP_MASK_CAUSAL 1 /* key k visible iff k <= start_pos + q */
#define GRANITE_HIP_MASK_TREE 2   /* cache keys visible; extra keys by ancestor walk */

/* ---- backend: lifecycle, memory, stream ------------------------------- *
 * Stand in for the parts of IComputeBackend that touch the device
 * (include/granite/backend.h:30-183: initialize/shutdown, create_buffer,
 * write_buffer/read_buffer/copy_buffer, wait_for_completion) and for
 * MetalCompute::{initialize,shutdown,sync,commit,create_buffer}
 * (include/granite/metal_compute.h:29-43, 944). */
typedef struct granite_hip_device_info {
    char name[128];
    char arch[32];
    size_t total_memory;
    size_t max_buffer_size;
    size_t shared_memory_per_block;
    int max_threads_per_block;
    int wavefront_size;
    int compute_units;
    int clock_khz;
} granite_hip_device_info;

int granite_hip_init(int device);
int granite_hip_shutdown(void);
int granite_hip_is_initialized(void);
int granite_hip_get_device_info(granite_hip_device_info *info);
const char *granite_hip_error_string(int code);
const char *granite_hip_version(void);

int granite_hip_malloc(void **ptr, size_t bytes, int memory_kind);
int granite_hip_free(void *ptr, int memory_kind);
int granite_hip_memcpy_h2d(void *dst, const void *src, size_t bytes);
int granite_hip_memcpy_d2h(void *dst, const void *src, size_t bytes);
int granite_hip_memcpy_d2d(void *dst, const void *src, size_t bytes);
int granite_hip_memset(void *dst, int value, size_t bytes);
int granite_hip_sync(void);
/* Use `stream` (a hipStream_t) for all later launches; NULL restores the
 * library's own stream.  The hand-over is ordered: the new stream first waits
 * for everything queued on the old one, because all launches share one
 * scratch buffer.  Launches are single-threaded and go to one stream at a
 * time, like the one command queue of MetalCompute
 * (src/backend/metal/metal_compute.mm:150-207); the library takes no lock. */
int granite_hip_set_stream(void *stream);
void *granite_hip_get_stream(void);

/* Timing on the launch stream (MetalCompute::enable_kernel_timing analogue,
 * metal_compute.h:51-59): events are created, recorded on the launch stream
 * and compared in milliseconds. */
int granite_hip_event_create(void **event);
int granite_hip_event_destroy(void *event);
int granite_hip_event_record(void *event);
int granite_hip_event_synchronize(void *event);
int granite_hip_event_elapsed_ms(void *start, void *stop, float *ms);

/* Per-kernel GPU time, bucketed by kernel name (MetalCompute::enable_kernel_timing,
 * reset_kernel_timing, get_kernel_timing_stats; include/granite/metal_compute.h:51-59).
 * While enabled every launch is bracketed by two events on the launch stream.
 * Names: "kv_append", "kv_gather", "decode_stream" or "decode_splitk",
 * "decode_merge", "attention_tiles", "attention_merge", "tree_mask", "rope_append",
 * "matvec_q4k", "copy_rows".  granite_hip_kernel_timing_names() writes the
 * names seen so far, comma separated. */
int granite_hip_enable_kernel_timing(int enable);
int granite_hip_reset_kernel_timing(void);
int granite_hip_get_kernel_timing(const char *kernel_name, double *total_ms,
                                  uint64_t *dispatches);
int granite_hip_kernel_timing_names(char *buffer, size_t buffer_bytes);

/* ---- KV cache append / gather ----------------------------------------- */

/* MetalCompute::kv_cache_append (include/granite/metal_compute.h:784-797;
 * kernel metal_shaders_attention.h:102-125).  new_k/new_v: [new_len,
 * num_kv_heads, D] float; cache_k/cache_v: contiguous cache.  Rows
 * current_len .. current_len+new_len-1 are written; conversion is
 * GRANITE_HIP_ROUND_TRUNCATE (the CPU path's, transformer.mm:1687-1688).
 * current_len + new_len > max_seq_len -> GRANITE_HIP_EOVERFLOW. */
int granite_hip_kv_cache_append(void *cache_k, void *cache_v, const void *new_k,
                                const void *new_v, uint32_t num_kv_heads, uint32_t head_dim,
                                uint32_t current_len, uint32_t new_len, uint32_t max_seq_len);

/* General form.  src_dtype F32 (converted with `rounding`) or F16 (bit copy).
 * Source element (token s, head h, d) is at s*src_tok_stride +
 * h*src_head_stride + d, so [new_len,Hkv,D] (tok stride Hkv*D, head stride D)
 * and KVCache::append's [Hkv,new_len,D] (src/llm/kv_cache.cpp:86-94; tok
 * stride D, head stride new_len*D) are both covered. */
int granite_hip_kv_cache_append_ex(void *cache_k, void *cache_v, const void *new_k,
                                   const void *new_v, int src_dtype, int64_t src_tok_stride,
                                   int64_t src_head_stride, uint32_t num_kv_heads,
                                   uint32_t head_dim, uint32_t current_len, uint32_t new_len,
                                   uint32_t max_seq_len, int rounding);

/* MetalCompute::paged_kv_cache_append (metal_compute.h:887-898; kernel
 * metal_shaders_attention.h:2142-2176).  new_k/new_v: [num_kv_heads, new_len,
 * D] float; pools paged; block_table: int32[>= ceil((start_pos+new_len)/bs)].
 * Conversion GRANITE_HIP_ROUND_TRUNCATE. */
int granite_hip_paged_kv_cache_append(const void *new_k, const void *new_v, void *k_cache,
                                      void *v_cache, const int32_t *block_table,
                                      uint32_t num_kv_heads, uint32_t head_dim,
                                      uint32_t start_pos, uint32_t new_len, uint32_t block_size);

/* General form (strided source, F32 or F16 source, rounding choice).
 * max_blocks: entries the block table holds; start_pos + new_len tokens must fit
 * that many blocks or the call fails with GRANITE_HIP_EOVERFLOW before anything is
 * written.  0: not stated, as in the reference's entry point, which takes no
 * bound -- a table that is too short is then read past its end. */
int granite_hip_paged_kv_cache_append_ex(const void *new_k, const void *new_v, int src_dtype,
                                         int64_t src_tok_stride, int64_t src_head_stride,
                                         void *k_cache, void *v_cache,
                                         const int32_t *block_table, uint32_t num_kv_heads,
                                         uint32_t head_dim, uint32_t start_pos,
                                         uint32_t new_len, uint32_t block_size, int rounding,
                                         uint32_t max_blocks);

/* Commit of a speculation tree's accepted path.  After find_accepted_path
 * (src/llm/speculation_tree.cpp:85-143) the runner only truncates the target
 * cache to "original + accepted" (src/llm/speculative_runner.cpp:871-882),
 * which assumes the tree's K/V had been appended in path order; the
 * reference's attention_tree (transformer.mm:1870-2140, 2146-2402) appends
 * nothing, so that step is unfinished upstream and this entry point defines
 * it: row i of the cache range [start_pos, start_pos + num_accepted) receives
 * tree node accepted_nodes[i] (device int32) of k_tree / v_tree, whose element
 * (node s, head h, d) sits at s*src_tok_stride + h*src_head_stride + d
 * ([num_kv_heads, num_nodes, D]: tok stride D, head stride num_nodes*D).  F16
 * sources are copied bit for bit, F32 ones converted with `rounding`.  A node
 * index outside [0, num_nodes) leaves its row unwritten.  block_table NULL:
 * contiguous cache with row stride max_seq_len; else paged with block_size. */
int granite_hip_kv_commit_accepted(const void *k_tree, const void *v_tree, int src_dtype,
                                   int64_t src_tok_stride, int64_t src_head_stride,
                                   uint32_t num_nodes, const int32_t *accepted_nodes,
                                   uint32_t num_accepted, void *k_cache, void *v_cache,
                                   const int32_t *block_table, uint32_t num_kv_heads,
                                   uint32_t head_dim, uint32_t start_pos, uint32_t block_size,
                                   uint32_t max_seq_len, int rounding);

/* Gather of logical tokens [0, len) of one sequence out of the paged pools
 * into contiguous caches [num_kv_heads, max_seq_len, D] half (bit copy).  The
 * device form of the per-call gather in src/llm/transformer.mm:1750-1763 and
 * of sync_cpu_to_gpu_kv_cache (transformer.mm:4539-4620). */
int granite_hip_paged_kv_gather(void *dst_k, void *dst_v, const void *k_cache,
                                const void *v_cache, const int32_t *block_table,
                                uint32_t num_kv_heads, uint32_t head_dim, uint32_t len,
                                uint32_t block_size, uint32_t max_seq_len);

/* Strided row copy on the launch stream: for every row r < rows, the first copy_bytes of
 * src + r*src_row_bytes go to dst + r*dst_row_bytes and bytes copy_bytes .. fill_bytes-1 of
 * the destination row become zero (fill_bytes >= copy_bytes; equal: a plain 2-D copy).  All
 * byte counts, pitches and pointers are multiples of 2.  MetalAttentionOp walks mapped
 * buffers on the host for any head size (src/operators/metal/metal_operators.mm:1262-1300);
 * the HIP operator uses this copy to present head sizes that have no kernel zero-padded to 64
 * or 128 and to slice the result back. */
int granite_hip_copy_rows(void *dst, int64_t dst_row_bytes, const void *src, int64_t src_row_bytes,
                          uint64_t rows, uint32_t copy_bytes, uint32_t fill_bytes);

/* ---- attention --------------------------------------------------------- */

/* MetalCompute::multihead_attention (metal_compute.h:799-816;
 * metal_compute.mm:2253-2378).  K, V: contiguous cache with row stride
 * max_seq (0 = seq_kv).  seq_q == 1: decode, Q/out [num_heads, D] float.
 * seq_q > 1: causal prefill with start_pos 0, Q/out [seq_q, num_heads, D]
 * float (the layout the reference kernel indexes,
 * metal_shaders_attention.h:1640-1660).  Semantics are the CPU path's
 * (transformer.mm:1779-1840): no epsilon in the denominator, fp32 softmax. */
int granite_hip_multihead_attention(const void *q, const void *k, const void *v, void *out,
                                    uint32_t num_heads, uint32_t num_kv_heads, uint32_t seq_q,
                                    uint32_t seq_kv, uint32_t head_dim, float scale,
                                    uint32_t max_seq);

/* MetalCompute::attention_tree (metal_compute.h:830-844; metal_compute.mm:2463-2529).
 * Q/out [num_heads, num_nodes, D] float; k_cache/v_cache contiguous with row
 * stride cache_len (as the reference kernel indexes them,
 * metal_shaders_attention.h:1708-1709); k_tree/v_tree [num_kv_heads,
 * num_nodes, D] half; parent_indices int32[num_nodes], -1 = root.  Node i sees
 * the whole cache, itself and its ancestors (transformer.mm:822-840). */
int granite_hip_attention_tree(const void *q, const void *k_cache, const void *v_cache,
                               const void *k_tree, const void *v_tree,
                               const int32_t *parent_indices, void *out, uint32_t num_heads,
                               uint32_t num_kv_heads, uint32_t num_nodes, uint32_t cache_len,
                               uint32_t head_dim, float scale);

/* MetalCompute::paged_attention_decode (metal_compute.h:869-881;
 * metal_compute.mm:2535-2621).  Q/out [num_heads, D] float. */
int granite_hip_paged_attention_decode(const void *q, const void *k_cache, const void *v_cache,
                                       const int32_t *block_table, void *out,
                                       uint32_t num_heads, uint32_t num_kv_heads,
                                       uint32_t seq_len, uint32_t head_dim,
                                       uint32_t block_size, float scale);

/* MetalCompute::batched_paged_attention_decode (metal_compute.h:906-920;
 * metal_compute.mm:2658-2696).  Q/out [batch, num_heads, D] float;
 * block_tables int32[batch, max_blocks_per_seq]; seq_lens int32[batch] (device
 * memory); a sequence of length 0 leaves its output rows untouched. */
int granite_hip_batched_paged_attention_decode(const void *q, const void *k_cache,
                                               const void *v_cache,
                                               const int32_t *block_tables,
                                               const int32_t *seq_lens, void *out,
                                               uint32_t batch_size, uint32_t num_heads,
                                               uint32_t num_kv_heads, uint32_t head_dim,
                                               uint32_t block_size,
                                               uint32_t max_blocks_per_seq, float scale);

/* Decode, general form: adds half-precision Q, a log-sum-exp output and a
 * contiguous-cache variant to the two entry points above.
 *   q            [batch, num_heads, D], q_dtype F32 or F16
 *   out          [batch, num_heads, D] float
 *   lse          float[batch, num_heads] or NULL; natural-log-sum-exp of the
 *                scaled scores (no reference counterpart: the reference keeps
 *                max and sum internal, metal_shaders_attention.h:3046-3048)
 *   block_tables NULL selects the contiguous cache layout with row stride
 *                max_seq (batch must be 1); otherwise paged
 *   seq_lens     device int32[batch], bounded by max_blocks_per_seq*block_size
 *                (paged) or max_seq (contiguous), from which the grid is
 *                sized; NULL means every sequence has the host-known length
 *                fixed_seq_len. */
typedef struct granite_hip_decode_args {
    const void *q;
    int q_dtype;
    const void *k_cache;
    const void *v_cache;
    const int32_t *block_tables;
    const int32_t *seq_lens;
    void *out;
    float *lse;
    uint32_t batch_size, num_heads, num_kv_heads, head_dim;
    uint32_t block_size, max_blocks_per_seq; /* paged */
    uint32_t max_seq;                        /* contiguous: row stride and length bound */
    float scale;
    uint32_t fixed_seq_len; /* used when seq_lens is NULL */
    uint32_t chunk_tokens;  /* split-K chunk, multiple of 32; 0 = library default */
} granite_hip_decode_args;

int granite_hip_decode_attention(const granite_hip_decode_args *args);

/* Prefill / chunked prefill / tree attention, general form.  One sequence.
 * Keys are the concatenation of
 *   segment A: `cache_len` tokens from the KV cache -- contiguous (block_table
 *              NULL, row stride max_seq) or paged (block_table given);
 *   segment B: `extra_len` tokens from k_extra/v_extra [num_kv_heads,
 *              extra_len, D] half (tree nodes; NULL/0 when unused).
 * mask_mode CAUSAL: key k (index in the concatenation) visible iff
 *              k <= start_pos + q                       (transformer.mm:1797-1806)
 * mask_mode TREE:  segment A fully visible, key j of segment B visible to
 *              query i iff j == i or j is an ancestor of i via parents[]
 *              (transformer.mm:2066-2090, 822-840); seq_q must equal extra_len.
 * Q element (token t, head h, d) at t*q_tok_stride + h*q_head_stride + d;
 * same for out with its strides; lse float[num_heads, seq_q] or NULL. */
typedef struct granite_hip_attention_args {
    const void *q;
    int q_dtype;
    int64_t q_tok_stride, q_head_stride;
    void *out;
    int out_dtype;
    int64_t out_tok_stride, out_head_stride;
    float *lse;
    const void *k_cache;
    const void *v_cache;
    const int32_t *block_table;
    uint32_t block_size;
    uint32_t max_seq;
    uint32_t cache_len;
    const void *k_extra;
    const void *v_extra;
    uint32_t extra_len;
    const int32_t *parents;
    int mask_mode;
    uint32_t start_pos;
    uint32_t seq_q, num_heads, num_kv_heads, head_dim;
    float scale;
} granite_hip_attention_args;

int granite_hip_attention(const granite_hip_attention_args *args);

/* Ancestor bit mask from parent pointers (transformer.mm:822-840): row i holds
 * ceil(num_nodes/32) uint32 words, bit j of row i set iff node i may attend
 * node j.  The walk stops after num_nodes steps, so a malformed parent array
 * cannot hang the device. */
int granite_hip_build_tree_mask(const int32_t *parent_indices, uint32_t *mask_words,
                                uint32_t num_nodes);

/* ---- rotary position embedding, fused with the K/V append ---------------- */

/* MetalCompute::rope_multihead (include/granite/metal_compute.h:728-739;
 * kernel src/backend/metal/kernels/metal_shaders_util.h:596-635): q
 * [seq_len, num_heads_q, D] float and k [seq_len, num_heads_k, D] float are
 * rotated in place, pairs (2i, 2i+1) by (start_pos + s) * freq_base^(-2i/D),
 * cos/sin evaluated on the device in float as the reference kernel does. */
int granite_hip_rope_multihead(void *q, void *k, uint32_t num_heads_q, uint32_t num_heads_k,
                               uint32_t seq_len, uint32_t head_dim, uint32_t start_pos,
                               float freq_base);

/* General form: the rotation and, in the same pass, the append that follows it
 * on the path (MetalCompute::kv_cache_append / paged_kv_cache_append above;
 * call order src/llm/transformer.mm:3363 ff.).
 *   q, k          as above; either may be NULL.  k is rewritten in float only
 *                 when write_k_back is set (the reference always does).
 *   q_f16         optional half copy of the rotated q, same layout, round to
 *                 nearest (the dtype the prefill kernel reads directly)
 *   v             [seq_len, num_heads_k, D] float, NULL without cache_v
 *   cache_k/v     NULL: no append.  block_table NULL: contiguous cache
 *                 [num_heads_k, max_seq_len, D] half, rows start_pos ..;
 *                 else the paged pools [rows, num_heads_k, D] half
 *   cos_table,    RoPECache's tables (src/llm/rope.cpp:5-22), float
 *   sin_table     [table_positions, D/2] on the device: the rotation then uses
 *                 exactly these values and separately rounded products, and is
 *                 bit-identical to RoPECache::apply (rope.cpp:24-92); start_pos
 *                 + seq_len > table_positions -> GRANITE_HIP_EOVERFLOW, its
 *                 range check (rope.cpp:34-38).  Both NULL: evaluated from
 *                 freq_base on the device.
 *   rounding      float -> half conversion of the cache rows
 *   positions     NULL, or device int32[seq_len]: the position of every token
 *                 (a batch of decode steps: token s belongs to sequence s).
 *                 block_table then advances by table_stride entries per token
 *                 (0: one table) and holds max_blocks_per_seq entries per
 *                 sequence.  The host cannot check values that live on the
 *                 device, so the kernel does: a token whose position is
 *                 negative or beyond the cos/sin tables is left untouched, one
 *                 whose position is beyond its cache (max_seq_len, or
 *                 max_blocks_per_seq blocks) is rotated but not stored.
 *   max_blocks_per_seq  entries the block table holds (per sequence).  Without
 *                 positions, 0 means "not stated" (as in
 *                 MetalCompute::paged_kv_cache_append, which takes no bound);
 *                 otherwise start_pos + seq_len tokens must fit that many
 *                 blocks, or the call fails with GRANITE_HIP_EOVERFLOW. */
typedef struct granite_hip_rope_args {
    void *q;
    void *q_f16;
    void *k;
    const void *v;
    void *cache_k;
    void *cache_v;
    const int32_t *block_table;
    const float *cos_table;
    const float *sin_table;
    uint32_t table_positions;
    uint32_t num_heads_q, num_heads_k, seq_len, head_dim, start_pos;
    uint32_t max_seq_len; /* contiguous cache */
    uint32_t block_size;  /* paged */
    float freq_base;
    int write_k_back;
    int rounding;
    const int32_t *positions;
    int64_t table_stride;
    uint32_t max_blocks_per_seq;
} granite_hip_rope_args;

int granite_hip_rope_append(const granite_hip_rope_args *args);

/* ---- projections either side of attention, on Q4_K weights ----------------- *
 * A weight matrix is [N, K / 256] Q4_K super-blocks of 144 bytes, row n holding
 * the K inputs of output n (half d, half dmin, 12 bytes of 6-bit scales and
 * minima, 128 bytes of 4-bit values; a weight is d * scale * q - dmin * min,
 * src/model/gguf.cpp:952-1020).  K is a multiple of 256; x, the weights and
 * the strides are 16-byte aligned.  Results are float, accumulated in float
 * from the 4-bit values as the reference's GPU kernels do (no weight is ever
 * rounded to half, which is what separates them from its CPU path). */

/* MetalCompute::fused_qkv_matvec_q4k (include/granite/metal_compute.h:683-694;
 * kernel metal_shaders_quant.h:167-295; call sites transformer.mm:2966, 4752):
 * yq[Nq] = Wq x, yk[Nkv] = Wk x, yv[Nkv] = Wv x for one token, one launch. */
int granite_hip_fused_qkv_matvec_q4k(const void *x, const void *wq, const void *wk,
                                     const void *wv, void *yq, void *yk, void *yv, uint32_t K,
                                     uint32_t Nq, uint32_t Nkv);

/* The same for `batch` tokens (a batched decode step): x [batch, K] with rows
 * x_stride floats apart, yq [batch, Nq] rows yq_stride apart, yk and yv
 * [batch, Nkv] rows ykv_stride apart -- the layouts granite_hip_rope_append
 * takes as q, k and v.  Up to two tokens go through the vector kernel of the
 * single-token form; more go through the matrix cores, up to 64 tokens per pass
 * over the weights, a token's inputs of a 512-column chunk scaled by a power of
 * two into the middle of the half range and split into a half and a half
 * remainder (inputs of any float magnitude keep 22 bits of the chunk's largest)
 * and the 4-bit values multiplied as exact integers: results are float sums of
 * exact products, as in the other form.  The chunks of K are added by a second
 * launch through the library's scratch (chunks x batch, rounded up to whole
 * workgroups of 32 or 64 tokens, x (Nq + 2 Nkv) floats:
 * granite_hip_q4k_workspace_required). */
int granite_hip_fused_qkv_matvec_q4k_batched(const void *x, int64_t x_stride, const void *wq,
                                             const void *wk, const void *wv, void *yq, void *yk,
                                             void *yv, int64_t yq_stride, int64_t ykv_stride,
                                             uint32_t K, uint32_t Nq, uint32_t Nkv,
                                             uint32_t batch);

/* Bytes of library scratch a projection of `batch` tokens onto `rows` weight
 * rows (Nq + 2 Nkv for the fused form) needs; 0 for up to two tokens.  Reserve
 * it with granite_hip_reserve_workspace to keep the batched forms from
 * allocating on their first call. */
size_t granite_hip_q4k_workspace_required(uint32_t K, uint64_t rows, uint32_t batch);

/* MetalCompute::matvec_q4k (metal_compute.h:73-79; kernel metal_shaders_quant.h:59-163):
 * y[N] = W x, the output projection behind attention (transformer.mm:2650, 2955). */
int granite_hip_matvec_q4k(const void *x, const void *w, void *y, uint32_t K, uint32_t N);
int granite_hip_matvec_q4k_batched(const void *x, int64_t x_stride, const void *w, void *y,
                                   int64_t y_stride, uint32_t K, uint32_t N, uint32_t batch);

/* ---- scratch memory ------------------------------------------------------ *
 * Decode and prefill launches that split the keys over several workgroups
 * keep partial results (and the stream decode kernel its plan, large trees
 * their ancestor mask) in device scratch.  By default that is one buffer the
 * library owns and grows on demand; growing waits for the device, frees and
 * allocates, so a first call with a larger shape stalls.  MetalCompute's calls
 * only ever enqueue (src/backend/metal/metal_compute.mm:150-207); to get the
 * same here either reserve once, up front, what the largest launch will need,
 * or hand every launch its own scratch with the _ws forms, which never
 * allocate and never synchronise. */

/* Bytes of device scratch the library holds at the moment. */
size_t granite_hip_workspace_bytes(void);

/* Grows the library's scratch to at least `bytes` now (waits for the device
 * when it has to grow).  Later launches that need no more never allocate. */
int granite_hip_reserve_workspace(size_t bytes);

/* Scratch bytes the launch described by `args` needs (0 for shapes that need
 * none).  Nothing is launched; pointers in `args` are only tested for NULL. */
int granite_hip_decode_workspace_required(const granite_hip_decode_args *args, size_t *bytes);
int granite_hip_attention_workspace_required(const granite_hip_attention_args *args,
                                             size_t *bytes);

/* granite_hip_decode_attention / granite_hip_attention with caller-owned
 * scratch: `workspace` (256-byte aligned device memory of `workspace_bytes`)
 * is the only scratch the launch uses, and it stays in use until the launch
 * has run.  Too small -> GRANITE_HIP_ESCRATCH, nothing launched.  workspace
 * NULL: the library's buffer, as in the plain forms. */
int granite_hip_decode_attention_ws(const granite_hip_decode_args *args, void *workspace,
                                    size_t workspace_bytes);
int granite_hip_attention_ws(const granite_hip_attention_args *args, void *workspace,
                             size_t workspace_bytes);

/* granite_hip_decode_attention for callers that cannot allocate.  It has no
 * counterpart in the reference; it is for code under HIP graph capture, tight
 * serving loops and harnesses that forbid hipMalloc.  Same arguments, same
 * kernels and bit-identical results, but the scratch (the stream kernel's
 * plan and partial results) is a fixed array in device memory that the library
 * holds on every GPU it runs on, granite_hip_static_scratch_bytes() (32 MiB)
 * long, and the call makes no allocation of any kind: no hipMalloc, no
 * hipFree, no events (per-kernel timing skips these launches).  A launch that
 * needs more -- granite_hip_decode_workspace_required() tells -- fails with
 * GRANITE_HIP_ESCRATCH and launches nothing.  Every call on a GPU uses that
 * GPU's one array: calls that overlap on one GPU (two streams, two threads)
 * race; calls queued on the library's single stream are ordered and safe.
 * Nothing in the array has to start at zero, the kernels write every partial
 * they later read. */
int granite_hip_decode_attention_static(const granite_hip_decode_args *args);
size_t granite_hip_static_scratch_bytes(void);

#ifdef __cplusplus
}
#endif
#endif /* GRANITE_HIP_H */
