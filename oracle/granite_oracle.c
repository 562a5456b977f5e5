/*
 * granite_oracle.c -- CPU restatement of Granite's CPU attention path.
 *
 * THIS FILE IS TEST INFRASTRUCTURE.  It is the checker that the HIP kernels
 * are compared against and the timed "CPU baseline" of the benchmark.  It is
 * never linked into, imported by or called from the product library; the
 * product fails loudly when its HIP library is missing instead of falling
 * back to this code.
 *
 * Every function restates, loop for loop and in the same fp32 summation
 * order, a piece of the reference (paths relative to the reference tree):
 *
 *   go_fp16_to_fp32            src/llm/math_ops.cpp:18-43
 *   go_fp32_to_fp16            src/llm/math_ops.cpp:45-54   (truncating)
 *   go_parallel_for            src/llm/math_ops.h:41-69, math_ops.cpp:56-58
 *   go_kv_cache_append_f16     src/llm/kv_cache.cpp:55-107  (per-head memcpy)
 *   go_kv_cache_append_f32     src/backend/metal/kernels/metal_shaders_attention.h:102-125
 *                              with the CPU conversion of src/llm/transformer.mm:1682-1691
 *   go_paged_kv_cache_append   metal_shaders_attention.h:2142-2176 (address formula),
 *                              conversion as above
 *   go_paged_gather_*          tools/test_paged_flash_attention.mm:41-47 (address formula)
 *   go_attention               src/llm/transformer.mm:1703-1709, 1740-1770, 1779-1840
 *   go_tree_mask               src/llm/transformer.mm:822-840
 *   go_attention_tree          src/llm/transformer.mm:1978-1983, 2012-2042, 2044-2126
 *   go_block_manager_*         src/llm/paged_kv_cache.cpp:17-98
 *   go_paged_cache_*           src/llm/paged_kv_cache.cpp:104-187
 *   go_rope_table              src/llm/rope.cpp:5-22
 *   go_rope_apply              src/llm/rope.cpp:24-92
 *   go_q4k_dequantize          src/model/gguf.cpp:952-1020  (Q4_K super-blocks)
 *   go_matmul_transb_fp16      src/llm/math_ops.cpp:67-103  (portable branch)
 *   go_matvec_q4k              the projection of MetalCompute::fused_qkv_matvec_q4k
 *                              (src/backend/metal/kernels/metal_shaders_quant.h:167-295):
 *                              weights dequantised by the formula above, not rounded
 *                              to half, dot product in fp32
 *
 * Pinning (what fixes each function besides re-reading it):
 *   conversions     all 65536 halves against the compiler's _Float16, the
 *                   known-answer list in tests/golden/fp16_kat.json, and the
 *                   reference's own math_ops.cpp compiled into oracle/_ref.
 *   attention core  the reference's Vulkan attention known-answer test
 *                   (tests/test_vulkan.cpp:353-482), an independent float64
 *                   numpy implementation on small shapes, and the invariants
 *                   listed in tests/test_oracle_attention.py.
 *   log-sum-exp     NOT a reference output (the reference CPU path never
 *                   forms it); defined here by the closed form
 *                   lse = max_k s_k + ln sum_k exp(s_k - max), pinned by the
 *                   float64 implementation.
 *   block manager   closed forms (LIFO hand-out order N-1, N-2, ...).
 *   rope            the reference's table tests (tests/test_llm.cpp:14-63: size,
 *                   position 0 is (1, 0), position 1 against libm), a float64
 *                   evaluation of the same fp32 angle, and what a rotation fixes:
 *                   pair norms kept, position 0 is the identity, two rotations
 *                   compose, a unit vector maps to (cos, sin).
 *   Q4_K            the sizes the reference's tests hold (tests/test_gguf.cpp:78, 106:
 *                   256 values and 144 bytes per block), ggml's published packing of
 *                   the 6-bit scales and minima run backwards (pack, then unpack, all
 *                   64 x 64 values in all 8 positions), hand-built blocks with closed-form
 *                   values, and a float64 numpy dequantisation written independently;
 *                   go_matmul_transb_fp16 against the reference's own math_ops.cpp in
 *                   oracle/_ref.
 */
#define _GNU_SOURCE
#include <math.h>
#include <pthread.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#include <unistd.h>

/* ------------------------------------------------------------------------- */
/* fp16 <-> fp32                                                             */
/* ------------------------------------------------------------------------- */

/* math_ops.cpp:18-43 -- exact widening, subnormals renormalised by shifting,
 * NaN payload moved up by 13 bits. */
float go_fp16_to_fp32(uint16_t h)
{
    uint32_t sign = (uint32_t)(h >> 15) & 1u;
    uint32_t exp = (uint32_t)(h >> 10) & 0x1Fu;
    uint32_t mant = (uint32_t)h & 0x3FFu;
    uint32_t bits;
    float out;

    if (exp == 0) {
        if (mant == 0) {
            bits = sign << 31;
            memcpy(&out, &bits, 4);
            return out;
        }
        while ((mant & 0x400u) == 0) {
            mant <<= 1;
            exp--; /* wraps below zero exactly as the unsigned reference does */
        }
        exp++;
        mant &= 0x3FFu;
    } else if (exp == 31) {
        bits = (sign << 31) | 0x7F800000u | (mant << 13);
        memcpy(&out, &bits, 4);
        return out;
    }
    bits = (sign << 31) | ((exp + 112u) << 23) | (mant << 13);
    memcpy(&out, &bits, 4);
    return out;
}

/* math_ops.cpp:45-54 -- drops the low 13 mantissa bits (no rounding), flushes
 * everything with a biased half exponent <= 0 to signed zero and everything
 * with exponent >= 31 (Inf and NaN alike) to signed infinity. */
uint16_t go_fp32_to_fp16(float f)
{
    uint32_t bits;
    memcpy(&bits, &f, 4);
    uint32_t sign = (bits >> 16) & 0x8000u;
    int32_t exp = (int32_t)((bits >> 23) & 0xFFu) - 127 + 15;
    uint32_t mant = (bits >> 13) & 0x3FFu;
    if (exp <= 0) return (uint16_t)sign;
    if (exp >= 31) return (uint16_t)(sign | 0x7C00u);
    return (uint16_t)(sign | ((uint32_t)exp << 10) | mant);
}

void go_fp16_to_fp32_array(const uint16_t *src, float *dst, size_t n)
{
    for (size_t i = 0; i < n; i++) dst[i] = go_fp16_to_fp32(src[i]);
}

void go_fp32_to_fp16_array(const float *src, uint16_t *dst, size_t n)
{
    for (size_t i = 0; i < n; i++) dst[i] = go_fp32_to_fp16(src[i]);
}

/* ------------------------------------------------------------------------- */
/* parallel_for: static chunks over freshly created threads                  */
/* ------------------------------------------------------------------------- */

typedef void (*go_work_fn)(size_t idx, void *arg);

static int g_threads_override = 0;

/* math_ops.cpp:56-58 uses std::thread::hardware_concurrency(); the override
 * exists so tests can pin the count. */
void go_set_num_threads(int n) { g_threads_override = n; }

int go_get_num_threads(void)
{
    if (g_threads_override > 0) return g_threads_override;
    long n = sysconf(_SC_NPROCESSORS_ONLN);
    return n > 0 ? (int)n : 1;
}

struct go_chunk {
    go_work_fn fn;
    void *arg;
    size_t begin, end;
};

static void *go_chunk_main(void *p)
{
    struct go_chunk *c = (struct go_chunk *)p;
    for (size_t i = c->begin; i < c->end; i++) c->fn(i, c->arg);
    return NULL;
}

/* math_ops.h:41-69 -- serial when there is one thread or fewer items than
 * threads; otherwise ceil(n/threads) items per thread, threads created for
 * this call and joined before it returns. */
void go_parallel_for(size_t n, size_t num_threads, go_work_fn fn, void *arg)
{
    if (num_threads <= 1 || n < num_threads) {
        for (size_t i = 0; i < n; i++) fn(i, arg);
        return;
    }
    size_t chunk = (n + num_threads - 1) / num_threads;
    pthread_t *tids = (pthread_t *)malloc(num_threads * sizeof(pthread_t));
    struct go_chunk *chunks = (struct go_chunk *)malloc(num_threads * sizeof(struct go_chunk));
    size_t started = 0;
    for (size_t t = 0; t < num_threads; t++) {
        size_t begin = t * chunk;
        size_t end = begin + chunk < n ? begin + chunk : n;
        if (begin >= n) break;
        chunks[t].fn = fn;
        chunks[t].arg = arg;
        chunks[t].begin = begin;
        chunks[t].end = end;
        pthread_create(&tids[t], NULL, go_chunk_main, &chunks[t]);
        started++;
    }
    for (size_t t = 0; t < started; t++) pthread_join(tids[t], NULL);
    free(chunks);
    free(tids);
}

/* Which thread of go_parallel_for ran each index, as the smallest index that thread ran
 * (owner[i] == owner[j] iff one thread ran both): the partition as executed, for comparison
 * with the reference's (tests only). */
struct go_owner_probe {
    pthread_t *ran;
};
static void go_owner_probe_fn(size_t i, void *arg) { ((struct go_owner_probe *)arg)->ran[i] = pthread_self(); }
void go_parallel_for_owner(size_t n, size_t num_threads, int32_t *owner)
{
    struct go_owner_probe probe;
    probe.ran = (pthread_t *)malloc((n + 1) * sizeof(pthread_t));
    go_parallel_for(n, num_threads, go_owner_probe_fn, &probe);
    for (size_t i = 0; i < n; i++) {
        size_t first = i;
        for (size_t j = 0; j < i; j++)
            if (pthread_equal(probe.ran[j], probe.ran[i])) {
                first = j;
                break;
            }
        owner[i] = (int32_t)first;
    }
    free(probe.ran);
}

/* ------------------------------------------------------------------------- */
/* KV cache append / gather                                                  */
/* ------------------------------------------------------------------------- */

/* kv_cache.cpp:55-107.  src [Hkv, new_len, D] halves, cache [Hkv, max_seq, D]
 * halves; one memcpy per head at row current_len.  Returns -1 on overflow
 * (kv_cache.cpp:61-65) and leaves the cache untouched. */
int go_kv_cache_append_f16(uint16_t *cache, const uint16_t *src, int num_kv_heads,
                           int head_dim, int current_len, int new_len, int max_seq)
{
    if (current_len + new_len > max_seq) return -1;
    size_t stride = (size_t)max_seq * head_dim;
    for (int h = 0; h < num_kv_heads; h++) {
        size_t dst_off = (size_t)h * stride + (size_t)current_len * head_dim;
        size_t src_off = (size_t)h * new_len * head_dim;
        memcpy(cache + dst_off, src + src_off, (size_t)new_len * head_dim * sizeof(uint16_t));
    }
    return 0;
}

/* metal_shaders_attention.h:102-125 for the indexing (src [new_len, Hkv, D]
 * floats -> cache [Hkv, max_seq, D] halves at row current_len); the float to
 * half step is the CPU path's truncating conversion (transformer.mm:1687). */
int go_kv_cache_append_f32(uint16_t *cache, const float *src, int num_kv_heads, int head_dim,
                           int current_len, int new_len, int max_seq)
{
    if (current_len + new_len > max_seq) return -1;
    for (int h = 0; h < num_kv_heads; h++)
        for (int s = 0; s < new_len; s++)
            for (int d = 0; d < head_dim; d++) {
                size_t si = ((size_t)s * num_kv_heads + h) * head_dim + d;
                size_t di = ((size_t)h * max_seq + current_len + s) * head_dim + d;
                cache[di] = go_fp32_to_fp16(src[si]);
            }
    return 0;
}

/* Physical row of logical token `pos` (metal_shaders_attention.h:2163-2168,
 * tools/test_paged_flash_attention.mm:41-47). */
static inline size_t go_phys_row(const int32_t *table, int block_size, int pos)
{
    return (size_t)table[pos / block_size] * block_size + (size_t)(pos % block_size);
}

/* metal_shaders_attention.h:2142-2176.  src [Hkv, new_len, D] floats -> pool
 * [num_blocks*bs, Hkv, D] halves for positions start_pos .. start_pos+new_len-1. */
void go_paged_kv_cache_append_f32(uint16_t *pool, const float *src, const int32_t *table,
                                  int num_kv_heads, int head_dim, int start_pos, int new_len,
                                  int block_size)
{
    for (int h = 0; h < num_kv_heads; h++)
        for (int s = 0; s < new_len; s++) {
            size_t row = go_phys_row(table, block_size, start_pos + s);
            for (int d = 0; d < head_dim; d++) {
                size_t si = ((size_t)h * new_len + s) * head_dim + d;
                size_t di = (row * num_kv_heads + h) * head_dim + d;
                pool[di] = go_fp32_to_fp16(src[si]);
            }
        }
}

/* Same scatter for a source that is already half precision (bit copy);
 * src_tok_stride / src_head_stride are in elements so that both
 * [Hkv, new_len, D] and [new_len, Hkv, D] sources are covered. */
void go_paged_kv_cache_append_f16(uint16_t *pool, const uint16_t *src, const int32_t *table,
                                  int num_kv_heads, int head_dim, int start_pos, int new_len,
                                  int block_size, long src_tok_stride, long src_head_stride)
{
    for (int h = 0; h < num_kv_heads; h++)
        for (int s = 0; s < new_len; s++) {
            size_t row = go_phys_row(table, block_size, start_pos + s);
            memcpy(pool + (row * num_kv_heads + h) * head_dim,
                   src + (size_t)s * src_tok_stride + (size_t)h * src_head_stride,
                   (size_t)head_dim * sizeof(uint16_t));
        }
}

/* Gather of logical tokens [0, len) out of the pool into the contiguous cache
 * layout [Hkv, max_seq, D] (bit copy). */
void go_paged_gather_f16(uint16_t *cache, const uint16_t *pool, const int32_t *table,
                         int num_kv_heads, int head_dim, int len, int block_size, int max_seq)
{
    for (int h = 0; h < num_kv_heads; h++)
        for (int s = 0; s < len; s++) {
            size_t row = go_phys_row(table, block_size, s);
            memcpy(cache + ((size_t)h * max_seq + s) * head_dim,
                   pool + (row * num_kv_heads + h) * head_dim,
                   (size_t)head_dim * sizeof(uint16_t));
        }
}

/* ------------------------------------------------------------------------- */
/* Causal GQA attention (transformer.mm:1703-1840)                           */
/* ------------------------------------------------------------------------- */

struct go_attn_job {
    const float *q;      /* [B, Sq, Hq, D] */
    const float *k_all;  /* [total_seq, Hkv, D] */
    const float *v_all;
    float *context;      /* [B, Sq, Hq*D] */
    float *lse;          /* [B, Hq, Sq] or NULL */
    int batch, seq_len, num_heads, num_kv_heads, head_dim, total_seq, start_pos;
    float scale;
};

/* transformer.mm:1789-1840, one (b, h, q_pos) item. */
static void go_attn_item(size_t work_idx_u, void *arg)
{
    const struct go_attn_job *j = (const struct go_attn_job *)arg;
    int work_idx = (int)work_idx_u;
    int num_heads = j->num_heads, seq_len = j->seq_len, head_dim = j->head_dim;
    int total_seq = j->total_seq, num_kv_heads = j->num_kv_heads;
    int heads_per_kv = num_heads / num_kv_heads;

    int b = work_idx / (num_heads * seq_len);
    int rem = work_idx % (num_heads * seq_len);
    int h = rem / seq_len;
    int q_pos = rem % seq_len;
    int kv_h = h / heads_per_kv;
    int abs_pos = j->start_pos + q_pos;

    if (total_seq <= 0) return; /* the reference is undefined here (max over nothing) */
    float *scores = (float *)malloc((size_t)total_seq * sizeof(float));
    const float *q_vec = j->q + ((size_t)(b * seq_len + q_pos) * num_heads + h) * head_dim;

    for (int k_pos = 0; k_pos < total_seq; k_pos++) {
        if (k_pos > abs_pos) {
            scores[k_pos] = -INFINITY;
        } else {
            const float *k_vec = j->k_all + ((size_t)k_pos * num_kv_heads + kv_h) * head_dim;
            float dot = 0;
            for (int d = 0; d < head_dim; d++) dot += q_vec[d] * k_vec[d];
            scores[k_pos] = dot * j->scale;
        }
    }

    float max_score = scores[0];
    for (int i = 1; i < total_seq; i++)
        if (scores[i] > max_score) max_score = scores[i];

    if (j->lse) {
        /* Not part of the reference: closed form over the same fp32 scores,
         * summed in double. */
        double acc = 0.0;
        for (int i = 0; i < total_seq; i++) acc += exp((double)scores[i] - (double)max_score);
        j->lse[((size_t)b * num_heads + h) * seq_len + q_pos] = (float)((double)max_score + log(acc));
    }

    float sum = 0;
    for (int i = 0; i < total_seq; i++) {
        scores[i] = expf(scores[i] - max_score);
        sum += scores[i];
    }
    float inv_sum = 1.0f / sum;
    for (int i = 0; i < total_seq; i++) scores[i] *= inv_sum;

    float *ctx = j->context + ((size_t)(b * seq_len + q_pos) * num_heads + h) * head_dim;
    for (int d = 0; d < head_dim; d++) ctx[d] = 0.0f;
    for (int v_pos = 0; v_pos < total_seq; v_pos++) {
        const float *v_vec = j->v_all + ((size_t)v_pos * num_kv_heads + kv_h) * head_dim;
        float w = scores[v_pos];
        for (int d = 0; d < head_dim; d++) ctx[d] += w * v_vec[d];
    }
    free(scores);
}

/* The attention core over K/V that are already [total_seq, Hkv, D] floats
 * (the "no cache" branch, transformer.mm:1771-1777). */
void go_attention_core(const float *q, const float *k_all, const float *v_all, float *context,
                       float *lse, int batch, int seq_len, int num_heads, int num_kv_heads,
                       int head_dim, int total_seq, int start_pos, float scale)
{
    struct go_attn_job job = {q, k_all, v_all, context, lse, batch, seq_len, num_heads,
                              num_kv_heads, head_dim, total_seq, start_pos, scale};
    size_t total_work = (size_t)batch * num_heads * seq_len;
    go_parallel_for(total_work, (size_t)go_get_num_threads(), go_attn_item, &job);
}

/* Full cached path: single-threaded half->float transposing gather of the
 * contiguous cache [Hkv, max_seq, D] into [total_seq, Hkv, D]
 * (transformer.mm:1750-1763), then the core.  scale = 1/sqrtf(D) when the
 * caller passes scale <= 0 (transformer.mm:1705). */
void go_attention_cached(const float *q, const uint16_t *cache_k, const uint16_t *cache_v,
                         float *context, float *lse, int batch, int seq_len, int num_heads,
                         int num_kv_heads, int head_dim, int total_seq, int max_seq,
                         int start_pos, float scale)
{
    size_t n = (size_t)total_seq * num_kv_heads * head_dim;
    float *k_buf = (float *)malloc(n * sizeof(float));
    float *v_buf = (float *)malloc(n * sizeof(float));
    for (int h = 0; h < num_kv_heads; h++)
        for (int s = 0; s < total_seq; s++)
            for (int d = 0; d < head_dim; d++) {
                size_t si = ((size_t)h * max_seq + s) * head_dim + d;
                size_t di = ((size_t)s * num_kv_heads + h) * head_dim + d;
                k_buf[di] = go_fp16_to_fp32(cache_k[si]);
                v_buf[di] = go_fp16_to_fp32(cache_v[si]);
            }
    if (scale <= 0) scale = 1.0f / sqrtf((float)head_dim);
    go_attention_core(q, k_buf, v_buf, context, lse, batch, seq_len, num_heads, num_kv_heads,
                      head_dim, total_seq, start_pos, scale);
    free(k_buf);
    free(v_buf);
}

/* Same computation with the cache held in paged form [rows, Hkv, D]: the
 * gather walks the block table (address formula of
 * tools/test_paged_flash_attention.mm:41-47) and produces the identical
 * [total_seq, Hkv, D] float arrays, so results equal the contiguous path bit
 * for bit. */
void go_attention_paged(const float *q, const uint16_t *pool_k, const uint16_t *pool_v,
                        const int32_t *table, int block_size, float *context, float *lse,
                        int batch, int seq_len, int num_heads, int num_kv_heads, int head_dim,
                        int total_seq, int start_pos, float scale)
{
    size_t n = (size_t)total_seq * num_kv_heads * head_dim;
    float *k_buf = (float *)malloc(n * sizeof(float));
    float *v_buf = (float *)malloc(n * sizeof(float));
    for (int s = 0; s < total_seq; s++) {
        size_t row = go_phys_row(table, block_size, s);
        for (int h = 0; h < num_kv_heads; h++)
            for (int d = 0; d < head_dim; d++) {
                size_t si = (row * num_kv_heads + h) * head_dim + d;
                size_t di = ((size_t)s * num_kv_heads + h) * head_dim + d;
                k_buf[di] = go_fp16_to_fp32(pool_k[si]);
                v_buf[di] = go_fp16_to_fp32(pool_v[si]);
            }
    }
    if (scale <= 0) scale = 1.0f / sqrtf((float)head_dim);
    go_attention_core(q, k_buf, v_buf, context, lse, batch, seq_len, num_heads, num_kv_heads,
                      head_dim, total_seq, start_pos, scale);
    free(k_buf);
    free(v_buf);
}

/* Batched paged decode: `batch` independent sequences, one query token each,
 * every sequence run through go_attention_paged with seq_len 1 and
 * start_pos = len-1 (all cached keys visible).  Layouts follow
 * include/granite/metal_compute.h:906-920: q/out [B, Hq, D], tables
 * [B, max_blocks], seq_lens [B].  A sequence of length 0 is skipped
 * (metal_shaders_attention.h:2186-2304). */
void go_batched_paged_decode(const float *q, const uint16_t *pool_k, const uint16_t *pool_v,
                             const int32_t *tables, const int32_t *seq_lens, float *out,
                             float *lse, int batch, int num_heads, int num_kv_heads,
                             int head_dim, int block_size, int max_blocks, float scale)
{
    for (int b = 0; b < batch; b++) {
        int len = seq_lens[b];
        if (len <= 0) continue;
        go_attention_paged(q + (size_t)b * num_heads * head_dim, pool_k, pool_v,
                           tables + (size_t)b * max_blocks, block_size,
                           out + (size_t)b * num_heads * head_dim,
                           lse ? lse + (size_t)b * num_heads : NULL, 1, 1, num_heads,
                           num_kv_heads, head_dim, len, len - 1, scale);
    }
}

/* ------------------------------------------------------------------------- */
/* Tree attention (transformer.mm:822-840, 1978-2126)                        */
/* ------------------------------------------------------------------------- */

/* transformer.mm:822-840: mask[i][i] = 1, then every ancestor reached by
 * walking parent[].  mask is num_nodes*num_nodes bytes.  The reference has no
 * cycle guard; inputs must satisfy parent[i] < i.  Returns -1 when a parent
 * is outside [-1, num_nodes) (transformer.mm:806-813). */
int go_tree_mask(const int32_t *parent, int num_nodes, uint8_t *mask)
{
    for (int i = 0; i < num_nodes; i++)
        if (parent[i] < -1 || parent[i] >= num_nodes) return -1;
    memset(mask, 0, (size_t)num_nodes * num_nodes);
    for (int i = 0; i < num_nodes; i++) {
        mask[(size_t)i * num_nodes + i] = 1;
        int current = parent[i];
        while (current >= 0 && current < num_nodes) {
            mask[(size_t)i * num_nodes + current] = 1;
            current = parent[current];
        }
    }
    return 0;
}

struct go_tree_job {
    const float *q;        /* [B, N, Hq, D] */
    const float *k_cached; /* [cached_len, Hkv, D] */
    const float *v_cached;
    const float *k_tree;   /* [B, N, Hkv, D] */
    const float *v_tree;
    const uint8_t *mask;   /* [N, N] */
    float *context;        /* [B, N, Hq*D] */
    float *lse;            /* [B, Hq, N] or NULL */
    int batch, num_nodes, num_heads, num_kv_heads, head_dim, cached_len;
    float scale;
};

/* transformer.mm:2051-2126, one (b, h, q_node) item. */
static void go_tree_item(size_t work_idx_u, void *arg)
{
    const struct go_tree_job *j = (const struct go_tree_job *)arg;
    int work_idx = (int)work_idx_u;
    int num_heads = j->num_heads, num_nodes = j->num_nodes, head_dim = j->head_dim;
    int num_kv_heads = j->num_kv_heads, cached_len = j->cached_len;
    int heads_per_kv = num_heads / num_kv_heads;
    int total_kv = cached_len + num_nodes;

    int b = work_idx / (num_heads * num_nodes);
    int rem = work_idx % (num_heads * num_nodes);
    int h = rem / num_nodes;
    int q_node = rem % num_nodes;
    int kv_h = h / heads_per_kv;

    float *scores = (float *)malloc((size_t)total_kv * sizeof(float));
    const float *q_vec = j->q + ((size_t)(b * num_nodes + q_node) * num_heads + h) * head_dim;

    for (int k_pos = 0; k_pos < cached_len; k_pos++) {
        const float *k_vec = j->k_cached + ((size_t)k_pos * num_kv_heads + kv_h) * head_dim;
        float dot = 0;
        for (int d = 0; d < head_dim; d++) dot += q_vec[d] * k_vec[d];
        scores[k_pos] = dot * j->scale;
    }
    for (int k_node = 0; k_node < num_nodes; k_node++) {
        int k_pos_in_total = cached_len + k_node;
        if (j->mask[(size_t)q_node * num_nodes + k_node]) {
            const float *k_vec =
                j->k_tree + ((size_t)(b * num_nodes + k_node) * num_kv_heads + kv_h) * head_dim;
            float dot = 0;
            for (int d = 0; d < head_dim; d++) dot += q_vec[d] * k_vec[d];
            scores[k_pos_in_total] = dot * j->scale;
        } else {
            scores[k_pos_in_total] = -INFINITY;
        }
    }

    float max_score = scores[0];
    for (int i = 1; i < total_kv; i++)
        if (scores[i] > max_score) max_score = scores[i];

    if (j->lse) {
        double acc = 0.0;
        for (int i = 0; i < total_kv; i++) acc += exp((double)scores[i] - (double)max_score);
        j->lse[((size_t)b * num_heads + h) * num_nodes + q_node] =
            (float)((double)max_score + log(acc));
    }

    float sum = 0;
    for (int i = 0; i < total_kv; i++) {
        scores[i] = expf(scores[i] - max_score);
        sum += scores[i];
    }
    float inv_sum = 1.0f / sum;
    for (int i = 0; i < total_kv; i++) scores[i] *= inv_sum;

    float *ctx = j->context + ((size_t)(b * num_nodes + q_node) * num_heads + h) * head_dim;
    for (int d = 0; d < head_dim; d++) ctx[d] = 0.0f;
    for (int v_pos = 0; v_pos < cached_len; v_pos++) {
        const float *v_vec = j->v_cached + ((size_t)v_pos * num_kv_heads + kv_h) * head_dim;
        float w = scores[v_pos];
        for (int d = 0; d < head_dim; d++) ctx[d] += w * v_vec[d];
    }
    for (int v_node = 0; v_node < num_nodes; v_node++) {
        const float *v_vec =
            j->v_tree + ((size_t)(b * num_nodes + v_node) * num_kv_heads + kv_h) * head_dim;
        float w = scores[cached_len + v_node];
        for (int d = 0; d < head_dim; d++) ctx[d] += w * v_vec[d];
    }
    free(scores);
}

/* Tree attention with the prefix in the contiguous cache [Hkv, max_seq, D]
 * (table == NULL) or in a paged pool [rows, Hkv, D] (table != NULL).  Tree
 * K/V are floats [B, N, Hkv, D] as on the reference CPU path. */
int go_attention_tree(const float *q, const uint16_t *cache_k, const uint16_t *cache_v,
                      const int32_t *table, int block_size, int max_seq, const float *k_tree,
                      const float *v_tree, const int32_t *parent, float *context, float *lse,
                      int batch, int num_nodes, int num_heads, int num_kv_heads, int head_dim,
                      int cached_len, float scale)
{
    uint8_t *mask = (uint8_t *)malloc((size_t)num_nodes * num_nodes + 1);
    if (go_tree_mask(parent, num_nodes, mask) != 0) {
        free(mask);
        return -1;
    }
    size_t n = (size_t)cached_len * num_kv_heads * head_dim;
    float *k_buf = (float *)malloc((n + 1) * sizeof(float));
    float *v_buf = (float *)malloc((n + 1) * sizeof(float));
    for (int h = 0; h < num_kv_heads; h++)
        for (int s = 0; s < cached_len; s++) {
            size_t src_row = table ? go_phys_row(table, block_size, s) * num_kv_heads + h
                                   : (size_t)h * max_seq + s;
            for (int d = 0; d < head_dim; d++) {
                size_t di = ((size_t)s * num_kv_heads + h) * head_dim + d;
                k_buf[di] = go_fp16_to_fp32(cache_k[src_row * head_dim + d]);
                v_buf[di] = go_fp16_to_fp32(cache_v[src_row * head_dim + d]);
            }
        }
    if (scale <= 0) scale = 1.0f / sqrtf((float)head_dim);
    struct go_tree_job job = {q, k_buf, v_buf, k_tree, v_tree, mask, context, lse, batch,
                              num_nodes, num_heads, num_kv_heads, head_dim, cached_len, scale};
    size_t total_work = (size_t)batch * num_heads * num_nodes;
    go_parallel_for(total_work, (size_t)go_get_num_threads(), go_tree_item, &job);
    free(k_buf);
    free(v_buf);
    free(mask);
    return 0;
}

/* ------------------------------------------------------------------------- */
/* Block manager and paged cache bookkeeping (paged_kv_cache.cpp)            */
/* ------------------------------------------------------------------------- */

struct go_block_manager {
    int num_blocks, block_size, num_free;
    int *free_list;
    uint8_t *allocated;
};

/* paged_kv_cache.cpp:17-36: free list holds 0..N-1; allocation pops from the
 * end, so a fresh pool hands out N-1 first. */
struct go_block_manager *go_block_manager_new(int num_blocks, int block_size)
{
    if (num_blocks <= 0 || block_size <= 0) return NULL;
    struct go_block_manager *m = (struct go_block_manager *)malloc(sizeof(*m));
    m->num_blocks = num_blocks;
    m->block_size = block_size;
    m->num_free = num_blocks;
    m->free_list = (int *)malloc((size_t)num_blocks * sizeof(int));
    m->allocated = (uint8_t *)calloc((size_t)num_blocks, 1);
    for (int i = 0; i < num_blocks; i++) m->free_list[i] = i;
    return m;
}

void go_block_manager_delete(struct go_block_manager *m)
{
    if (!m) return;
    free(m->free_list);
    free(m->allocated);
    free(m);
}

/* paged_kv_cache.cpp:73-82 */
int go_block_manager_allocate(struct go_block_manager *m)
{
    if (m->num_free == 0) return -1;
    int idx = m->free_list[--m->num_free];
    m->allocated[idx] = 1;
    return idx;
}

/* paged_kv_cache.cpp:84-98: out-of-range and double frees are ignored. */
void go_block_manager_free(struct go_block_manager *m, int idx)
{
    if (idx < 0 || idx >= m->num_blocks) return;
    if (!m->allocated[idx]) return;
    m->allocated[idx] = 0;
    m->free_list[m->num_free++] = idx;
}

int go_block_manager_num_free(const struct go_block_manager *m) { return m->num_free; }

struct go_paged_cache {
    struct go_block_manager *mgr;
    int *table;
    int num_blocks, cap, seq_len;
};

struct go_paged_cache *go_paged_cache_new(struct go_block_manager *mgr)
{
    struct go_paged_cache *c = (struct go_paged_cache *)calloc(1, sizeof(*c));
    c->mgr = mgr;
    return c;
}

void go_paged_cache_delete(struct go_paged_cache *c)
{
    if (!c) return;
    free(c->table);
    free(c);
}

/* paged_kv_cache.cpp:120-143: blocks_needed = ceil((len+n)/bs); on exhaustion
 * returns 0 with the blocks obtained so far kept and seq_len unchanged. */
int go_paged_cache_append_tokens(struct go_paged_cache *c, int num_tokens)
{
    int bs = c->mgr->block_size;
    int new_len = c->seq_len + num_tokens;
    int needed = (new_len + bs - 1) / bs;
    while (c->num_blocks < needed) {
        int blk = go_block_manager_allocate(c->mgr);
        if (blk < 0) return 0;
        if (c->num_blocks == c->cap) {
            c->cap = c->cap ? c->cap * 2 : 16;
            c->table = (int *)realloc(c->table, (size_t)c->cap * sizeof(int));
        }
        c->table[c->num_blocks++] = blk;
    }
    c->seq_len = new_len;
    return 1;
}

/* paged_kv_cache.cpp:169-187 */
void go_paged_cache_truncate(struct go_paged_cache *c, int new_len)
{
    if (new_len >= c->seq_len) return;
    int bs = c->mgr->block_size;
    int needed = (new_len + bs - 1) / bs;
    if (new_len == 0) needed = 0;
    while (c->num_blocks > needed) go_block_manager_free(c->mgr, c->table[--c->num_blocks]);
    c->seq_len = new_len;
}

/* paged_kv_cache.cpp:108-118 */
void go_paged_cache_release(struct go_paged_cache *c)
{
    for (int i = 0; i < c->num_blocks; i++) go_block_manager_free(c->mgr, c->table[i]);
    c->num_blocks = 0;
    c->seq_len = 0;
}

int go_paged_cache_seq_len(const struct go_paged_cache *c) { return c->seq_len; }
int go_paged_cache_num_blocks(const struct go_paged_cache *c) { return c->num_blocks; }
const int *go_paged_cache_table(const struct go_paged_cache *c) { return c->table; }

/* paged_kv_cache.cpp:145-161 */
int go_paged_cache_physical_block(const struct go_paged_cache *c, int pos)
{
    int lb = pos / c->mgr->block_size;
    if (lb >= c->num_blocks) return -1;
    return c->table[lb];
}

int go_paged_cache_block_offset(const struct go_paged_cache *c, int pos)
{
    return pos % c->mgr->block_size;
}

/* ------------------------------------------------------------------------- */
/* Rotary position embedding                                                 */
/* ------------------------------------------------------------------------- */

/* RoPECache::initialize, src/llm/rope.cpp:5-22: cos/sin [max_seq_len, head_dim/2],
 * freq = 1 / pow(theta, 2i / head_dim) and angle = pos * freq, all in float (the
 * reference calls std::pow / std::cos / std::sin on float arguments). */
void go_rope_table(float *cos_out, float *sin_out, int max_seq_len, int head_dim, float theta)
{
    int half_dim = head_dim / 2;
    for (int pos = 0; pos < max_seq_len; pos++) {
        for (int i = 0; i < half_dim; i++) {
            float freq = 1.0f / powf(theta, (float)(2 * i) / head_dim);
            float angle = (float)pos * freq;
            cos_out[(size_t)pos * half_dim + i] = cosf(angle);
            sin_out[(size_t)pos * half_dim + i] = sinf(angle);
        }
    }
}

/* RoPECache::apply, src/llm/rope.cpp:24-92, on one tensor [seq_len, num_heads, head_dim]
 * (the reference runs the same loop over Q and then over K).  Returns -1 for the range
 * error of rope.cpp:34-38. */
int go_rope_apply(float *x, int seq_len, int num_heads, int head_dim, int start_pos,
                  const float *cos_t, const float *sin_t, int max_seq_len)
{
    if (start_pos + seq_len > max_seq_len) return -1;
    int half_dim = head_dim / 2;
    for (int s = 0; s < seq_len; s++) {
        int pos = start_pos + s;
        for (int h = 0; h < num_heads; h++) {
            float *p = x + ((size_t)s * num_heads + h) * head_dim;
            for (int i = 0; i < half_dim; i++) {
                float c = cos_t[(size_t)pos * half_dim + i];
                float sn = sin_t[(size_t)pos * half_dim + i];
                float x0 = p[2 * i];
                float x1 = p[2 * i + 1];
                p[2 * i] = x0 * c - x1 * sn;
                p[2 * i + 1] = x0 * sn + x1 * c;
            }
        }
    }
    return 0;
}


/* ------------------------------------------------------------------------- */
/* Q4_K weights and the projections either side of attention                 */
/* ------------------------------------------------------------------------- */

/* A Q4_K super-block holds 256 weights in 144 bytes: d and dmin (half), 12 bytes of packed
 * 6-bit scales and minima for 8 sub-blocks of 32, 128 bytes of 4-bit values
 * (src/model/gguf.cpp:952-960). */
#define GO_QK_K 256
#define GO_Q4K_BLOCK_BYTES 144

/* gguf.cpp:963-971 (ggml's get_scale_min_k4): scale and minimum of sub-block j (0..7). */
void go_q4k_scale_min(int j, const uint8_t *q, uint8_t *sc, uint8_t *m)
{
    if (j < 4) {
        *sc = q[j] & 63;
        *m = q[j + 4] & 63;
    } else {
        *sc = (uint8_t)((q[j + 4] & 0xF) | ((q[j - 4] >> 6) << 4));
        *m = (uint8_t)((q[j + 4] >> 4) | ((q[j] >> 6) << 4));
    }
}

/* gguf.cpp:973-1016: weights of `numel` values (whole super-blocks).  out_f32 receives
 * d * sc * q - dmin * m as the reference forms it in float; out_f16 what the reference
 * stores, that value through its truncating fp32_to_fp16.  Either may be NULL. */
void go_q4k_dequantize(const uint8_t *blocks, size_t numel, float *out_f32, uint16_t *out_f16)
{
    size_t num_blocks = (numel + GO_QK_K - 1) / GO_QK_K;
    const uint8_t *src = blocks;
    for (size_t b = 0; b < num_blocks; b++) {
        uint16_t d_bits, dmin_bits;
        memcpy(&d_bits, src, 2);
        memcpy(&dmin_bits, src + 2, 2);
        float d = go_fp16_to_fp32(d_bits);
        float dmin = go_fp16_to_fp32(dmin_bits);
        const uint8_t *scales = src + 4;
        const uint8_t *qs = src + 16;
        int is = 0;
        for (int j = 0; j < GO_QK_K; j += 64) {
            uint8_t sc, m;
            go_q4k_scale_min(is, scales, &sc, &m);
            float d1 = d * (float)sc, m1 = dmin * (float)m;
            go_q4k_scale_min(is + 1, scales, &sc, &m);
            float d2 = d * (float)sc, m2 = dmin * (float)m;
            for (int l = 0; l < 32; l++) {
                size_t idx = b * GO_QK_K + j + l;
                if (idx >= numel) break;
                float val = d1 * (float)(qs[l] & 0xF) - m1;
                if (out_f32) out_f32[idx] = val;
                if (out_f16) out_f16[idx] = go_fp32_to_fp16(val);
            }
            for (int l = 0; l < 32; l++) {
                size_t idx = b * GO_QK_K + j + 32 + l;
                if (idx >= numel) break;
                float val = d2 * (float)(qs[l] >> 4) - m2;
                if (out_f32) out_f32[idx] = val;
                if (out_f16) out_f16[idx] = go_fp32_to_fp16(val);
            }
            qs += 32;
            is += 2;
        }
        src += GO_Q4K_BLOCK_BYTES;
    }
}

/* math_ops.cpp:67-103, the branch without Accelerate: B [N, K] half widened to float,
 * C[m][n] = sum_k A[m][k] * B[n][k], summed in float in the order of k.  This is how the
 * reference's CPU attention projects Q, K and V (transformer.mm:1623-1634) from weights
 * that were dequantised to half when the model was loaded. */
void go_matmul_transb_fp16(const float *A, const uint16_t *B_fp16, float *C, int M, int N, int K)
{
    float *B = (float *)malloc((size_t)N * K * sizeof(float));
    go_fp16_to_fp32_array(B_fp16, B, (size_t)N * K);
    for (int m = 0; m < M; m++)
        for (int n = 0; n < N; n++) {
            float sum = 0;
            for (int k = 0; k < K; k++) sum += A[(size_t)m * K + k] * B[(size_t)n * K + k];
            C[(size_t)m * N + n] = sum;
        }
    free(B);
}

struct go_matvec_job {
    const float *x;
    const uint8_t *W;
    float *y;
    int K, N, batch;
};

static void go_matvec_q4k_row(size_t n, void *arg)
{
    const struct go_matvec_job *job = (const struct go_matvec_job *)arg;
    const int K = job->K;
    float *w = (float *)malloc((size_t)K * sizeof(float));
    go_q4k_dequantize(job->W + n * (size_t)(K / GO_QK_K) * GO_Q4K_BLOCK_BYTES, (size_t)K, w, NULL);
    for (int b = 0; b < job->batch; b++) {
        const float *x = job->x + (size_t)b * K;
        float sum = 0;
        for (int k = 0; k < K; k++) sum += x[k] * w[k];
        job->y[(size_t)b * job->N + n] = sum;
    }
    free(w);
}

/* y[b][n] = sum_k x[b][k] * w[n][k] with W [N, K/256] Q4_K super-blocks, the weights in
 * float exactly as the dequantisation formula gives them (the GPU path multiplies the
 * 4-bit values directly, metal_shaders_quant.h:244-280; it never rounds a weight to
 * half).  Rows are spread over threads as the reference spreads work (parallel_for). */
void go_matvec_q4k(const float *x, const uint8_t *W, float *y, int K, int N, int batch)
{
    struct go_matvec_job job = {x, W, y, K, N, batch};
    go_parallel_for((size_t)N, (size_t)go_get_num_threads(), go_matvec_q4k_row, &job);
}
