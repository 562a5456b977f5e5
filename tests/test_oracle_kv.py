"""Pins the oracle's KV append / gather and block bookkeeping
(src/llm/kv_cache.cpp:55-107, src/llm/paged_kv_cache.cpp:17-187,
metal_shaders_attention.h:102-125 and :2142-2176) through invariants and
closed forms."""
import numpy as np
import pytest

import ref64

SENT = 0xBEEF


def test_contiguous_append_f16_invariant(oracle):
    rng = np.random.default_rng(1)
    hkv, d, max_seq, cur, new = 3, 8, 20, 5, 7
    cache = np.full((hkv, max_seq, d), SENT, np.uint16)
    src = rng.integers(0, 65536, (hkv, new, d)).astype(np.uint16)
    rc = oracle.lib.go_kv_cache_append_f16(cache.reshape(-1), src.reshape(-1), hkv, d, cur, new, max_seq)
    assert rc == 0
    assert np.array_equal(cache[:, cur:cur + new], src)
    untouched = np.ones(max_seq, bool)
    untouched[cur:cur + new] = False
    assert np.all(cache[:, untouched] == SENT)


def test_contiguous_append_overflow_is_rejected(oracle):
    cache = np.full((1, 4, 8), SENT, np.uint16)
    src = np.zeros((1, 2, 8), np.uint16)
    assert oracle.lib.go_kv_cache_append_f16(cache.reshape(-1), src.reshape(-1), 1, 8, 3, 2, 4) == -1
    assert np.all(cache == SENT)   # kv_cache.cpp:61-65: error before any write
    assert oracle.lib.go_kv_cache_append_f16(cache.reshape(-1), src.reshape(-1), 1, 8, 2, 2, 4) == 0


def test_contiguous_append_f32_transposes_and_truncates(oracle):
    rng = np.random.default_rng(2)
    hkv, d, max_seq, cur, new = 2, 8, 9, 1, 4
    src = (rng.standard_normal((new, hkv, d)) * 3).astype(np.float32)   # [new, Hkv, D]
    cache = np.full((hkv, max_seq, d), SENT, np.uint16)
    assert oracle.lib.go_kv_cache_append_f32(cache.reshape(-1), src.reshape(-1), hkv, d, cur, new, max_seq) == 0
    want = oracle.fp32_to_fp16(np.transpose(src, (1, 0, 2)).copy())
    assert np.array_equal(cache[:, cur:cur + new], want)
    assert np.all(cache[:, :cur] == SENT) and np.all(cache[:, cur + new:] == SENT)


def test_paged_append_then_gather_is_identity(oracle):
    rng = np.random.default_rng(3)
    hkv, d, bs, nblk_pool = 2, 8, 4, 9
    total, start, new = 13, 6, 7
    nblk = (total + bs - 1) // bs
    table = rng.permutation(nblk_pool)[:nblk].astype(np.int32)
    pool = np.full((nblk_pool * bs, hkv, d), SENT, np.uint16)
    src = rng.integers(0, 0x7C00, (hkv, new, d)).astype(np.uint16)       # [Hkv, new, D]
    oracle.lib.go_paged_kv_cache_append_f16(pool.reshape(-1), src.reshape(-1), table, hkv, d,
                                            start, new, bs, d, new * d)
    cache = np.full((hkv, 16, d), 0, np.uint16)
    oracle.lib.go_paged_gather_f16(cache.reshape(-1), pool.reshape(-1), table, hkv, d, total, bs, 16)
    assert np.array_equal(cache[:, start:total], src)
    assert np.all(cache[:, :start] == SENT)                               # never written
    # rows outside the touched positions keep the sentinel
    pos = np.arange(start, total)
    rows = table[pos // bs].astype(np.int64) * bs + pos % bs
    mask = np.ones(nblk_pool * bs, bool)
    mask[rows] = False
    assert np.all(pool[mask] == SENT)
    # independent gather agrees
    assert np.array_equal(ref64.gather_paged(pool, table, bs, total)[start:],
                          np.transpose(src, (1, 0, 2)))


def test_paged_equals_contiguous_when_table_is_identity(oracle):
    rng = np.random.default_rng(4)
    hkv, d, bs, new = 2, 8, 4, 10
    src = (rng.standard_normal((hkv, new, d)) * 2).astype(np.float32)
    table = np.arange(3, dtype=np.int32)
    pool = np.zeros((12, hkv, d), np.uint16)
    oracle.lib.go_paged_kv_cache_append_f32(pool.reshape(-1), src.reshape(-1), table, hkv, d, 0, new, bs)
    assert np.array_equal(np.transpose(pool[:new], (1, 0, 2)), oracle.fp32_to_fp16(src))


# ---- block manager / paged cache --------------------------------------------

def test_block_manager_lifo_order(oracle):
    L = oracle.lib
    m = L.go_block_manager_new(5, 16)
    got = [L.go_block_manager_allocate(m) for _ in range(5)]
    assert got == [4, 3, 2, 1, 0]                       # paged_kv_cache.cpp:30-36, 73-82
    assert L.go_block_manager_allocate(m) == -1
    L.go_block_manager_free(m, 2)
    L.go_block_manager_free(m, 2)                        # double free ignored
    L.go_block_manager_free(m, 99)                       # out of range ignored
    L.go_block_manager_free(m, -1)
    assert L.go_block_manager_num_free(m) == 1
    assert L.go_block_manager_allocate(m) == 2           # last freed comes back first
    L.go_block_manager_free(m, 0)
    L.go_block_manager_free(m, 4)
    assert [L.go_block_manager_allocate(m), L.go_block_manager_allocate(m)] == [4, 0]
    L.go_block_manager_delete(m)
    assert not L.go_block_manager_new(0, 16) and not L.go_block_manager_new(4, 0)


def test_paged_cache_append_truncate_release(oracle):
    L = oracle.lib
    m = L.go_block_manager_new(6, 4)
    c = L.go_paged_cache_new(m)
    assert L.go_paged_cache_append_tokens(c, 5) == 1     # ceil(5/4) = 2 blocks
    assert L.go_paged_cache_num_blocks(c) == 2 and L.go_paged_cache_seq_len(c) == 5
    assert [L.go_paged_cache_table(c)[i] for i in range(2)] == [5, 4]
    assert L.go_paged_cache_append_tokens(c, 3) == 1     # 8 tokens still 2 blocks
    assert L.go_paged_cache_num_blocks(c) == 2
    assert L.go_paged_cache_append_tokens(c, 1) == 1     # 9 -> 3 blocks
    assert L.go_paged_cache_physical_block(c, 8) == 3 and L.go_paged_cache_block_offset(c, 9) == 1
    assert L.go_paged_cache_physical_block(c, 12) == -1
    L.go_paged_cache_truncate(c, 4)                      # keeps ceil(4/4) = 1 block
    assert L.go_paged_cache_num_blocks(c) == 1 and L.go_block_manager_num_free(m) == 5
    L.go_paged_cache_truncate(c, 10)                     # growing is a no-op
    assert L.go_paged_cache_seq_len(c) == 4
    # exhaustion keeps what was obtained and leaves the length (paged_kv_cache.cpp:131-139)
    assert L.go_paged_cache_append_tokens(c, 100) == 0
    assert L.go_paged_cache_seq_len(c) == 4 and L.go_paged_cache_num_blocks(c) == 6
    assert L.go_block_manager_num_free(m) == 0
    L.go_paged_cache_release(c)
    assert L.go_block_manager_num_free(m) == 6 and L.go_paged_cache_seq_len(c) == 0
    L.go_paged_cache_truncate(c, 0)
    L.go_paged_cache_delete(c)
    L.go_block_manager_delete(m)
