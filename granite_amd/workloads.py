"""Seeded synthetic inputs for the five attention workloads the benchmark and
the parity tests run (shapes of the reference's decode, prefill, paged decode,
tree and chunked-prefill paths).  Pure numpy, host side only: the same arrays
are handed to the GPU entry points and to the CPU checker.

All values are N(0,1) drawn in float32 from numpy's PCG64 generator with the
seed given, then rounded to half (nearest-even) wherever the tensor is half
precision, so CPU and GPU start from identical bits.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Optional

import numpy as np

SEED_BASE = 0x6772616E00  # "gran\0"


def _normal(rng: np.random.Generator, shape, scale: float = 1.0) -> np.ndarray:
    x = rng.standard_normal(shape, dtype=np.float32)
    if scale != 1.0:
        x *= np.float32(scale)
    return x


def _normal_f16(rng: np.random.Generator, shape, scale: float = 1.0) -> np.ndarray:
    """Large tensors are drawn in slabs to bound the float32 temporary."""
    shape = tuple(int(s) for s in shape)
    out = np.empty(shape, dtype=np.float16)
    flat = out.reshape(-1)
    step = 1 << 26
    for i in range(0, flat.size, step):
        n = min(step, flat.size - i)
        flat[i:i + n] = _normal(rng, n, scale).astype(np.float16)
    return out


@dataclass
class DecodeContiguousCase:
    """Single-token decode over a contiguous cache [Hkv, max_seq, D]."""
    q: np.ndarray          # [Hq, D] float32
    k_cache: np.ndarray    # [Hkv, max_seq, D] float16
    v_cache: np.ndarray
    seq_kv: int
    max_seq: int
    num_heads: int
    num_kv_heads: int
    head_dim: int
    scale: float

    def algorithmic_bytes(self) -> int:
        kv = 2 * self.num_kv_heads * self.seq_kv * self.head_dim * 2
        return self.q.nbytes + kv + self.num_heads * self.head_dim * 4 + self.num_heads * 4

    def flops(self) -> int:
        return 4 * self.num_heads * self.head_dim * self.seq_kv


def make_decode_contiguous(seed=SEED_BASE + 0, num_heads=32, num_kv_heads=8, head_dim=128,
                           seq_kv=512, max_seq=None) -> DecodeContiguousCase:
    rng = np.random.default_rng(seed)
    max_seq = max_seq or seq_kv
    q = _normal(rng, (num_heads, head_dim))
    k = _normal_f16(rng, (num_kv_heads, max_seq, head_dim))
    v = _normal_f16(rng, (num_kv_heads, max_seq, head_dim))
    return DecodeContiguousCase(q, k, v, seq_kv, max_seq, num_heads, num_kv_heads, head_dim,
                                float(1.0 / np.sqrt(np.float32(head_dim))))


@dataclass
class PrefillCase:
    """Causal prefill: Q [S, Hq, D] half, K/V in cache layout [Hkv, max_seq, D] half."""
    q: np.ndarray
    k_cache: np.ndarray
    v_cache: np.ndarray
    seq: int
    max_seq: int
    num_heads: int
    num_kv_heads: int
    head_dim: int
    scale: float

    def flops(self) -> int:
        s = self.seq
        return 4 * self.num_heads * self.head_dim * (s * (s + 1) // 2)

    def algorithmic_bytes(self) -> int:
        return 2 * self.q.nbytes + self.k_cache.nbytes + self.v_cache.nbytes


def make_prefill(seed=SEED_BASE + 1, seq=2048, num_heads=32, num_kv_heads=8, head_dim=128,
                 max_seq=None) -> PrefillCase:
    rng = np.random.default_rng(seed)
    max_seq = max_seq or seq
    q = _normal_f16(rng, (seq, num_heads, head_dim))
    k = _normal_f16(rng, (num_kv_heads, max_seq, head_dim))
    v = _normal_f16(rng, (num_kv_heads, max_seq, head_dim))
    return PrefillCase(q, k, v, seq, max_seq, num_heads, num_kv_heads, head_dim,
                       float(1.0 / np.sqrt(np.float32(head_dim))))


@dataclass
class PagedDecodeCase:
    """Batched paged decode: one query token per sequence."""
    q: np.ndarray            # [B, Hq, D] float16
    k_pool: np.ndarray       # [num_blocks*bs, Hkv, D] float16
    v_pool: np.ndarray
    block_tables: np.ndarray  # [B, max_blocks] int32 (unused entries = 0)
    seq_lens: np.ndarray     # [B] int32
    block_size: int
    max_blocks: int
    num_blocks: int
    num_heads: int
    num_kv_heads: int
    head_dim: int
    scale: float

    @property
    def batch(self) -> int:
        return int(self.seq_lens.shape[0])

    def algorithmic_bytes(self) -> int:
        """K and V rows counted once per KV head, plus Q, output, LSE and the
        block-table entries actually used (the reference tool's convention,
        tools/benchmark_attention.mm:136-140)."""
        tokens = int(self.seq_lens.sum())
        kv = tokens * 2 * self.num_kv_heads * self.head_dim * 2
        blocks = int(((self.seq_lens + self.block_size - 1) // self.block_size).sum())
        b = self.batch
        return (kv + self.q.nbytes + b * self.num_heads * self.head_dim * 4 +
                b * self.num_heads * 4 + blocks * 4)

    def flops(self) -> int:
        return 4 * self.num_heads * self.head_dim * int(self.seq_lens.sum())


def make_paged_decode(seed=SEED_BASE + 2, batch=64, num_heads=32, num_kv_heads=8, head_dim=128,
                      block_size=16, ctx_min=256, ctx_max=8192, pool_slack=1.25,
                      seq_lens: Optional[np.ndarray] = None) -> PagedDecodeCase:
    rng = np.random.default_rng(seed)
    if seq_lens is None:
        seq_lens = rng.integers(ctx_min, ctx_max + 1, size=batch, dtype=np.int64)
    seq_lens = np.asarray(seq_lens, dtype=np.int32)
    batch = int(seq_lens.shape[0])
    blocks_per_seq = (seq_lens.astype(np.int64) + block_size - 1) // block_size
    used = int(blocks_per_seq.sum())
    num_blocks = max(int(np.ceil(pool_slack * used)), 1)
    max_blocks = max(int((max(ctx_max, int(seq_lens.max(initial=1))) + block_size - 1)
                         // block_size), 1)
    perm = rng.permutation(num_blocks).astype(np.int32)
    tables = np.zeros((batch, max_blocks), dtype=np.int32)
    at = 0
    for b in range(batch):
        nb = int(blocks_per_seq[b])
        tables[b, :nb] = perm[at:at + nb]
        at += nb
    q = _normal_f16(rng, (batch, num_heads, head_dim))
    k_pool = _normal_f16(rng, (num_blocks * block_size, num_kv_heads, head_dim))
    v_pool = _normal_f16(rng, (num_blocks * block_size, num_kv_heads, head_dim))
    return PagedDecodeCase(q, k_pool, v_pool, tables, seq_lens, block_size, max_blocks, num_blocks,
                           num_heads, num_kv_heads, head_dim,
                           float(1.0 / np.sqrt(np.float32(head_dim))))


def random_tree(rng: np.random.Generator, num_nodes=64, max_children=4, max_depth=8) -> np.ndarray:
    """parent[0] = -1; node i>0 hangs under a uniformly chosen earlier node that
    still has fewer than max_children children and depth < max_depth, so
    parent[i] < i always holds (what the reference's mask builder relies on,
    src/llm/transformer.mm:829-839)."""
    parent = np.full(num_nodes, -1, dtype=np.int32)
    depth = np.zeros(num_nodes, dtype=np.int32)
    children = np.zeros(num_nodes, dtype=np.int32)
    for i in range(1, num_nodes):
        cand = [j for j in range(i) if children[j] < max_children and depth[j] < max_depth]
        if not cand:
            parent[i] = -1
            continue
        j = int(cand[int(rng.integers(0, len(cand)))])
        parent[i] = j
        depth[i] = depth[j] + 1
        children[j] += 1
    return parent


@dataclass
class TreeCase:
    """Tree attention over a paged prefix plus `num_nodes` draft tokens."""
    q: np.ndarray            # [Hq, N, D] float32, values representable in half
    k_pool: np.ndarray       # paged prefix
    v_pool: np.ndarray
    block_table: np.ndarray  # [ceil(prefix/bs)] int32
    k_tree: np.ndarray       # [Hkv, N, D] float16
    v_tree: np.ndarray
    parents: np.ndarray      # [N] int32
    prefix_len: int
    block_size: int
    num_heads: int
    num_kv_heads: int
    head_dim: int
    scale: float

    @property
    def num_nodes(self) -> int:
        return int(self.parents.shape[0])

    def depths(self) -> np.ndarray:
        d = np.zeros(self.num_nodes, dtype=np.int64)
        for i in range(self.num_nodes):
            if self.parents[i] >= 0:
                d[i] = d[self.parents[i]] + 1
        return d

    def flops(self) -> int:
        vis = int((self.prefix_len + self.depths() + 1).sum())
        return 4 * self.num_heads * self.head_dim * vis

    def algorithmic_bytes(self) -> int:
        kv = self.prefix_len * 2 * self.num_kv_heads * self.head_dim * 2
        return kv + self.k_tree.nbytes + self.v_tree.nbytes + 2 * self.q.nbytes


def make_tree(seed=SEED_BASE + 3, prefix_len=4096, num_nodes=64, num_heads=32, num_kv_heads=8,
              head_dim=128, block_size=16, max_children=4, max_depth=8, pool_slack=1.25) -> TreeCase:
    rng = np.random.default_rng(seed)
    nblk = (prefix_len + block_size - 1) // block_size
    num_blocks = max(int(np.ceil(pool_slack * nblk)), 1)
    table = rng.permutation(num_blocks).astype(np.int32)[:nblk]
    parents = random_tree(rng, num_nodes, max_children, max_depth)
    q = _normal_f16(rng, (num_heads, num_nodes, head_dim)).astype(np.float32)
    k_pool = _normal_f16(rng, (num_blocks * block_size, num_kv_heads, head_dim))
    v_pool = _normal_f16(rng, (num_blocks * block_size, num_kv_heads, head_dim))
    k_tree = _normal_f16(rng, (num_kv_heads, num_nodes, head_dim))
    v_tree = _normal_f16(rng, (num_kv_heads, num_nodes, head_dim))
    return TreeCase(q, k_pool, v_pool, table, k_tree, v_tree, parents, prefix_len, block_size,
                    num_heads, num_kv_heads, head_dim, float(1.0 / np.sqrt(np.float32(head_dim))))


@dataclass
class ChunkedPrefillCase:
    """A chunk of `chunk` new tokens over `prefix_len` tokens already in a paged
    cache; the chunk's K/V are appended into fresh physical blocks first."""
    q: np.ndarray            # [chunk, Hq, D] float16
    k_new: np.ndarray        # [chunk, Hkv, D] float16
    v_new: np.ndarray
    k_pool: np.ndarray       # [num_blocks*bs, Hkv, D] float16, prefix filled, rest N(0,1)
    v_pool: np.ndarray
    block_table: np.ndarray  # [ceil((prefix+chunk)/bs)] int32
    prefix_len: int
    chunk: int
    block_size: int
    num_heads: int
    num_kv_heads: int
    head_dim: int
    scale: float

    def flops(self) -> int:
        c = self.chunk
        pairs = c * self.prefix_len + c * (c + 1) // 2
        return 4 * self.num_heads * self.head_dim * pairs

    def algorithmic_bytes(self) -> int:
        kv = (self.prefix_len + self.chunk) * 2 * self.num_kv_heads * self.head_dim * 2
        return kv + 2 * self.q.nbytes


def make_chunked_prefill(seed=SEED_BASE + 4, prefix_len=32768, chunk=512, num_heads=64,
                         num_kv_heads=8, head_dim=128, block_size=32, value_scale=0.5,
                         pool_slack=1.0625) -> ChunkedPrefillCase:
    rng = np.random.default_rng(seed)
    nblk = (prefix_len + chunk + block_size - 1) // block_size
    num_blocks = max(int(np.ceil(pool_slack * nblk)), nblk)
    table = rng.permutation(num_blocks).astype(np.int32)[:nblk]
    q = _normal_f16(rng, (chunk, num_heads, head_dim), value_scale)
    k_new = _normal_f16(rng, (chunk, num_kv_heads, head_dim), value_scale)
    v_new = _normal_f16(rng, (chunk, num_kv_heads, head_dim), value_scale)
    k_pool = _normal_f16(rng, (num_blocks * block_size, num_kv_heads, head_dim), value_scale)
    v_pool = _normal_f16(rng, (num_blocks * block_size, num_kv_heads, head_dim), value_scale)
    return ChunkedPrefillCase(q, k_new, v_new, k_pool, v_pool, table, prefix_len, chunk,
                              block_size, num_heads, num_kv_heads, head_dim,
                              float(1.0 / np.sqrt(np.float32(head_dim))))


# ---- Q4_K weights (the projections either side of attention) --------------------

QK_K = 256             # weights per super-block
Q4K_BLOCK_BYTES = 144  # half d, half dmin, 12 bytes of 6-bit scales / minima, 128 bytes of nibbles


def pack_q4k(d: np.ndarray, dmin: np.ndarray, scales: np.ndarray, mins: np.ndarray,
             q: np.ndarray) -> np.ndarray:
    """Q4_K super-blocks [nb, 144] uint8 from their fields: d, dmin [nb] half; scales, mins
    [nb, 8] in 0..63; q [nb, 256] in 0..15.  The 6-bit fields are packed the way ggml's
    quantiser packs them (sub-blocks 0..3 in the low six bits of bytes 0..7, sub-blocks 4..7
    split between the nibbles of bytes 8..11 and the top two bits of bytes 0..7); of every
    64 weights the first 32 take the low nibbles of 32 bytes, the next 32 the high ones."""
    nb = d.shape[0]
    out = np.zeros((nb, Q4K_BLOCK_BYTES), np.uint8)
    out[:, 0:2] = np.ascontiguousarray(d, np.float16).view(np.uint8).reshape(nb, 2)
    out[:, 2:4] = np.ascontiguousarray(dmin, np.float16).view(np.uint8).reshape(nb, 2)
    ls, lm = scales.astype(np.uint8), mins.astype(np.uint8)
    packed = out[:, 4:16]
    for j in range(8):
        if j < 4:
            packed[:, j] |= ls[:, j]
            packed[:, j + 4] |= lm[:, j]
        else:
            packed[:, j + 4] = (ls[:, j] & 0xF) | ((lm[:, j] & 0xF) << 4)
            packed[:, j - 4] |= (ls[:, j] >> 4) << 6
            packed[:, j] |= (lm[:, j] >> 4) << 6
    q = q.astype(np.uint8).reshape(nb, 4, 2, 32)
    out[:, 16:] = (q[:, :, 0, :] | (q[:, :, 1, :] << 4)).reshape(nb, 128)
    return out


@dataclass
class QkvProjectionCase:
    """x [batch, K] float32 and the three Q4_K weight matrices of a fused Q/K/V projection
    ([N, K/256] super-blocks, row major: weight row n holds the K inputs of output n)."""
    x: np.ndarray
    wq: np.ndarray   # [Nq, K/256, 144] uint8
    wk: np.ndarray   # [Nkv, K/256, 144]
    wv: np.ndarray
    K: int
    Nq: int
    Nkv: int

    @property
    def batch(self) -> int:
        return int(self.x.shape[0])

    def algorithmic_bytes(self) -> int:
        out = self.batch * (self.Nq + 2 * self.Nkv) * 4
        return self.wq.nbytes + self.wk.nbytes + self.wv.nbytes + self.x.nbytes + out

    def flops(self) -> int:
        return 2 * self.batch * self.K * (self.Nq + 2 * self.Nkv)


def random_q4k(rng: np.random.Generator, rows: int, K: int) -> np.ndarray:
    """Random Q4_K rows whose dequantised weights look like a trained matrix's (|w| of a
    few hundredths): every field of the format is drawn, so all code paths of the
    dequantisation are exercised."""
    nb = rows * (K // QK_K)
    d = (rng.uniform(0.5, 1.5, nb) * 4e-4).astype(np.float16)
    dmin = (rng.uniform(0.5, 1.5, nb) * 4e-4).astype(np.float16)
    scales = rng.integers(0, 64, (nb, 8))
    mins = rng.integers(0, 64, (nb, 8))
    q = rng.integers(0, 16, (nb, QK_K))
    return pack_q4k(d, dmin, scales, mins, q).reshape(rows, K // QK_K, Q4K_BLOCK_BYTES)


def make_qkv_projection(seed=SEED_BASE + 6, K=4096, num_heads=32, num_kv_heads=8, head_dim=128,
                        batch=1) -> QkvProjectionCase:
    rng = np.random.default_rng(seed)
    nq, nkv = num_heads * head_dim, num_kv_heads * head_dim
    x = _normal(rng, (batch, K))
    return QkvProjectionCase(x, random_q4k(rng, nq, K), random_q4k(rng, nkv, K), random_q4k(rng, nkv, K),
                             K, nq, nkv)
