"""Independent float64 attention used to pin the CPU oracle.  Written from the
mathematical definition (softmax(scale * Q K^T + mask) V), not from the
reference's loops, so a dropped term or wrong index in the oracle shows up."""
from __future__ import annotations

import numpy as np


def half_bits_to_f64(bits: np.ndarray) -> np.ndarray:
    return np.ascontiguousarray(bits).view(np.float16).astype(np.float64)


def attention64(q, k, v, visible, scale):
    """q [Sq,Hq,D], k/v [T,Hkv,D] (any float dtype), visible bool [Sq,T].
    Returns out [Sq,Hq,D] and natural-log lse [Hq,Sq], all float64."""
    q = np.asarray(q, np.float64)
    k = np.asarray(k, np.float64)
    v = np.asarray(v, np.float64)
    Sq, Hq, D = q.shape
    T, Hkv, _ = k.shape
    G = Hq // Hkv
    out = np.zeros((Sq, Hq, D))
    lse = np.zeros((Hq, Sq))
    for h in range(Hq):
        kh, vh = k[:, h // G, :], v[:, h // G, :]
        s = (q[:, h, :] @ kh.T) * scale
        s = np.where(visible, s, -np.inf)
        m = s.max(axis=1, keepdims=True)
        e = np.exp(s - m)
        z = e.sum(axis=1, keepdims=True)
        out[:, h, :] = (e / z) @ vh
        lse[h] = (m + np.log(z))[:, 0]
    return out, lse


def causal_visible(seq_q: int, total: int, start_pos: int) -> np.ndarray:
    qpos = np.arange(seq_q)[:, None] + start_pos
    return np.arange(total)[None, :] <= qpos


def tree_visible(parents, prefix_len: int) -> np.ndarray:
    """Closed form of the ancestor mask: node i sees node j iff j is on the
    path from i to its root."""
    n = len(parents)
    vis = np.zeros((n, prefix_len + n), dtype=bool)
    vis[:, :prefix_len] = True
    for i in range(n):
        j = i
        steps = 0
        while j >= 0 and steps <= n:
            vis[i, prefix_len + j] = True
            j = int(parents[j])
            steps += 1
    return vis


def gather_paged(pool, table, block_size, length):
    """pool [rows,Hkv,D] -> [length,Hkv,D] following the block table."""
    pos = np.arange(length)
    rows = np.asarray(table)[pos // block_size].astype(np.int64) * block_size + pos % block_size
    return pool[rows]


def compare(got, want, abs_tol=2e-3, rel_tol=1e-2):
    """Element passes if |d| <= abs_tol or |d| <= rel_tol*|want| (the reference
    tool's abs-OR-rel rule, tools/test_paged_flash_attention.mm:270-277).
    Returns (ok, max_abs, max_rel_over_failing_abs)."""
    got = np.asarray(got, np.float64)
    want = np.asarray(want, np.float64)
    d = np.abs(got - want)
    ok = (d <= abs_tol) | (d <= rel_tol * np.abs(want))
    rel = d / (np.abs(want) + 1e-6)
    return bool(ok.all() and np.isfinite(got).all()), float(d.max(initial=0.0)), float(rel.max(initial=0.0))
