"""GPU parity of the two prefill kernels behind granite_hip_attention: the direct-to-LDS
kernel (attention_tiles_dma_kernel, the default where it applies: head size 128, half or
float queries, contiguous cache or blocks of a power of two >= 8 tokens) and the register-staged
kernel it falls back to (attention_tiles_kernel, forced here with
GRANITE_HIP_PREFILL_KERNEL=tiles).  Both against the oracle's restatement of
src/llm/transformer.mm:1779-1840 and :2044-2126, and against each other.
Tolerances: outputs |d| <= 2e-3 or <= 1e-2 |ref|; lse 1e-4."""
import os

import numpy as np
import pytest

from granite_amd import F16, F32, MASK_CAUSAL, MASK_NONE, MASK_TREE
from granite_amd import workloads as W
from gpu_util import assert_close, assert_lse, dev, say

pytestmark = pytest.mark.gpu


def _run(gpu, case_q, dk, dv, hq, hkv, seq_q, total, start, scale, out_dtype, table, bs, max_seq, mask, kernel):
    odt = np.float32 if out_dtype == F32 else np.float16
    out, lse = dev(np.zeros((seq_q, hq, 128), odt)), dev(np.zeros((hq, seq_q), np.float32))
    old = os.environ.pop("GRANITE_HIP_PREFILL_KERNEL", None)
    if kernel == "tiles":
        os.environ["GRANITE_HIP_PREFILL_KERNEL"] = "tiles"
    try:
        gpu.attention(q=dev(case_q), q_dtype=F16, q_tok_stride=hq * 128, q_head_stride=128, out=out,
                      out_dtype=out_dtype, out_tok_stride=hq * 128, out_head_stride=128, lse=lse, seq_q=seq_q,
                      num_heads=hq, num_kv_heads=hkv, head_dim=128, scale=scale, k_cache=dk, v_cache=dv,
                      cache_len=total, max_seq=max_seq, block_table=table, block_size=bs, mask_mode=mask,
                      start_pos=start)
        gpu.sync()
    finally:
        os.environ.pop("GRANITE_HIP_PREFILL_KERNEL", None)
        if old is not None:
            os.environ["GRANITE_HIP_PREFILL_KERNEL"] = old
    return out.read(odt, (seq_q, hq, 128)).astype(np.float32), lse.read(np.float32, (hq, seq_q))


@pytest.mark.parametrize("prefix,chunk,bs,hq,hkv,out_dtype", [
    (0, 1, 8, 4, 4, F16), (0, 63, 8, 8, 2, F16), (0, 64, 16, 8, 2, F32), (7, 65, 16, 4, 1, F16),
    (64, 192, 32, 8, 8, F16), (129, 257, 64, 8, 2, F32), (1000, 128, 128, 16, 2, F16),
    (4100, 300, 16, 8, 1, F16),    # key splits (few workgroups, many tiles)
    (16000, 64, 32, 4, 1, F16),    # more than 64 tiles per wave: the block-table entries are refilled
    (20000, 40, 8, 2, 2, F32),
    # a long prompt from position 0: the waves of a workgroup's early run go idle after a few tiles
    # and stage the shares of the late run's waves for the rest of its walk, across two refills
    # of the block-table entries
    (0, 9000, 16, 2, 1, F16),
    (300, 4500, 8, 2, 2, F32),
])
def test_paged_chunk_both_kernels(gpu, oracle, prefix, chunk, bs, hq, hkv, out_dtype):
    say(f"prefill kernels paged prefix={prefix} chunk={chunk} bs={bs} hq={hq} hkv={hkv} out={out_dtype}")
    case = W.make_chunked_prefill(seed=prefix + 7 * chunk + bs, prefix_len=prefix, chunk=chunk, num_heads=hq,
                                  num_kv_heads=hkv, block_size=bs, pool_slack=1.3)
    total = prefix + chunk
    dk, dv, dt = dev(case.k_pool), dev(case.v_pool), dev(case.block_table)
    gpu.paged_kv_cache_append_ex(dev(case.k_new), dev(case.v_new), F16, hkv * 128, 128, dk, dv, dt, hkv, 128,
                                 prefix, chunk, bs)
    gpu.sync()
    pool_k, pool_v = dk.read(np.uint16, case.k_pool.shape), dv.read(np.uint16, case.v_pool.shape)
    want, want_lse = oracle.attention_paged(case.q[None].astype(np.float32), pool_k, pool_v, case.block_table, bs,
                                            total, prefix, case.scale)
    results = {}
    for kernel in ("dma", "tiles"):
        got, got_lse = _run(gpu, case.q, dk, dv, hq, hkv, chunk, total, prefix, case.scale, out_dtype, dt, bs, 0,
                            MASK_CAUSAL, kernel)
        assert_close(got, want[0], f"{kernel} out")
        assert_lse(got_lse, want_lse[0], f"{kernel} lse")
        results[kernel] = (got, got_lse)
    # the two kernels do the same arithmetic in the same order
    assert np.abs(results["dma"][0] - results["tiles"][0]).max() <= 1e-3
    assert np.abs(results["dma"][1] - results["tiles"][1]).max() <= 1e-5


@pytest.mark.parametrize("seq,hq,hkv,max_seq,mask", [(1, 4, 4, 8, MASK_CAUSAL), (64, 4, 1, 64, MASK_CAUSAL),
                                                     (100, 8, 2, 100, MASK_CAUSAL), (257, 4, 2, 300, MASK_CAUSAL),
                                                     (513, 8, 8, 520, MASK_CAUSAL), (200, 4, 2, 256, MASK_NONE),
                                                     # no mask and at most 128 rows: the empty run's waves
                                                     # stage for the others from the first tile on
                                                     (100, 4, 2, 128, MASK_NONE), (128, 8, 8, 300, MASK_NONE),
                                                     # at most 64 rows: two waves per row block, a sub-tile of every
                                                     # tile each (causal from the start, and unmasked)
                                                     (33, 4, 2, 40, MASK_CAUSAL), (64, 8, 2, 100, MASK_NONE),
                                                     (20, 4, 4, 64, MASK_NONE), (47, 2, 1, 47, MASK_NONE)])
def test_contiguous_both_kernels(gpu, oracle, seq, hq, hkv, max_seq, mask):
    say(f"prefill kernels contiguous seq={seq} hq={hq} hkv={hkv} max_seq={max_seq} mask={mask}")
    case = W.make_prefill(seed=5 * seq + hq, seq=seq, num_heads=hq, num_kv_heads=hkv, max_seq=max_seq)
    dk, dv = dev(case.k_cache), dev(case.v_cache)
    if mask == MASK_CAUSAL:
        want, want_lse = oracle.attention_cached(case.q[None].astype(np.float32), case.k_cache, case.v_cache, seq,
                                                 0, case.scale)
    else:  # every query sees every key: the causal routine with all queries at the last position
        rows = [oracle.attention_cached(case.q[None, i:i + 1].astype(np.float32), case.k_cache, case.v_cache, seq,
                                        seq - 1, case.scale) for i in range(seq)]
        want = np.concatenate([r[0] for r in rows], axis=1)
        want_lse = np.concatenate([r[1] for r in rows], axis=2)
    for kernel in ("dma", "tiles"):
        got, got_lse = _run(gpu, case.q, dk, dv, hq, hkv, seq, seq, 0, case.scale, F16, None, 0, max_seq, mask,
                            kernel)
        assert_close(got, want[0], f"{kernel} out")
        assert_lse(got_lse, want_lse[0], f"{kernel} lse")


@pytest.mark.parametrize("kernel", ["dma", "tiles"])
def test_softmax_reference_moves_mid_stream(gpu, oracle, kernel):
    """Keys whose scores grow along the sequence, by far more than the 2^14 headroom of the
    lazy softmax reference: the reference has to move (and O and l be rescaled) many times per
    row, also inside the steady-state loop."""
    seq, hq, hkv = 700, 4, 2
    case = W.make_prefill(seed=99, seq=seq, num_heads=hq, num_kv_heads=hkv, max_seq=seq)
    ramp = (1.0 + np.arange(seq, dtype=np.float32) / 78.0)[None, :, None]  # scores grow from about 5 to 45 nats
    k = (np.abs(case.k_cache.astype(np.float32)) * ramp).astype(np.float16)
    q = np.abs(case.q.astype(np.float32)).astype(np.float16)               # all scores positive and growing
    want, want_lse = oracle.attention_cached(q[None].astype(np.float32), k, case.v_cache, seq, 0, case.scale)
    got, got_lse = _run(gpu, q, dev(k), dev(case.v_cache), hq, hkv, seq, seq, 0, case.scale, F32, None, 0, seq,
                        MASK_CAUSAL, kernel)
    assert np.isfinite(got).all()
    assert_close(got, want[0], "out")
    assert_lse(got_lse, want_lse[0], "lse")


@pytest.mark.parametrize("prefix,chunk,bs,hq,hkv,q_dtype,out_dtype,splits", [
    (0, 1, 16, 4, 4, F16, F16, 0), (0, 33, 16, 8, 2, F32, F32, 0), (5, 64, 1, 4, 1, F16, F32, 0),
    (127, 32, 12, 8, 2, F32, F16, 0), (128, 31, 8, 8, 8, F16, F16, 0), (129, 64, 4, 4, 2, F32, F32, 0),
    (1000, 17, 16, 12, 3, F16, F32, 0),
    (4096, 64, 16, 8, 2, F32, F32, 0),     # keys split over workgroups (few heads, many tiles)
    (4100, 40, 32, 8, 1, F16, F16, 5),     # a split count that does not divide the tiles
    (300, 64, 16, 4, 1, F16, F16, 7),      # more splits than tiles: empty shares write neutral partials
])
def test_short_chunk_default_kernel_and_tiles_kernel(gpu, oracle, prefix, chunk, bs, hq, hkv, q_dtype, out_dtype, splits):
    """A chunk of at most 64 tokens (a quarter of a workgroup's rows) over a paged prefix, block
    sizes on both sides of what the direct-to-LDS kernel takes, both query and output types,
    split counts that do not divide the tiles and that exceed them: the kernel chosen by
    default and the register-staged kernel against the oracle and against each other."""
    say(f"short chunk prefix={prefix} chunk={chunk} bs={bs} hq={hq} hkv={hkv} q={q_dtype} out={out_dtype} "
        f"splits={splits}")
    case = W.make_chunked_prefill(seed=3 * prefix + chunk + bs, prefix_len=prefix, chunk=chunk, num_heads=hq,
                                  num_kv_heads=hkv, block_size=bs, pool_slack=1.3)
    total = prefix + chunk
    dk, dv, dt = dev(case.k_pool), dev(case.v_pool), dev(case.block_table)
    gpu.paged_kv_cache_append_ex(dev(case.k_new), dev(case.v_new), F16, hkv * 128, 128, dk, dv, dt, hkv, 128,
                                 prefix, chunk, bs)
    gpu.sync()
    pool_k, pool_v = dk.read(np.uint16, case.k_pool.shape), dv.read(np.uint16, case.v_pool.shape)
    want, want_lse = oracle.attention_paged(case.q[None].astype(np.float32), pool_k, pool_v, case.block_table, bs,
                                            total, prefix, case.scale)
    q_host = case.q if q_dtype == F16 else case.q.astype(np.float32)
    odt = np.float32 if out_dtype == F32 else np.float16
    old = os.environ.pop("GRANITE_HIP_ATTN_SPLITS", None)
    if splits:
        os.environ["GRANITE_HIP_ATTN_SPLITS"] = str(splits)
    results = {}
    try:
        for kernel in ("default", "tiles"):
            out, lse = dev(np.zeros((chunk, hq, 128), odt)), dev(np.zeros((hq, chunk), np.float32))
            if kernel == "tiles":
                os.environ["GRANITE_HIP_PREFILL_KERNEL"] = "tiles"
            try:
                gpu.attention(q=dev(q_host), q_dtype=q_dtype, q_tok_stride=hq * 128, q_head_stride=128, out=out,
                              out_dtype=out_dtype, out_tok_stride=hq * 128, out_head_stride=128, lse=lse,
                              seq_q=chunk, num_heads=hq, num_kv_heads=hkv, head_dim=128, scale=case.scale,
                              k_cache=dk, v_cache=dv, cache_len=total, block_table=dt, block_size=bs,
                              mask_mode=MASK_CAUSAL, start_pos=prefix)
                gpu.sync()
            finally:
                os.environ.pop("GRANITE_HIP_PREFILL_KERNEL", None)
            got, got_lse = out.read(odt, (chunk, hq, 128)).astype(np.float32), lse.read(np.float32, (hq, chunk))
            assert_close(got, want[0], f"{kernel} out")
            assert_lse(got_lse, want_lse[0], f"{kernel} lse")
            results[kernel] = (got, got_lse)
    finally:
        os.environ.pop("GRANITE_HIP_ATTN_SPLITS", None)
        if old is not None:
            os.environ["GRANITE_HIP_ATTN_SPLITS"] = old
    assert np.abs(results["default"][0] - results["tiles"][0]).max() <= 2e-3
    assert np.abs(results["default"][1] - results["tiles"][1]).max() <= 1e-4


@pytest.mark.parametrize("prefix,n,hq,hkv,bs,paged", [(0, 1, 4, 4, 16, True), (0, 40, 8, 2, 16, True),
                                                     (100, 33, 8, 2, 12, True), (2000, 64, 32, 8, 16, True),
                                                     (700, 64, 8, 2, 16, False), (4096, 20, 4, 1, 1, True),
                                                     # the direct-to-LDS kernel's tree form: a prefix that ends inside a
                                                     # tile, on a tile boundary and one key behind it; trees of more
                                                     # than one tile and of the largest size it builds masks for
                                                     (63, 64, 8, 2, 16, True), (64, 64, 8, 2, 16, True), (65, 70, 8, 2, 8, True),
                                                     (3000, 200, 8, 2, 32, True), (1000, 256, 4, 1, 8, True),
                                                     (130, 129, 8, 2, 16, False), (5, 3, 4, 4, 64, True),
                                                     # small trees behind a long prefix: the heads of a KV group side by
                                                     # side in one workgroup (two heads of 64 nodes, four of 20, two of
                                                     # three heads of 40: no packing, 128 rows exactly)
                                                     (8200, 64, 8, 2, 16, True), (9000, 20, 8, 2, 32, False),
                                                     (8192, 40, 6, 2, 16, True), (8300, 32, 16, 4, 8, True)])
def test_tree_default_kernel_and_tiles_kernel(gpu, oracle, prefix, n, hq, hkv, bs, paged):
    """Tree attention (fp32 queries, a prefix in a paged or contiguous cache, the nodes as the
    extra segment), launched as by default and with the register-staged kernel forced."""
    say(f"tree kernels prefix={prefix} nodes={n} hq={hq} hkv={hkv} bs={bs} paged={paged}")
    case = W.make_tree(seed=prefix + n, prefix_len=prefix, num_nodes=n, num_heads=hq, num_kv_heads=hkv,
                       block_size=bs)
    q = np.transpose(case.q, (1, 0, 2))[None]
    kt = np.transpose(case.k_tree, (1, 0, 2))[None].astype(np.float32)
    vt = np.transpose(case.v_tree, (1, 0, 2))[None].astype(np.float32)
    want, want_lse = oracle.attention_tree(q, case.k_pool, case.v_pool, kt, vt, case.parents, prefix, case.scale,
                                           table=case.block_table, block_size=bs)
    if paged:
        cache = dict(k_cache=dev(case.k_pool), v_cache=dev(case.v_pool), block_size=bs,
                     block_table=dev(case.block_table) if prefix else None, max_seq=prefix)
    else:  # the same prefix gathered into [Hkv, prefix, D]
        rows = (case.block_table[np.arange(prefix) // bs] * bs + np.arange(prefix) % bs) if prefix else np.zeros(0, int)
        kc = np.ascontiguousarray(np.transpose(case.k_pool[rows], (1, 0, 2)))
        vc = np.ascontiguousarray(np.transpose(case.v_pool[rows], (1, 0, 2)))
        cache = dict(k_cache=dev(kc), v_cache=dev(vc), max_seq=prefix)
    results = {}
    for kernel in ("default", "tiles"):
        out, lse = dev(np.zeros((hq, n, 128), np.float32)), dev(np.zeros((hq, n), np.float32))
        if kernel == "tiles":
            os.environ["GRANITE_HIP_PREFILL_KERNEL"] = "tiles"
        try:
            gpu.attention(q=dev(case.q), q_dtype=F32, q_tok_stride=128, q_head_stride=n * 128, out=out, out_dtype=F32,
                          out_tok_stride=128, out_head_stride=n * 128, lse=lse, seq_q=n, num_heads=hq,
                          num_kv_heads=hkv, head_dim=128, scale=case.scale, cache_len=prefix,
                          k_extra=dev(case.k_tree), v_extra=dev(case.v_tree), extra_len=n, parents=dev(case.parents),
                          mask_mode=MASK_TREE, **cache)
            gpu.sync()
        finally:
            os.environ.pop("GRANITE_HIP_PREFILL_KERNEL", None)
        got, got_lse = out.read(np.float32, (hq, n, 128)), lse.read(np.float32, (hq, n))
        assert_close(got, np.transpose(want[0], (1, 0, 2)), f"{kernel} out")
        assert_lse(got_lse, want_lse[0], f"{kernel} lse")
        results[kernel] = (got, got_lse)
    assert np.abs(results["default"][0] - results["tiles"][0]).max() <= 2e-3


@pytest.mark.parametrize("prefix,chunk,bs,hq,hkv,out_dtype", [
    (0, 300, 16, 8, 2, F32),       # a prompt from position 0: the early run's waves hand over
    (2000, 257, 32, 8, 8, F32),    # behind a prefix: the plain loop
    (5000, 100, 8, 4, 1, F16),     # key splits; float queries with half output
    (0, 1, 16, 4, 4, F32),
])
def test_float_queries_both_kernels(gpu, oracle, prefix, chunk, bs, hq, hkv, out_dtype):
    """Float queries (what the reference's callers pass): both kernels take them as an fp16 head
    and an fp16 remainder, so they must agree with the oracle's float arithmetic to the same
    tolerance as half queries do -- also with queries whose remainders matter (values with 20
    significant bits)."""
    say(f"float queries prefix={prefix} chunk={chunk} bs={bs} hq={hq} hkv={hkv} out={out_dtype}")
    case = W.make_chunked_prefill(seed=11 * prefix + chunk, prefix_len=prefix, chunk=chunk, num_heads=hq,
                                  num_kv_heads=hkv, block_size=bs, pool_slack=1.3)
    rng = np.random.default_rng(prefix + chunk)
    q = (case.q.astype(np.float32) * (1.0 + rng.integers(-512, 512, case.q.shape).astype(np.float32) * 2.0 ** -20))
    total = prefix + chunk
    dk, dv, dt = dev(case.k_pool), dev(case.v_pool), dev(case.block_table)
    gpu.paged_kv_cache_append_ex(dev(case.k_new), dev(case.v_new), F16, hkv * 128, 128, dk, dv, dt, hkv, 128,
                                 prefix, chunk, bs)
    gpu.sync()
    pool_k, pool_v = dk.read(np.uint16, case.k_pool.shape), dv.read(np.uint16, case.v_pool.shape)
    want, want_lse = oracle.attention_paged(q[None], pool_k, pool_v, case.block_table, bs, total, prefix, case.scale)
    odt = np.float32 if out_dtype == F32 else np.float16
    results = {}
    for kernel in ("dma", "tiles"):
        out, lse = dev(np.zeros((chunk, hq, 128), odt)), dev(np.zeros((hq, chunk), np.float32))
        if kernel == "tiles":
            os.environ["GRANITE_HIP_PREFILL_KERNEL"] = "tiles"
        try:
            gpu.attention(q=dev(q), q_dtype=F32, q_tok_stride=hq * 128, q_head_stride=128, out=out,
                          out_dtype=out_dtype, out_tok_stride=hq * 128, out_head_stride=128, lse=lse, seq_q=chunk,
                          num_heads=hq, num_kv_heads=hkv, head_dim=128, scale=case.scale, k_cache=dk, v_cache=dv,
                          cache_len=total, block_table=dt, block_size=bs, mask_mode=MASK_CAUSAL, start_pos=prefix)
            gpu.sync()
        finally:
            os.environ.pop("GRANITE_HIP_PREFILL_KERNEL", None)
        got, got_lse = out.read(odt, (chunk, hq, 128)).astype(np.float32), lse.read(np.float32, (hq, chunk))
        assert_close(got, want[0], f"{kernel} out")
        assert_lse(got_lse, want_lse[0], f"{kernel} lse")
        results[kernel] = (got, got_lse)
    assert np.abs(results["dma"][0] - results["tiles"][0]).max() <= 1e-3
    assert np.abs(results["dma"][1] - results["tiles"][1]).max() <= 1e-5


@pytest.mark.parametrize("prefix,n,hq,hkv,bs,paged", [(500, 64, 8, 2, 16, True), (200, 150, 4, 1, 32, False)])
def test_tree_half_queries_and_output(gpu, oracle, prefix, n, hq, hkv, bs, paged):
    """Tree attention with half queries and half output (the default kernel's tree form is
    instantiated for both query and both output types)."""
    say(f"tree half prefix={prefix} nodes={n} hq={hq} hkv={hkv} bs={bs} paged={paged}")
    case = W.make_tree(seed=3 * prefix + n, prefix_len=prefix, num_nodes=n, num_heads=hq, num_kv_heads=hkv,
                       block_size=bs)
    qh = case.q.astype(np.float16)                                     # [hq, n, 128]
    q = np.transpose(qh.astype(np.float32), (1, 0, 2))[None]
    kt = np.transpose(case.k_tree, (1, 0, 2))[None].astype(np.float32)
    vt = np.transpose(case.v_tree, (1, 0, 2))[None].astype(np.float32)
    want, want_lse = oracle.attention_tree(q, case.k_pool, case.v_pool, kt, vt, case.parents, prefix, case.scale,
                                           table=case.block_table, block_size=bs)
    if paged:
        cache = dict(k_cache=dev(case.k_pool), v_cache=dev(case.v_pool), block_size=bs,
                     block_table=dev(case.block_table), max_seq=prefix)
    else:
        rows = case.block_table[np.arange(prefix) // bs] * bs + np.arange(prefix) % bs
        kc = np.ascontiguousarray(np.transpose(case.k_pool[rows], (1, 0, 2)))
        vc = np.ascontiguousarray(np.transpose(case.v_pool[rows], (1, 0, 2)))
        cache = dict(k_cache=dev(kc), v_cache=dev(vc), max_seq=prefix)
    out, lse = dev(np.zeros((hq, n, 128), np.float16)), dev(np.zeros((hq, n), np.float32))
    gpu.attention(q=dev(qh), q_dtype=F16, q_tok_stride=128, q_head_stride=n * 128, out=out, out_dtype=F16,
                  out_tok_stride=128, out_head_stride=n * 128, lse=lse, seq_q=n, num_heads=hq, num_kv_heads=hkv,
                  head_dim=128, scale=case.scale, cache_len=prefix, k_extra=dev(case.k_tree), v_extra=dev(case.v_tree),
                  extra_len=n, parents=dev(case.parents), mask_mode=MASK_TREE, **cache)
    gpu.sync()
    assert_close(out.read(np.float16, (hq, n, 128)).astype(np.float32), np.transpose(want[0], (1, 0, 2)), "out")
    assert_lse(lse.read(np.float32, (hq, n)), want_lse[0], "lse")
