"""GPU parity of the two prefill kernels behind granite_hip_attention: the direct-to-LDS
kernel (attention_tiles_dma_kernel, the default where it applies: head size 128, half
queries, contiguous cache or blocks of a power of two >= 8 tokens) and the register-staged
kernel it falls back to (attention_tiles_kernel, forced here with
GRANITE_HIP_PREFILL_KERNEL=tiles).  Both against the oracle's restatement of
src/llm/transformer.mm:1779-1840, and against each other.
Tolerances: outputs |d| <= 2e-3 or <= 1e-2 |ref|; lse 1e-4."""
import os

import numpy as np
import pytest

from granite_amd import F16, F32, MASK_CAUSAL, MASK_NONE
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
                                                     (513, 8, 8, 520, MASK_CAUSAL), (200, 4, 2, 256, MASK_NONE)])
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
