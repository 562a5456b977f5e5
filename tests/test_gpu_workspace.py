"""GPU checks of the scratch-memory interface: a reservation made once keeps every later
launch from allocating, caller-owned scratch gives bit-identical results and is refused
when too small, and a change of stream is ordered after the work queued before it."""
import ctypes as C

import numpy as np
import pytest

from granite_amd import F16, F32, MASK_CAUSAL, GraniteHipError, _capi
from granite_amd import workloads as W
from gpu_util import assert_close, assert_lse, dev, say

pytestmark = pytest.mark.gpu


def _decode_kwargs(case, out, lse):
    return dict(q=dev(case.q), q_dtype=F16, k_cache=dev(case.k_pool), v_cache=dev(case.v_pool),
                block_tables=dev(case.block_tables), seq_lens=dev(case.seq_lens), out=out, lse=lse,
                batch_size=case.batch, num_heads=case.num_heads, num_kv_heads=case.num_kv_heads, head_dim=128,
                scale=case.scale, block_size=case.block_size, max_blocks_per_seq=case.max_blocks)


def _prefill_kwargs(case, out, lse, hq, hkv, chunk, prefix, bs):
    return dict(q=dev(case.q), q_dtype=F16, q_tok_stride=hq * 128, q_head_stride=128, out=out, out_dtype=F32,
                out_tok_stride=hq * 128, out_head_stride=128, lse=lse, seq_q=chunk, num_heads=hq,
                num_kv_heads=hkv, head_dim=128, scale=case.scale, k_cache=dev(case.k_pool),
                v_cache=dev(case.v_pool), cache_len=prefix, block_table=dev(case.block_table), block_size=bs,
                mask_mode=MASK_CAUSAL, start_pos=prefix - chunk)


def test_reserved_workspace_is_never_regrown(gpu, oracle):
    """Ask what a decode batch and a split-K prefill need, reserve the larger once: no launch
    afterwards changes the library's scratch size, and results still match the oracle."""
    lens = np.array([1500, 40, 2048, 777, 1, 1024, 333, 2000], np.int32)
    dcase = W.make_paged_decode(seed=21, ctx_max=2048, seq_lens=lens)
    hq, hkv, bs, prefix, chunk = 8, 2, 16, 3000, 96
    pcase = W.make_chunked_prefill(seed=22, prefix_len=prefix - chunk, chunk=chunk, num_heads=hq, num_kv_heads=hkv,
                                   block_size=bs, pool_slack=1.2)
    # the chunk's rows are placed by hand: this test is about scratch, not about the append
    pool_k, pool_v = pcase.k_pool.copy(), pcase.v_pool.copy()
    for t in range(chunk):
        pos = prefix - chunk + t
        row = pcase.block_table[pos // bs] * bs + pos % bs
        pool_k[row], pool_v[row] = pcase.k_new[t], pcase.v_new[t]
    pcase.k_pool, pcase.v_pool = pool_k, pool_v

    dout, dlse = dev(np.zeros((8, 32, 128), np.float32)), dev(np.zeros((8, 32), np.float32))
    pout, plse = dev(np.zeros((chunk, hq, 128), np.float32)), dev(np.zeros((hq, chunk), np.float32))
    dk = _decode_kwargs(dcase, dout, dlse)
    pk = _prefill_kwargs(pcase, pout, plse, hq, hkv, chunk, prefix, bs)
    need_d = gpu.decode_attention(**dk, query_workspace=True)
    need_p = gpu.attention(**pk, query_workspace=True)
    say(f"scratch needed: decode {need_d} B, split-K prefill {need_p} B")
    assert need_d > 0 and need_p > 0
    gpu.reserve_workspace(max(need_d, need_p))
    held = gpu.workspace_bytes()
    assert held >= max(need_d, need_p)
    for _ in range(2):
        gpu.decode_attention(**dk)
        assert gpu.workspace_bytes() == held
        gpu.attention(**pk)
        assert gpu.workspace_bytes() == held
    gpu.sync()
    want, want_lse = oracle.batched_paged_decode(dcase.q.astype(np.float32), dcase.k_pool, dcase.v_pool,
                                                 dcase.block_tables, dcase.seq_lens, dcase.block_size, dcase.scale)
    assert_close(dout.read(np.float32, (8, 32, 128)), want, "decode")
    assert_lse(dlse.read(np.float32, (8, 32)), want_lse, "decode lse")
    want, want_lse = oracle.attention_paged(pcase.q[None].astype(np.float32), pool_k, pool_v, pcase.block_table, bs,
                                            prefix, prefix - chunk, pcase.scale)
    assert_close(pout.read(np.float32, (chunk, hq, 128)), want[0], "prefill")
    assert_lse(plse.read(np.float32, (hq, chunk)), want_lse[0], "prefill lse")


def test_caller_owned_workspace(gpu):
    """The _ws forms use the buffer given and nothing else; results are bit-identical to the
    plain forms; a buffer that is too small is refused before anything is launched."""
    lens = np.array([900, 1200, 64, 2047], np.int32)
    case = W.make_paged_decode(seed=23, ctx_max=2048, seq_lens=lens)
    out_a, lse_a = dev(np.zeros((4, 32, 128), np.float32)), dev(np.zeros((4, 32), np.float32))
    out_b, lse_b = dev(np.zeros((4, 32, 128), np.float32)), dev(np.zeros((4, 32), np.float32))
    ka, kb = _decode_kwargs(case, out_a, lse_a), _decode_kwargs(case, out_b, lse_b)
    need = gpu.decode_attention(**ka, query_workspace=True)
    gpu.decode_attention(**ka)
    held = gpu.workspace_bytes()
    ws = gpu.create_buffer(need)
    ws.fill(0xFF)
    gpu.decode_attention(**kb, workspace=ws)
    gpu.sync()
    assert gpu.workspace_bytes() == held
    assert np.array_equal(out_a.read(np.uint32, (4, 32, 128)), out_b.read(np.uint32, (4, 32, 128)))
    assert np.array_equal(lse_a.read(np.uint32, (4, 32)), lse_b.read(np.uint32, (4, 32)))
    sentinel = out_b.read(np.uint32, (4, 32, 128)).copy()
    with pytest.raises(GraniteHipError) as e:
        gpu.decode_attention(**kb, workspace=ws, workspace_bytes=need - 256)
    assert e.value.code == _capi.ESCRATCH
    gpu.sync()
    assert np.array_equal(out_b.read(np.uint32, (4, 32, 128)), sentinel)


def test_set_stream_orders_the_hand_over(gpu, oracle):
    """Launches before and after granite_hip_set_stream share the scratch buffer; the new
    stream must wait for the old one.  Both results are checked against the oracle."""
    hip = C.CDLL("libamdhip64.so")
    stream = C.c_void_p()
    assert hip.hipStreamCreate(C.byref(stream)) == 0
    lib = _capi.load()
    try:
        outs = []
        for seed in (31, 32):
            lens = np.array([2048, 1999, 1500, 1800], np.int32)
            case = W.make_paged_decode(seed=seed, ctx_max=2048, seq_lens=lens)
            out, lse = dev(np.zeros((4, 32, 128), np.float32)), dev(np.zeros((4, 32), np.float32))
            outs.append((case, out, lse, _decode_kwargs(case, out, lse)))
        gpu.decode_attention(**outs[0][3])                # on the library's own stream
        _capi.check(lib.granite_hip_set_stream(stream), "set_stream")
        gpu.decode_attention(**outs[1][3])                # on the caller's stream, same scratch
        gpu.sync()
        _capi.check(lib.granite_hip_set_stream(None), "set_stream")
        gpu.sync()
        for case, out, lse, _ in outs:
            want, want_lse = oracle.batched_paged_decode(case.q.astype(np.float32), case.k_pool, case.v_pool,
                                                         case.block_tables, case.seq_lens, case.block_size,
                                                         case.scale)
            assert_close(out.read(np.float32, (4, 32, 128)), want, "decode")
            assert_lse(lse.read(np.float32, (4, 32)), want_lse, "lse")
    finally:
        lib.granite_hip_set_stream(None)
        hip.hipStreamDestroy(stream)
