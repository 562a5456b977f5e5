"""Seeded random sweeps through the C ABI, both head sizes: batched paged decode (growable and
static scratch), chunked prefill over a paged cache and tree attention, each against the
oracle.  Tolerances: outputs |d| <= 2e-3 or <= 1e-2 |ref|; log-sum-exp 1e-4."""
import numpy as np
import pytest

from granite_amd import F16, F32, MASK_CAUSAL, MASK_TREE, GraniteHipError, _capi
from granite_amd import workloads as W
from gpu_util import assert_close, assert_lse, dev, say

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("trial", range(24))
def test_random_batched_paged_decode(gpu, oracle, trial):
    rng = np.random.default_rng(7000 + trial)
    D = int(rng.choice([64, 128]))
    hkv = int(rng.choice([8, 16, 4, 2, 1, 3, 5]))
    hq = hkv * int(rng.choice([1, 2, 4, 8, 16, 20, 33]))
    if hq > 200:
        hq = hkv
    B = int(rng.integers(1, 48))
    kind = trial % 5
    if kind == 0:
        lens = rng.integers(0, 300, B)
    elif kind == 1:
        lens = rng.integers(1, 5000, B)
    elif kind == 2:
        lens = np.where(rng.random(B) < 0.3, 0, rng.integers(1, 1200, B))
    elif kind == 3:
        lens = rng.choice([1, 31, 32, 33, 63, 64, 65, 767, 768, 769, 1024], B)
    else:
        lens = np.full(B, int(rng.integers(1, 3000)))
    lens = lens.astype(np.int32)
    lens[0] = max(int(lens[0]), 2)
    bs = int(rng.choice([16, 32, 8, 12, 1, 64]))
    static = trial % 4 == 1
    q_dtype = F16 if trial % 3 else F32
    say(f"random decode trial={trial} D={D} hq={hq} hkv={hkv} B={B} bs={bs} tokens={int(lens.sum())} "
        f"q_dtype={q_dtype} static_scratch={static}")
    case = W.make_paged_decode(seed=8000 + trial, num_heads=hq, num_kv_heads=hkv, head_dim=D, block_size=bs,
                               ctx_max=int(max(lens.max(), 64)), seq_lens=lens)
    want, want_lse = oracle.batched_paged_decode(case.q.astype(np.float32), case.k_pool, case.v_pool,
                                                 case.block_tables, case.seq_lens, bs, case.scale)
    out, lse = dev(np.full((B, hq, D), -7.0, np.float32)), dev(np.full((B, hq), -7.0, np.float32))
    bufs = (dev(case.q if q_dtype == F16 else case.q.astype(np.float32)), dev(case.k_pool), dev(case.v_pool),
            dev(case.block_tables), dev(case.seq_lens))
    kwargs = dict(q=bufs[0], q_dtype=q_dtype, k_cache=bufs[1], v_cache=bufs[2], block_tables=bufs[3], seq_lens=bufs[4],
                  out=out, lse=lse, batch_size=B, num_heads=hq, num_kv_heads=hkv, head_dim=D, scale=case.scale,
                  block_size=bs, max_blocks_per_seq=case.max_blocks)
    if static and gpu.decode_attention(**kwargs, query_workspace=True) > _capi.load().granite_hip_static_scratch_bytes():
        with pytest.raises(GraniteHipError) as e:     # more partial slots than the static array holds
            gpu.decode_attention(**kwargs, static_scratch=True)
        assert e.value.code == _capi.ESCRATCH
        static = False
    gpu.decode_attention(**kwargs, static_scratch=static)
    gpu.sync()
    got, got_lse = out.read(np.float32, (B, hq, D)), lse.read(np.float32, (B, hq))
    live = lens > 0
    assert_close(got[live], want[live], "out")
    assert_lse(got_lse[live], want_lse[live], "lse")
    assert np.all(got[~live] == -7.0) and np.all(got_lse[~live] == -7.0)


@pytest.mark.parametrize("trial", range(16))
def test_random_chunked_prefill(gpu, oracle, trial):
    rng = np.random.default_rng(7100 + trial)
    D = int(rng.choice([64, 128]))
    hkv = int(rng.choice([1, 2, 4, 8]))
    hq = hkv * int(rng.choice([1, 2, 4, 8]))
    chunk = int(rng.choice([1, 31, 64, 100, 127, 128, 129, 255, 256, 257, 300, 384, 385, 511, 640, 700, 1025]))
    prefix = int(rng.choice([0, 0, 1, 63, 64, 100, 500, 1500, 4000]))
    bs = int(rng.choice([16, 32, 8, 12]))
    f32 = trial % 3 == 0
    say(f"random prefill trial={trial} D={D} hq={hq} hkv={hkv} chunk={chunk} prefix={prefix} bs={bs} f32={f32}")
    case = W.make_chunked_prefill(seed=8100 + trial, prefix_len=prefix, chunk=chunk, num_heads=hq, num_kv_heads=hkv,
                                  head_dim=D, block_size=bs, pool_slack=1.3, value_scale=1.0)
    total = prefix + chunk
    dk, dv, dt = dev(case.k_pool), dev(case.v_pool), dev(case.block_table)
    gpu.paged_kv_cache_append_ex(dev(case.k_new), dev(case.v_new), F16, hkv * D, D, dk, dv, dt, hkv, D, prefix, chunk,
                                 bs, max_blocks=len(case.block_table))
    gpu.sync()
    pool_k, pool_v = dk.read(np.uint16, case.k_pool.shape), dv.read(np.uint16, case.v_pool.shape)
    want, want_lse = oracle.attention_paged(case.q[None].astype(np.float32), pool_k, pool_v, case.block_table, bs,
                                            total, prefix, case.scale)
    odt = np.float32 if f32 else np.float16
    out, lse = dev(np.zeros((chunk, hq, D), odt)), dev(np.zeros((hq, chunk), np.float32))
    gpu.attention(q=dev(case.q.astype(np.float32) if f32 else case.q), q_dtype=F32 if f32 else F16,
                  q_tok_stride=hq * D, q_head_stride=D, out=out, out_dtype=F32 if f32 else F16, out_tok_stride=hq * D,
                  out_head_stride=D, lse=lse, seq_q=chunk, num_heads=hq, num_kv_heads=hkv, head_dim=D,
                  scale=case.scale, k_cache=dk, v_cache=dv, cache_len=total, block_table=dt, block_size=bs,
                  mask_mode=MASK_CAUSAL, start_pos=prefix)
    gpu.sync()
    assert_close(out.read(odt, (chunk, hq, D)).astype(np.float32), want[0], "out")
    assert_lse(lse.read(np.float32, (hq, chunk)), want_lse[0], "lse")


@pytest.mark.parametrize("trial", range(10))
def test_random_tree_attention(gpu, oracle, trial):
    rng = np.random.default_rng(7200 + trial)
    D = int(rng.choice([64, 128]))
    hkv = int(rng.choice([1, 2, 8]))
    hq = hkv * int(rng.choice([1, 4, 8]))
    n = int(rng.choice([1, 5, 31, 32, 33, 64, 100, 200, 256, 257, 300]))
    prefix = int(rng.choice([0, 17, 64, 500, 3000]))
    bs = int(rng.choice([16, 8, 4]))
    say(f"random tree trial={trial} D={D} hq={hq} hkv={hkv} nodes={n} prefix={prefix} bs={bs}")
    case = W.make_tree(seed=8200 + trial, prefix_len=prefix, num_nodes=n, num_heads=hq, num_kv_heads=hkv, head_dim=D,
                       block_size=bs, max_children=3, max_depth=12)
    q = np.transpose(case.q, (1, 0, 2))[None]
    kt = np.transpose(case.k_tree, (1, 0, 2))[None].astype(np.float32)
    vt = np.transpose(case.v_tree, (1, 0, 2))[None].astype(np.float32)
    ctx, want_lse = oracle.attention_tree(q, case.k_pool if prefix else None, case.v_pool if prefix else None, kt, vt,
                                          case.parents, prefix, case.scale,
                                          table=case.block_table if prefix else None, block_size=bs)
    out, lse = dev(np.zeros((hq, n, D), np.float32)), dev(np.zeros((hq, n), np.float32))
    gpu.attention(q=dev(case.q), q_dtype=F32, q_tok_stride=D, q_head_stride=n * D, out=out, out_dtype=F32,
                  out_tok_stride=D, out_head_stride=n * D, lse=lse, seq_q=n, num_heads=hq, num_kv_heads=hkv,
                  head_dim=D, scale=case.scale, k_cache=dev(case.k_pool), v_cache=dev(case.v_pool), cache_len=prefix,
                  block_table=dev(case.block_table) if prefix else None, block_size=bs, max_seq=prefix,
                  k_extra=dev(case.k_tree), v_extra=dev(case.v_tree), extra_len=n, parents=dev(case.parents),
                  mask_mode=MASK_TREE)
    gpu.sync()
    assert_close(out.read(np.float32, (hq, n, D)), np.transpose(ctx[0], (1, 0, 2)), "out")
    assert_lse(lse.read(np.float32, (hq, n)), want_lse[0], "lse")
