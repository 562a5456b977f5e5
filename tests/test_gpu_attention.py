"""GPU parity: prefill, chunked prefill over a paged cache and tree attention
against the oracle's restatement of src/llm/transformer.mm:1779-1840 and
:2044-2126.  Tolerances: outputs |d| <= 2e-3 or <= 1e-2 |ref|; lse 1e-4."""
import numpy as np
import pytest

from granite_amd import (F16, F32, MASK_CAUSAL, MASK_NONE, MASK_TREE, GraniteHipError, _capi)
from granite_amd import workloads as W
from gpu_util import assert_close, assert_lse, dev, say
import ref64

pytestmark = pytest.mark.gpu


def _prefill(gpu, q, k_cache, v_cache, seq_q, total, start, hq, hkv, max_seq, scale, q_dtype, out_dtype,
             table=None, bs=0):
    """q [seq_q, hq, 128]; returns out [seq_q, hq, 128] (as float32) and lse [hq, seq_q]."""
    odt = np.float32 if out_dtype == F32 else np.float16
    out = dev(np.zeros((seq_q, hq, 128), odt))
    lse = dev(np.zeros((hq, seq_q), np.float32))
    gpu.attention(q=dev(q), q_dtype=q_dtype, q_tok_stride=hq * 128, q_head_stride=128, out=out,
                  out_dtype=out_dtype, out_tok_stride=hq * 128, out_head_stride=128, lse=lse, seq_q=seq_q,
                  num_heads=hq, num_kv_heads=hkv, head_dim=128, scale=scale, k_cache=dev(k_cache),
                  v_cache=dev(v_cache), cache_len=total, max_seq=max_seq,
                  block_table=None if table is None else dev(table), block_size=bs, mask_mode=MASK_CAUSAL,
                  start_pos=start)
    gpu.sync()
    return out.read(odt, (seq_q, hq, 128)).astype(np.float32), lse.read(np.float32, (hq, seq_q))


@pytest.mark.parametrize("seq,hq,hkv,max_seq", [(1, 4, 4, 8), (5, 8, 2, 64), (64, 4, 1, 64), (65, 8, 8, 100),
                                                (127, 4, 2, 128), (128, 4, 2, 128), (129, 4, 2, 200),
                                                (300, 32, 8, 300), (512, 16, 2, 1024)])
@pytest.mark.parametrize("q_dtype,out_dtype", [(F16, F16), (F32, F32)])
def test_causal_prefill_small(gpu, oracle, seq, hq, hkv, max_seq, q_dtype, out_dtype):
    say(f"prefill seq={seq} hq={hq} hkv={hkv} max_seq={max_seq} q={q_dtype} out={out_dtype}")
    case = W.make_prefill(seed=seq * 3 + hq, seq=seq, num_heads=hq, num_kv_heads=hkv, max_seq=max_seq)
    q32 = case.q.astype(np.float32)
    if q_dtype == F32:   # exercise the fp32-Q path with values that are NOT half-representable
        q32 = q32 + np.random.default_rng(1).standard_normal(q32.shape).astype(np.float32) * 1e-3
    want, want_lse = oracle.attention_cached(q32[None], case.k_cache, case.v_cache, seq, 0, case.scale)
    got, got_lse = _prefill(gpu, q32 if q_dtype == F32 else case.q, case.k_cache, case.v_cache, seq, seq, 0, hq,
                            hkv, max_seq, case.scale, q_dtype, out_dtype)
    assert_close(got, want[0], "out")
    assert_lse(got_lse, want_lse[0], "lse")
    # query 0 sees only key 0: the output row is V[0] (up to the final 1/l multiply)
    for h in range(hq):
        assert np.allclose(got[0, h], case.v_cache[h // (hq // hkv), 0].astype(np.float32), rtol=1e-6, atol=0)


def test_causal_prefill_config(gpu, oracle):
    """seq 2048, 32 q heads, 8 KV heads, D=128, fp16 in/out."""
    case = W.make_prefill()
    say("prefill config seq=2048")
    got, got_lse = _prefill(gpu, case.q, case.k_cache, case.v_cache, 2048, 2048, 0, 32, 8, 2048, case.scale, F16,
                            F16)
    # every one of the 2048 rows against the oracle (34 GFLOP of scalar code: seconds)
    want, want_lse = oracle.attention_cached(case.q[None].astype(np.float32), case.k_cache, case.v_cache, 2048, 0,
                                             case.scale)
    assert_close(got, want[0], "out")
    assert_lse(got_lse, want_lse[0], "lse")


def test_reference_entry_point_multihead_attention(gpu, oracle):
    """MetalCompute::multihead_attention with seq_q > 1: fp32 Q/out [seq, Hq, D],
    cache stride max_seq, start_pos 0."""
    case = W.make_prefill(seed=11, seq=200, num_heads=8, num_kv_heads=2, max_seq=256)
    q32 = case.q.astype(np.float32) * np.float32(1.001)
    want, _ = oracle.attention_cached(q32[None], case.k_cache, case.v_cache, 200, 0, case.scale)
    out = dev(np.zeros((200, 8, 128), np.float32))
    gpu.multihead_attention(dev(q32), dev(case.k_cache), dev(case.v_cache), out, 8, 2, 200, 200, 128, case.scale,
                            256)
    gpu.sync()
    assert_close(out.read(np.float32, (200, 8, 128)), want[0], "out")


@pytest.mark.parametrize("prefix,chunk,bs,hq,hkv", [(0, 40, 16, 8, 2), (100, 30, 16, 8, 2), (1000, 128, 32, 16, 2),
                                                    (511, 65, 4, 8, 8), (300, 200, 12, 4, 1)])
def test_chunked_prefill_over_paged_cache_small(gpu, oracle, prefix, chunk, bs, hq, hkv):
    say(f"chunked prefill prefix={prefix} chunk={chunk} bs={bs} hq={hq} hkv={hkv}")
    case = W.make_chunked_prefill(seed=prefix + chunk, prefix_len=prefix, chunk=chunk, num_heads=hq,
                                  num_kv_heads=hkv, block_size=bs, pool_slack=1.5)
    total = prefix + chunk
    dk, dv, dt = dev(case.k_pool), dev(case.v_pool), dev(case.block_table)
    # append the chunk's K/V (half, [chunk, Hkv, D]) at positions prefix.. : bit exact
    gpu.paged_kv_cache_append_ex(dev(case.k_new), dev(case.v_new), F16, hkv * 128, 128, dk, dv, dt, hkv, 128,
                                 prefix, chunk, bs)
    want_k, want_v = case.k_pool.view(np.uint16).copy(), case.v_pool.view(np.uint16).copy()
    oracle.lib.go_paged_kv_cache_append_f16(want_k.reshape(-1), case.k_new.view(np.uint16).reshape(-1),
                                            case.block_table, hkv, 128, prefix, chunk, bs, hkv * 128, 128)
    oracle.lib.go_paged_kv_cache_append_f16(want_v.reshape(-1), case.v_new.view(np.uint16).reshape(-1),
                                            case.block_table, hkv, 128, prefix, chunk, bs, hkv * 128, 128)
    gpu.sync()
    assert np.array_equal(dk.read(np.uint16, want_k.shape), want_k)
    assert np.array_equal(dv.read(np.uint16, want_v.shape), want_v)
    want, want_lse = oracle.attention_paged(case.q[None].astype(np.float32), want_k, want_v, case.block_table, bs,
                                            total, prefix, case.scale)
    out, lse = dev(np.zeros((chunk, hq, 128), np.float16)), dev(np.zeros((hq, chunk), np.float32))
    gpu.attention(q=dev(case.q), q_dtype=F16, q_tok_stride=hq * 128, q_head_stride=128, out=out, out_dtype=F16,
                  out_tok_stride=hq * 128, out_head_stride=128, lse=lse, seq_q=chunk, num_heads=hq,
                  num_kv_heads=hkv, head_dim=128, scale=case.scale, k_cache=dk, v_cache=dv, cache_len=total,
                  block_table=dt, block_size=bs, mask_mode=MASK_CAUSAL, start_pos=prefix)
    gpu.sync()
    assert_close(out.read(np.float16, (chunk, hq, 128)).astype(np.float32), want[0], "out")
    assert_lse(lse.read(np.float32, (hq, chunk)), want_lse[0], "lse")


@pytest.mark.parametrize("trial", range(12))
def test_chunked_prefill_random_shapes(gpu, oracle, trial):
    """Seeded random chunk lengths around the 128- and 256-row edges, prefixes, head counts and
    block sizes, fp16 and fp32 queries: exercises the pairing of row runs, the key splits and
    the first-tile handling of the softmax reference."""
    rng = np.random.default_rng(500 + trial)
    hkv = int(rng.choice([1, 2, 4, 8]))
    hq = hkv * int(rng.choice([1, 2, 4, 8]))
    chunk = int(rng.choice([1, 31, 64, 127, 128, 129, 255, 256, 257, 384, 385, 511, 640]))
    prefix = int(rng.choice([0, 1, 63, 64, 100, 500, 1200]))
    bs = int(rng.choice([16, 32, 8, 12]))
    say(f"chunked prefill random trial={trial} hq={hq} hkv={hkv} chunk={chunk} prefix={prefix} bs={bs}")
    case = W.make_chunked_prefill(seed=trial, prefix_len=prefix, chunk=chunk, num_heads=hq, num_kv_heads=hkv,
                                  block_size=bs, pool_slack=1.3, value_scale=1.0)
    total = prefix + chunk
    dk, dv, dt = dev(case.k_pool), dev(case.v_pool), dev(case.block_table)
    gpu.paged_kv_cache_append_ex(dev(case.k_new), dev(case.v_new), F16, hkv * 128, 128, dk, dv, dt, hkv, 128,
                                 prefix, chunk, bs)
    gpu.sync()
    pool_k, pool_v = dk.read(np.uint16, case.k_pool.shape), dv.read(np.uint16, case.v_pool.shape)
    want, want_lse = oracle.attention_paged(case.q[None].astype(np.float32), pool_k, pool_v, case.block_table, bs,
                                            total, prefix, case.scale)
    f32 = trial % 3 == 0
    q_host = case.q.astype(np.float32) if f32 else case.q
    out = dev(np.zeros((chunk, hq, 128), np.float32 if f32 else np.float16))
    lse = dev(np.zeros((hq, chunk), np.float32))
    gpu.attention(q=dev(q_host), q_dtype=F32 if f32 else F16, q_tok_stride=hq * 128, q_head_stride=128, out=out,
                  out_dtype=F32 if f32 else F16, out_tok_stride=hq * 128, out_head_stride=128, lse=lse, seq_q=chunk,
                  num_heads=hq, num_kv_heads=hkv, head_dim=128, scale=case.scale, k_cache=dk, v_cache=dv,
                  cache_len=total, block_table=dt, block_size=bs, mask_mode=MASK_CAUSAL, start_pos=prefix)
    gpu.sync()
    got = out.read(np.float32 if f32 else np.float16, (chunk, hq, 128)).astype(np.float32)
    assert_close(got, want[0], "out")
    assert_lse(lse.read(np.float32, (hq, chunk)), want_lse[0], "lse")


def test_chunked_prefill_config(gpu, oracle):
    """32768-token paged prefix (block 32), 512-token chunk, 64 q heads, 8 KV
    heads, values 0.5*N(0,1); append bit-exact, attention on every 8th row and the
    rows at the run edges."""
    case = W.make_chunked_prefill()
    say("chunked prefill config prefix=32768 chunk=512")
    hq, hkv, bs, prefix, chunk = 64, 8, 32, case.prefix_len, case.chunk
    total = prefix + chunk
    dk, dv, dt = dev(case.k_pool), dev(case.v_pool), dev(case.block_table)
    gpu.paged_kv_cache_append_ex(dev(case.k_new), dev(case.v_new), F16, hkv * 128, 128, dk, dv, dt, hkv, 128,
                                 prefix, chunk, bs)
    gpu.sync()
    k_all = ref64.gather_paged(case.k_pool, case.block_table, bs, total).copy()
    v_all = ref64.gather_paged(case.v_pool, case.block_table, bs, total).copy()
    k_all[prefix:], v_all[prefix:] = case.k_new, case.v_new
    gk = dev(np.zeros((hkv, total, 128), np.uint16))
    gv = dev(np.zeros((hkv, total, 128), np.uint16))
    gpu.paged_kv_gather(gk, gv, dk, dv, dt, hkv, 128, total, bs, total)
    gpu.sync()
    assert np.array_equal(gk.read(np.uint16, (hkv, total, 128)), np.transpose(k_all.view(np.uint16), (1, 0, 2)))
    assert np.array_equal(gv.read(np.uint16, (hkv, total, 128)), np.transpose(v_all.view(np.uint16), (1, 0, 2)))
    out, lse = dev(np.zeros((chunk, hq, 128), np.float16)), dev(np.zeros((hq, chunk), np.float32))
    gpu.attention(q=dev(case.q), q_dtype=F16, q_tok_stride=hq * 128, q_head_stride=128, out=out, out_dtype=F16,
                  out_tok_stride=hq * 128, out_head_stride=128, lse=lse, seq_q=chunk, num_heads=hq,
                  num_kv_heads=hkv, head_dim=128, scale=case.scale, k_cache=dk, v_cache=dv, cache_len=total,
                  block_table=dt, block_size=bs, mask_mode=MASK_CAUSAL, start_pos=prefix)
    gpu.sync()
    got = out.read(np.float16, (chunk, hq, 128)).astype(np.float32)
    got_lse = lse.read(np.float32, (hq, chunk))
    k32, v32 = k_all.astype(np.float32), v_all.astype(np.float32)
    # every 8th row, the rows either side of the 128-row run edges and of the seam where the
    # paired runs of a workgroup meet, and the first and last row of the chunk
    rows = sorted(set(range(0, chunk, 8)) | {1, 31, 127, 128, 129, 255, 256, 257, 383, 384, 385, 510, 511})
    for r in rows:
        want, want_lse = oracle.attention_core(case.q[None, r:r + 1].astype(np.float32), k32[:prefix + r + 1],
                                               v32[:prefix + r + 1], prefix + r, case.scale)
        assert_close(got[r], want[0, 0], f"row {r}")
        assert_lse(got_lse[:, r], want_lse[0, :, 0], f"lse row {r}")


# ---- tree ---------------------------------------------------------------------

def _tree_oracle(oracle, case):
    n = case.num_nodes
    q = np.transpose(case.q, (1, 0, 2))[None]                       # [1, N, Hq, D]
    kt = np.transpose(case.k_tree, (1, 0, 2))[None].astype(np.float32)
    vt = np.transpose(case.v_tree, (1, 0, 2))[None].astype(np.float32)
    ctx, lse = oracle.attention_tree(q, case.k_pool if case.prefix_len else None,
                                     case.v_pool if case.prefix_len else None, kt, vt, case.parents,
                                     case.prefix_len, case.scale, table=case.block_table if case.prefix_len else None,
                                     block_size=case.block_size)
    return np.transpose(ctx[0], (1, 0, 2)), lse[0]                  # [Hq, N, D], [Hq, N]


def _tree_gpu(gpu, case):
    hq, n = case.num_heads, case.num_nodes
    out, lse = dev(np.zeros((hq, n, 128), np.float32)), dev(np.zeros((hq, n), np.float32))
    gpu.attention(q=dev(case.q), q_dtype=F32, q_tok_stride=128, q_head_stride=n * 128, out=out, out_dtype=F32,
                  out_tok_stride=128, out_head_stride=n * 128, lse=lse, seq_q=n, num_heads=hq,
                  num_kv_heads=case.num_kv_heads, head_dim=128, scale=case.scale,
                  k_cache=dev(case.k_pool), v_cache=dev(case.v_pool), cache_len=case.prefix_len,
                  block_table=dev(case.block_table) if case.prefix_len else None, block_size=case.block_size,
                  max_seq=case.prefix_len, k_extra=dev(case.k_tree), v_extra=dev(case.v_tree), extra_len=n,
                  parents=dev(case.parents), mask_mode=MASK_TREE)
    gpu.sync()
    return out.read(np.float32, (hq, n, 128)), lse.read(np.float32, (hq, n))


@pytest.mark.parametrize("prefix,n,hq,hkv,bs", [(0, 1, 4, 4, 16), (0, 13, 8, 2, 16), (37, 5, 8, 2, 4),
                                                (500, 64, 32, 8, 16), (64, 100, 4, 1, 16), (200, 130, 8, 2, 8),
                                                # 256 nodes: the largest tree whose mask the attention kernel
                                                # builds itself; 257 and 300: through the mask kernel
                                                (30, 256, 4, 2, 16), (30, 257, 4, 2, 16), (0, 300, 2, 1, 16)])
def test_tree_attention_small(gpu, oracle, prefix, n, hq, hkv, bs):
    say(f"tree prefix={prefix} nodes={n} hq={hq} hkv={hkv} bs={bs}")
    case = W.make_tree(seed=prefix * 5 + n, prefix_len=prefix, num_nodes=n, num_heads=hq, num_kv_heads=hkv,
                       block_size=bs, max_children=3, max_depth=12)
    want, want_lse = _tree_oracle(oracle, case)
    got, got_lse = _tree_gpu(gpu, case)
    assert_close(got, want, "out")
    assert_lse(got_lse, want_lse, "lse")


def test_tree_attention_config(gpu, oracle):
    """4096-token paged prefix (block 16) + 64-node random tree (branching <= 4,
    depth <= 8), 32 q heads, 8 KV heads."""
    case = W.make_tree()
    say("tree config prefix=4096 nodes=64")
    want, want_lse = _tree_oracle(oracle, case)
    got, got_lse = _tree_gpu(gpu, case)
    assert_close(got, want, "out")
    assert_lse(got_lse, want_lse, "lse")


def test_tree_mask_kernel(gpu, oracle):
    rng = np.random.default_rng(2)
    for n in (1, 31, 32, 33, 64, 200):
        parents = W.random_tree(rng, n, 3, 20)
        words = (n + 31) // 32
        mask = dev(np.zeros((n, words), np.uint32))
        gpu.build_tree_mask(dev(parents), mask, n)
        gpu.sync()
        got = mask.read(np.uint32, (n, words))
        bits = ((got[:, :, None] >> np.arange(32, dtype=np.uint32)) & 1).reshape(n, words * 32)[:, :n]
        assert np.array_equal(bits.astype(np.uint8), oracle.tree_mask(parents))
    # a cyclic parent array must still terminate (bounded walk)
    cyc = np.array([1, 0, 1], np.int32)
    mask = dev(np.zeros((3, 1), np.uint32))
    gpu.build_tree_mask(dev(cyc), mask, 3)
    gpu.sync()
    assert mask.read(np.uint32, (3, 1))[2, 0] == 0b111


def test_reference_entry_point_attention_tree(gpu, oracle):
    """MetalCompute::attention_tree: contiguous cache with row stride cache_len."""
    rng = np.random.default_rng(4)
    hq, hkv, n, cache_len = 8, 2, 20, 77
    parents = W.random_tree(rng, n, 3, 6)
    q = rng.standard_normal((hq, n, 128)).astype(np.float16).astype(np.float32)
    ck = rng.standard_normal((hkv, cache_len, 128)).astype(np.float16)
    cv = rng.standard_normal((hkv, cache_len, 128)).astype(np.float16)
    kt = rng.standard_normal((hkv, n, 128)).astype(np.float16)
    vt = rng.standard_normal((hkv, n, 128)).astype(np.float16)
    scale = float(1 / np.sqrt(128))
    ctx, _ = oracle.attention_tree(np.transpose(q, (1, 0, 2))[None], ck, cv,
                                   np.transpose(kt, (1, 0, 2))[None].astype(np.float32),
                                   np.transpose(vt, (1, 0, 2))[None].astype(np.float32), parents, cache_len, scale,
                                   max_seq=cache_len)
    out = dev(np.zeros((hq, n, 128), np.float32))
    gpu.attention_tree(dev(q), dev(ck), dev(cv), dev(kt), dev(vt), dev(parents), out, hq, hkv, n, cache_len, 128,
                       scale)
    gpu.sync()
    assert_close(out.read(np.float32, (hq, n, 128)), np.transpose(ctx[0], (1, 0, 2)), "out")


def test_chain_tree_equals_causal_on_gpu(gpu):
    """parent[i] = i-1 over a contiguous prefix is causal attention."""
    rng = np.random.default_rng(6)
    hq, hkv, n, prefix = 8, 2, 70, 90
    total = prefix + n
    kc = rng.standard_normal((hkv, total, 128)).astype(np.float16)
    vc = rng.standard_normal((hkv, total, 128)).astype(np.float16)
    q = rng.standard_normal((n, hq, 128)).astype(np.float16)
    scale = float(1 / np.sqrt(128))
    causal, causal_lse = _prefill(gpu, q, kc, vc, n, total, prefix, hq, hkv, total, scale, F16, F32)
    out, lse = dev(np.zeros((n, hq, 128), np.float32)), dev(np.zeros((hq, n), np.float32))
    chain = np.arange(-1, n - 1, dtype=np.int32)
    gpu.attention(q=dev(q), q_dtype=F16, q_tok_stride=hq * 128, q_head_stride=128, out=out, out_dtype=F32,
                  out_tok_stride=hq * 128, out_head_stride=128, lse=lse, seq_q=n, num_heads=hq, num_kv_heads=hkv,
                  head_dim=128, scale=scale, k_cache=dev(kc), v_cache=dev(vc), cache_len=prefix, max_seq=total,
                  k_extra=dev(kc[:, prefix:].copy()), v_extra=dev(vc[:, prefix:].copy()), extra_len=n,
                  parents=dev(chain), mask_mode=MASK_TREE)
    gpu.sync()
    assert_close(out.read(np.float32, (n, hq, 128)), causal, "tree vs causal", abs_tol=1e-4, rel_tol=1e-4)
    assert_lse(lse.read(np.float32, (hq, n)), causal_lse, "lse", tol=2e-5)


def test_attention_rejects_bad_arguments(gpu):
    buf = dev(np.zeros(1 << 16, np.float32))
    base = dict(q=buf, q_dtype=F32, q_tok_stride=1024, q_head_stride=128, out=buf, out_dtype=F32,
                out_tok_stride=1024, out_head_stride=128, seq_q=4, num_heads=8, num_kv_heads=2, head_dim=128,
                scale=0.1, k_cache=buf, v_cache=buf, cache_len=4, max_seq=8, mask_mode=MASK_CAUSAL)
    for bad, code in ((dict(head_dim=96), _capi.EUNSUPPORTED), (dict(num_kv_heads=3), _capi.EINVAL),
                      (dict(out=None), _capi.ENULL), (dict(max_seq=2), _capi.EINVAL),
                      (dict(mask_mode=9), _capi.EINVAL), (dict(q_tok_stride=1022), _capi.EINVAL),
                      (dict(mask_mode=MASK_TREE), _capi.ENULL), (dict(cache_len=0), _capi.EINVAL),
                      (dict(k_extra=buf, v_extra=buf, extra_len=4), _capi.EUNSUPPORTED)):
        with pytest.raises(GraniteHipError) as e:
            gpu.attention(**{**base, **bad})
        assert e.value.code == code, bad


# ---- head size 64 (the reference's d64 kernels, metal_shaders_attention.h:1447-1660, 2769-2977) ----

@pytest.mark.parametrize("seq,hq,hkv,max_seq", [(1, 4, 4, 8), (65, 8, 2, 100), (128, 4, 2, 128), (300, 16, 4, 300),
                                                (700, 8, 8, 1024)])
@pytest.mark.parametrize("q_dtype,out_dtype", [(F16, F16), (F32, F32)])
def test_causal_prefill_head_dim_64(gpu, oracle, seq, hq, hkv, max_seq, q_dtype, out_dtype):
    say(f"prefill d64 seq={seq} hq={hq} hkv={hkv} max_seq={max_seq} q={q_dtype} out={out_dtype}")
    case = W.make_prefill(seed=seq + hq, seq=seq, num_heads=hq, num_kv_heads=hkv, head_dim=64, max_seq=max_seq)
    q32 = case.q.astype(np.float32)
    if q_dtype == F32:
        q32 = q32 + np.random.default_rng(1).standard_normal(q32.shape).astype(np.float32) * 1e-3
    want, want_lse = oracle.attention_cached(q32[None], case.k_cache, case.v_cache, seq, 0, case.scale)
    odt = np.float32 if out_dtype == F32 else np.float16
    out, lse = dev(np.zeros((seq, hq, 64), odt)), dev(np.zeros((hq, seq), np.float32))
    gpu.attention(q=dev(q32 if q_dtype == F32 else case.q), q_dtype=q_dtype, q_tok_stride=hq * 64, q_head_stride=64,
                  out=out, out_dtype=out_dtype, out_tok_stride=hq * 64, out_head_stride=64, lse=lse, seq_q=seq,
                  num_heads=hq, num_kv_heads=hkv, head_dim=64, scale=case.scale, k_cache=dev(case.k_cache),
                  v_cache=dev(case.v_cache), cache_len=seq, max_seq=max_seq, mask_mode=MASK_CAUSAL, start_pos=0)
    gpu.sync()
    assert_close(out.read(odt, (seq, hq, 64)).astype(np.float32), want[0], "out")
    assert_lse(lse.read(np.float32, (hq, seq)), want_lse[0], "lse")


@pytest.mark.parametrize("prefix,chunk,bs,hq,hkv", [(0, 40, 16, 8, 2), (1000, 128, 32, 16, 2), (3000, 96, 16, 8, 2),
                                                    (511, 300, 12, 4, 1)])
def test_chunked_prefill_head_dim_64(gpu, oracle, prefix, chunk, bs, hq, hkv):
    """Paged cache, key splits and the merge kernel at head size 64."""
    say(f"chunked prefill d64 prefix={prefix} chunk={chunk} bs={bs} hq={hq} hkv={hkv}")
    case = W.make_chunked_prefill(seed=prefix + chunk, prefix_len=prefix, chunk=chunk, num_heads=hq,
                                  num_kv_heads=hkv, head_dim=64, block_size=bs, pool_slack=1.5, value_scale=1.0)
    total = prefix + chunk
    dk, dv, dt = dev(case.k_pool), dev(case.v_pool), dev(case.block_table)
    gpu.paged_kv_cache_append_ex(dev(case.k_new), dev(case.v_new), F16, hkv * 64, 64, dk, dv, dt, hkv, 64, prefix,
                                 chunk, bs)
    gpu.sync()
    pool_k, pool_v = dk.read(np.uint16, case.k_pool.shape), dv.read(np.uint16, case.v_pool.shape)
    want, want_lse = oracle.attention_paged(case.q[None].astype(np.float32), pool_k, pool_v, case.block_table, bs,
                                            total, prefix, case.scale)
    out, lse = dev(np.zeros((chunk, hq, 64), np.float16)), dev(np.zeros((hq, chunk), np.float32))
    gpu.attention(q=dev(case.q), q_dtype=F16, q_tok_stride=hq * 64, q_head_stride=64, out=out, out_dtype=F16,
                  out_tok_stride=hq * 64, out_head_stride=64, lse=lse, seq_q=chunk, num_heads=hq, num_kv_heads=hkv,
                  head_dim=64, scale=case.scale, k_cache=dk, v_cache=dv, cache_len=total, block_table=dt,
                  block_size=bs, mask_mode=MASK_CAUSAL, start_pos=prefix)
    gpu.sync()
    assert_close(out.read(np.float16, (chunk, hq, 64)).astype(np.float32), want[0], "out")
    assert_lse(lse.read(np.float32, (hq, chunk)), want_lse[0], "lse")


@pytest.mark.parametrize("prefix,n,hq,hkv,bs", [(0, 13, 8, 2, 16), (500, 64, 32, 8, 16), (200, 130, 8, 2, 8)])
def test_tree_attention_head_dim_64(gpu, oracle, prefix, n, hq, hkv, bs):
    say(f"tree d64 prefix={prefix} nodes={n} hq={hq} hkv={hkv} bs={bs}")
    case = W.make_tree(seed=prefix * 5 + n, prefix_len=prefix, num_nodes=n, num_heads=hq, num_kv_heads=hkv,
                       head_dim=64, block_size=bs, max_children=3, max_depth=12)
    want, want_lse = _tree_oracle(oracle, case)
    out, lse = dev(np.zeros((hq, n, 64), np.float32)), dev(np.zeros((hq, n), np.float32))
    gpu.attention(q=dev(case.q), q_dtype=F32, q_tok_stride=64, q_head_stride=n * 64, out=out, out_dtype=F32,
                  out_tok_stride=64, out_head_stride=n * 64, lse=lse, seq_q=n, num_heads=hq,
                  num_kv_heads=hkv, head_dim=64, scale=case.scale, k_cache=dev(case.k_pool), v_cache=dev(case.v_pool),
                  cache_len=case.prefix_len, block_table=dev(case.block_table) if case.prefix_len else None,
                  block_size=bs, max_seq=case.prefix_len, k_extra=dev(case.k_tree), v_extra=dev(case.v_tree),
                  extra_len=n, parents=dev(case.parents), mask_mode=MASK_TREE)
    gpu.sync()
    assert_close(out.read(np.float32, (hq, n, 64)), want, "out")
    assert_lse(lse.read(np.float32, (hq, n)), want_lse, "lse")
