"""GPU parity: rotary embedding and the fused rotate-and-append through the C ABI, against the
oracle (src/llm/rope.cpp:5-92; kernel metal_shaders_util.h:596-635; appends
metal_shaders_attention.h:102-125, 2142-2176).  With the reference's cos/sin tables as input the
results must be bit-identical; with cos/sin evaluated on the device the bound is what two fp32
evaluations of the same angle can differ by."""
import numpy as np
import pytest

from granite_amd import ROUND_NEAREST, ROUND_TRUNCATE, GraniteHipError, _capi
from gpu_util import dev, say

pytestmark = pytest.mark.gpu
SENT = 0xBEEF


def _oracle_cache(oracle, k_rot, v, rounding):
    if rounding == ROUND_TRUNCATE:
        return oracle.fp32_to_fp16(k_rot), oracle.fp32_to_fp16(v)
    return k_rot.astype(np.float16).view(np.uint16), v.astype(np.float16).view(np.uint16)


@pytest.mark.parametrize("seq,hq,hkv,d,start", [(1, 32, 8, 128, 0), (1, 32, 8, 128, 777), (33, 8, 2, 64, 5),
                                                 (512, 64, 8, 128, 1024), (7, 4, 4, 8, 100), (40, 6, 1, 256, 0)])
def test_rope_tables_bit_exact(gpu, oracle, seq, hq, hkv, d, start):
    """RoPECache::apply semantics: rotated Q and K in float, in place."""
    say(f"rope tables seq={seq} hq={hq} hkv={hkv} d={d} start={start}")
    rng = np.random.default_rng(seq * 7 + d)
    q = rng.standard_normal((seq, hq, d)).astype(np.float32)
    k = rng.standard_normal((seq, hkv, d)).astype(np.float32)
    positions = start + seq + 3
    cos, sin = oracle.rope_table(positions, d, 10000.0)
    want_q, want_k = oracle.rope_apply(q, start, cos, sin), oracle.rope_apply(k, start, cos, sin)
    dq, dk, dcos, dsin = dev(q), dev(k), dev(cos), dev(sin)
    dq16 = dev(np.zeros((seq, hq, d), np.uint16))
    gpu.rope_append(seq_len=seq, head_dim=d, start_pos=start, q=dq, num_heads_q=hq, q_f16=dq16, k=dk,
                    num_heads_k=hkv, cos_table=dcos, sin_table=dsin, table_positions=positions)
    gpu.sync()
    got_q, got_k = dq.read(np.float32, q.shape), dk.read(np.float32, k.shape)
    assert np.array_equal(got_q.view(np.uint32), want_q.view(np.uint32))
    assert np.array_equal(got_k.view(np.uint32), want_k.view(np.uint32))
    assert np.array_equal(dq16.read(np.uint16, q.shape), want_q.astype(np.float16).view(np.uint16))


@pytest.mark.parametrize("rounding", [ROUND_TRUNCATE, ROUND_NEAREST])
@pytest.mark.parametrize("paged", [False, True])
def test_rope_append_fused_bit_exact(gpu, oracle, rounding, paged):
    """Rotate K, convert, scatter K and V into the cache rows of their positions: the same bits
    as the oracle's rotation followed by its append; everything else in the cache untouched."""
    seq, hq, hkv, d, start, bs = 70, 16, 4, 128, 37, 16
    say(f"rope+append fused rounding={rounding} paged={paged}")
    rng = np.random.default_rng(11 + rounding)
    q = rng.standard_normal((seq, hq, d)).astype(np.float32)
    k = (rng.standard_normal((seq, hkv, d)) * 3).astype(np.float32)
    v = (rng.standard_normal((seq, hkv, d)) * 3).astype(np.float32)
    v.reshape(-1)[:6] = [0.0, -0.0, 6e-5, 70000.0, -np.inf, 2.0 ** -15]
    cos, sin = oracle.rope_table(256, d, 10000.0)
    k_rot = oracle.rope_apply(k, start, cos, sin)
    hk, hv = _oracle_cache(oracle, k_rot, v, rounding)
    total = start + seq
    if paged:
        nblk = (total + bs - 1) // bs
        table = rng.permutation(nblk + 5)[:nblk].astype(np.int32)
        ck = np.full(((nblk + 5) * bs, hkv, d), SENT, np.uint16)
        cv = np.full(((nblk + 5) * bs, hkv, d), SENT + 1, np.uint16)
        want_k, want_v = ck.copy(), cv.copy()
        for s in range(seq):
            pos = start + s
            row = table[pos // bs] * bs + pos % bs
            want_k[row], want_v[row] = hk[s], hv[s]
        extra = dict(block_table=dev(table), block_size=bs)
    else:
        max_seq = 128
        ck = np.full((hkv, max_seq, d), SENT, np.uint16)
        cv = np.full((hkv, max_seq, d), SENT + 1, np.uint16)
        want_k, want_v = ck.copy(), cv.copy()
        want_k[:, start:total], want_v[:, start:total] = hk.transpose(1, 0, 2), hv.transpose(1, 0, 2)
        extra = dict(max_seq_len=max_seq)
    dq, dk, dv, dck, dcv, dcos, dsin = dev(q), dev(k), dev(v), dev(ck), dev(cv), dev(cos), dev(sin)
    gpu.rope_append(seq_len=seq, head_dim=d, start_pos=start, q=dq, num_heads_q=hq, k=dk, num_heads_k=hkv,
                    v=dv, cache_k=dck, cache_v=dcv, cos_table=dcos, sin_table=dsin, table_positions=256,
                    write_k_back=False, rounding=rounding, **extra)
    gpu.sync()
    assert np.array_equal(dck.read(np.uint16, ck.shape), want_k)
    assert np.array_equal(dcv.read(np.uint16, cv.shape), want_v)
    assert np.array_equal(dq.read(np.float32, q.shape), oracle.rope_apply(q, start, cos, sin))
    assert np.array_equal(dk.read(np.float32, k.shape), k)  # write_k_back off: K source untouched


def test_rope_multihead_device_cos_sin(gpu, oracle):
    """The reference-shaped entry point evaluates cos/sin on the device in float, as the Metal
    kernel does.  Two float evaluations of pos * base^(-2i/D) may differ by an ulp of the
    frequency times the position, so the bound grows with the position."""
    seq, hq, hkv, d = 64, 8, 2, 128
    for start in (0, 1000):
        rng = np.random.default_rng(start + 1)
        q = rng.standard_normal((seq, hq, d)).astype(np.float32)
        k = rng.standard_normal((seq, hkv, d)).astype(np.float32)
        cos, sin = oracle.rope_table(start + seq, d, 10000.0)
        want_q, want_k = oracle.rope_apply(q, start, cos, sin), oracle.rope_apply(k, start, cos, sin)
        dq, dk = dev(q), dev(k)
        gpu.rope_multihead(dq, dk, hq, hkv, seq, d, start, 10000.0)
        gpu.sync()
        tol = 2e-6 + (start + seq) * 2.0 ** -22
        for got, want, x in ((dq.read(np.float32, q.shape), want_q, q), (dk.read(np.float32, k.shape), want_k, k)):
            err = np.abs(got.astype(np.float64) - want)
            assert err.max() <= tol * np.abs(x).max(), (start, err.max())
        say(f"  rope_multihead start={start}: max err {err.max():.2e} (bound {tol * np.abs(x).max():.2e})")


def test_rope_full_chunk_shape_round_trip(gpu, oracle):
    """The chunked-prefill shape (512 new tokens at position 32768, 64 query heads, 8 KV heads,
    paged block 32): K cache rows against the oracle, and rotating back by the conjugate table
    recovers the input (the rotation loses nothing but rounding)."""
    seq, hq, hkv, d, start, bs = 512, 64, 8, 128, 32768, 32
    rng = np.random.default_rng(5)
    q = (rng.standard_normal((seq, hq, d)) * 0.5).astype(np.float32)
    k = (rng.standard_normal((seq, hkv, d)) * 0.5).astype(np.float32)
    v = (rng.standard_normal((seq, hkv, d)) * 0.5).astype(np.float32)
    positions = start + seq
    cos, sin = oracle.rope_table(positions, d, 10000.0)
    nblk = positions // bs
    table = rng.permutation(nblk).astype(np.int32)
    pool_k = np.zeros((nblk * bs, hkv, d), np.uint16)
    pool_v = np.zeros((nblk * bs, hkv, d), np.uint16)
    dq, dk, dv, dpk, dpv = dev(q), dev(k), dev(v), dev(pool_k), dev(pool_v)
    dcos, dsin, dt = dev(cos), dev(sin), dev(table)
    gpu.rope_append(seq_len=seq, head_dim=d, start_pos=start, q=dq, num_heads_q=hq, k=dk, num_heads_k=hkv,
                    v=dv, cache_k=dpk, cache_v=dpv, block_table=dt, block_size=bs, cos_table=dcos,
                    sin_table=dsin, table_positions=positions, rounding=ROUND_NEAREST)
    gpu.sync()
    k_rot = oracle.rope_apply(k, start, cos, sin)
    rows = table[(start + np.arange(seq)) // bs] * bs + (start + np.arange(seq)) % bs
    got_pool = dpk.read(np.uint16, pool_k.shape)
    assert np.array_equal(got_pool[rows], k_rot.astype(np.float16).view(np.uint16))
    assert np.array_equal(dpv.read(np.uint16, pool_v.shape)[rows], v.astype(np.float16).view(np.uint16))
    untouched = np.ones(nblk * bs, bool); untouched[rows] = False
    assert not got_pool[untouched].any()
    # rotate the device's Q back with (cos, -sin)
    dns = dev(-sin)
    gpu.rope_append(seq_len=seq, head_dim=d, start_pos=start, q=dq, num_heads_q=hq, cos_table=dcos,
                    sin_table=dns, table_positions=positions)
    gpu.sync()
    assert np.abs(dq.read(np.float32, q.shape) - q).max() <= 1e-6


def test_rope_append_batched_decode_positions(gpu, oracle):
    """A batch of decode steps: token s belongs to sequence s, at its own position and with its
    own block table.  Bit-exact against the oracle sequence by sequence; tokens whose position
    is negative or beyond the cos/sin tables are left alone, one beyond its block table is
    rotated but not stored."""
    B, hq, hkv, d, bs, max_blocks, positions_max = 6, 8, 2, 128, 16, 4, 100
    rng = np.random.default_rng(77)
    pos = np.array([0, 17, 63, -1, 100, 70], np.int32)   # 3: negative, 4: beyond the tables, 5: beyond 4 blocks
    q = rng.standard_normal((B, hq, d)).astype(np.float32)
    k = rng.standard_normal((B, hkv, d)).astype(np.float32)
    v = rng.standard_normal((B, hkv, d)).astype(np.float32)
    cos, sin = oracle.rope_table(positions_max, d, 10000.0)
    nblk = B * max_blocks
    tables = rng.permutation(nblk).astype(np.int32).reshape(B, max_blocks)
    pool_k = np.full((nblk * bs, hkv, d), SENT, np.uint16)
    pool_v = np.full((nblk * bs, hkv, d), SENT + 1, np.uint16)
    want_q, want_k, want_pk, want_pv = q.copy(), k.copy(), pool_k.copy(), pool_v.copy()
    for b in range(B):
        p = int(pos[b])
        if p < 0 or p >= positions_max:
            continue
        want_q[b:b + 1] = oracle.rope_apply(q[b:b + 1], p, cos, sin)
        want_k[b:b + 1] = oracle.rope_apply(k[b:b + 1], p, cos, sin)
        if p // bs < max_blocks:
            row = tables[b, p // bs] * bs + p % bs
            want_pk[row] = oracle.fp32_to_fp16(want_k[b])
            want_pv[row] = oracle.fp32_to_fp16(v[b])
    dq, dk, dv, dpk, dpv = dev(q), dev(k), dev(v), dev(pool_k), dev(pool_v)
    dcos, dsin, dt, dpos = dev(cos), dev(sin), dev(tables), dev(pos)
    gpu.rope_append(seq_len=B, head_dim=d, start_pos=0, q=dq, num_heads_q=hq, k=dk, num_heads_k=hkv, v=dv,
                    cache_k=dpk, cache_v=dpv, block_table=dt, block_size=bs, cos_table=dcos, sin_table=dsin,
                    table_positions=positions_max, positions=dpos, table_stride=max_blocks,
                    max_blocks_per_seq=max_blocks, rounding=ROUND_TRUNCATE)
    gpu.sync()
    assert np.array_equal(dq.read(np.float32, q.shape), want_q)
    assert np.array_equal(dk.read(np.float32, k.shape), want_k)
    assert np.array_equal(dpk.read(np.uint16, pool_k.shape), want_pk)
    assert np.array_equal(dpv.read(np.uint16, pool_v.shape), want_pv)
    with pytest.raises(GraniteHipError) as e:   # per-token positions over a paged cache need the table length
        gpu.rope_append(seq_len=B, head_dim=d, start_pos=0, k=dk, num_heads_k=hkv, v=dv, cache_k=dpk,
                        cache_v=dpv, block_table=dt, block_size=bs, positions=dpos, table_stride=max_blocks)
    assert e.value.code == _capi.EINVAL


def test_rope_argument_errors(gpu):
    buf = dev(np.zeros(4096, np.float32))
    base = dict(seq_len=2, head_dim=128, start_pos=0, q=buf, num_heads_q=2, k=buf, num_heads_k=1)
    for bad, code in ((dict(head_dim=6), _capi.EINVAL), (dict(head_dim=0), _capi.EINVAL),
                      (dict(cos_table=buf), _capi.ENULL), (dict(freq_base=0.0), _capi.EINVAL),
                      (dict(cos_table=buf, sin_table=buf, table_positions=1), _capi.EOVERFLOW),
                      (dict(cache_k=buf, cache_v=buf, v=buf, max_seq_len=1), _capi.EOVERFLOW),
                      (dict(cache_v=buf, v=buf), _capi.ENULL), (dict(cache_k=buf, cache_v=buf), _capi.ENULL),
                      (dict(q=None, k=None), _capi.ENULL), (dict(rounding=7), _capi.EINVAL)):
        with pytest.raises(GraniteHipError) as e:
            gpu.rope_append(**{**base, **bad})
        assert e.value.code == code, (bad, e.value.code)
    gpu.rope_append(**{**base, "seq_len": 0})  # nothing to do
