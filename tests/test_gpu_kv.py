"""GPU parity: KV append / gather through the C ABI, bit-exact against the
oracle (src/llm/kv_cache.cpp:55-107; metal_shaders_attention.h:102-125,
2142-2176)."""
import numpy as np
import pytest

from granite_amd import F16, F32, ROUND_NEAREST, ROUND_TRUNCATE, GraniteHipError, _capi
from gpu_util import dev, say

pytestmark = pytest.mark.gpu
SENT = 0xBEEF


def _interesting_floats(rng, shape):
    """Normals plus the values that separate truncation from rounding:
    subnormal-range, overflow-range, NaN, Inf, signed zeros."""
    x = (rng.standard_normal(shape) * 4).astype(np.float32)
    flat = x.reshape(-1)
    special = np.array([0.0, -0.0, 6e-5, -6e-5, 65520.0, 65536.0, -70000.0, np.inf, -np.inf,
                        np.nan, 1.0 + 3 * 2.0**-12, 2.0**-14, 2.0**-15, 1e-8, 3.4e38], np.float32)
    idx = rng.choice(flat.size, size=min(flat.size, special.size * 4), replace=False)
    flat[idx] = np.resize(special, idx.size)
    return x


@pytest.mark.parametrize("hkv,d,max_seq,cur,new", [(8, 128, 512, 0, 1), (8, 128, 512, 511, 1),
                                                   (8, 128, 2048, 100, 300), (2, 64, 40, 3, 17),
                                                   (1, 128, 8, 0, 8)])
def test_kv_cache_append_f32(gpu, oracle, hkv, d, max_seq, cur, new):
    say(f"kv_cache_append f32 hkv={hkv} d={d} max_seq={max_seq} cur={cur} new={new}")
    rng = np.random.default_rng(cur * 31 + new)
    nk, nv = _interesting_floats(rng, (new, hkv, d)), _interesting_floats(rng, (new, hkv, d))
    ck = np.full((hkv, max_seq, d), SENT, np.uint16)
    cv = np.full((hkv, max_seq, d), SENT + 1, np.uint16)
    want_k, want_v = ck.copy(), cv.copy()
    assert oracle.lib.go_kv_cache_append_f32(want_k.reshape(-1), nk.reshape(-1), hkv, d, cur, new, max_seq) == 0
    assert oracle.lib.go_kv_cache_append_f32(want_v.reshape(-1), nv.reshape(-1), hkv, d, cur, new, max_seq) == 0
    dck, dcv, dnk, dnv = dev(ck), dev(cv), dev(nk), dev(nv)
    gpu.kv_cache_append(dck, dcv, dnk, dnv, hkv, d, cur, new, max_seq)
    gpu.sync()
    assert np.array_equal(dck.read(np.uint16, ck.shape), want_k)
    assert np.array_equal(dcv.read(np.uint16, cv.shape), want_v)


def test_kv_cache_append_f32_nearest_matches_ieee(gpu):
    rng = np.random.default_rng(5)
    hkv, d, max_seq, new = 4, 128, 64, 33
    nk = _interesting_floats(rng, (new, hkv, d))
    nk = np.where(np.isnan(nk), np.float32(1.0), nk)
    ck = np.zeros((hkv, max_seq, d), np.uint16)
    dck, dcv, dnk = dev(ck), dev(ck), dev(nk)
    gpu.kv_cache_append_ex(dck, dcv, dnk, dnk, F32, hkv * d, d, hkv, d, 0, new, max_seq, ROUND_NEAREST)
    gpu.sync()
    with np.errstate(over="ignore"):
        want = np.transpose(nk, (1, 0, 2)).astype(np.float16).view(np.uint16)
    assert np.array_equal(dck.read(np.uint16, ck.shape)[:, :new], want)


def test_kv_cache_append_f16_is_per_head_memcpy(gpu, oracle):
    """KVCache::append layout: source [Hkv, new, D] halves."""
    rng = np.random.default_rng(6)
    hkv, d, max_seq, cur, new = 8, 128, 256, 37, 90
    src_k = rng.integers(0, 65536, (hkv, new, d)).astype(np.uint16)
    src_v = rng.integers(0, 65536, (hkv, new, d)).astype(np.uint16)
    ck = np.full((hkv, max_seq, d), SENT, np.uint16)
    want_k, want_v = ck.copy(), ck.copy()
    oracle.lib.go_kv_cache_append_f16(want_k.reshape(-1), src_k.reshape(-1), hkv, d, cur, new, max_seq)
    oracle.lib.go_kv_cache_append_f16(want_v.reshape(-1), src_v.reshape(-1), hkv, d, cur, new, max_seq)
    dck, dcv = dev(ck), dev(ck)
    gpu.kv_cache_append_ex(dck, dcv, dev(src_k), dev(src_v), F16, d, new * d, hkv, d, cur, new, max_seq)
    gpu.sync()
    assert np.array_equal(dck.read(np.uint16, ck.shape), want_k)
    assert np.array_equal(dcv.read(np.uint16, ck.shape), want_v)


def test_kv_cache_append_overflow(gpu):
    ck = dev(np.zeros((1, 4, 128), np.uint16))
    src = dev(np.zeros((2, 1, 128), np.float32))
    with pytest.raises(GraniteHipError) as e:
        gpu.kv_cache_append(ck, ck, src, src, 1, 128, 3, 2, 4)
    assert e.value.code == _capi.EOVERFLOW
    gpu.kv_cache_append(ck, ck, src, src, 1, 128, 2, 2, 4)
    gpu.kv_cache_append(ck, ck, src, src, 1, 128, 4, 0, 4)   # empty append is a no-op
    gpu.sync()


def test_kv_cache_append_unaligned_falls_to_scalar_path(gpu, oracle):
    rng = np.random.default_rng(7)
    hkv, d, max_seq, new = 2, 20, 16, 5          # head_dim not a multiple of 8
    nk = (rng.standard_normal((new, hkv, d)) * 3).astype(np.float32)
    ck = np.full((hkv, max_seq, d), SENT, np.uint16)
    want = ck.copy()
    oracle.lib.go_kv_cache_append_f32(want.reshape(-1), nk.reshape(-1), hkv, d, 2, new, max_seq)
    dck, dcv = dev(ck), dev(ck)
    gpu.kv_cache_append(dck, dcv, dev(nk), dev(nk), hkv, d, 2, new, max_seq)
    gpu.sync()
    assert np.array_equal(dck.read(np.uint16, ck.shape), want)


@pytest.mark.parametrize("hkv,d,bs,start,new,pool_blocks", [(8, 128, 16, 0, 1, 8), (8, 128, 16, 250, 70, 40),
                                                            (8, 128, 32, 32768, 512, 1100),
                                                            (2, 64, 5, 3, 19, 9), (8, 128, 16, 15, 2, 4)])
def test_paged_kv_cache_append_f32(gpu, oracle, hkv, d, bs, start, new, pool_blocks):
    say(f"paged_kv_cache_append hkv={hkv} d={d} bs={bs} start={start} new={new}")
    rng = np.random.default_rng(start + new)
    nblk = (start + new + bs - 1) // bs
    assert nblk <= pool_blocks
    table = rng.permutation(pool_blocks)[:nblk].astype(np.int32)
    nk, nv = _interesting_floats(rng, (hkv, new, d)), _interesting_floats(rng, (hkv, new, d))
    pk = np.full((pool_blocks * bs, hkv, d), SENT, np.uint16)
    pv = np.full((pool_blocks * bs, hkv, d), SENT + 1, np.uint16)
    want_k, want_v = pk.copy(), pv.copy()
    oracle.lib.go_paged_kv_cache_append_f32(want_k.reshape(-1), nk.reshape(-1), table, hkv, d, start, new, bs)
    oracle.lib.go_paged_kv_cache_append_f32(want_v.reshape(-1), nv.reshape(-1), table, hkv, d, start, new, bs)
    dpk, dpv = dev(pk), dev(pv)
    gpu.paged_kv_cache_append(dev(nk), dev(nv), dpk, dpv, dev(table), hkv, d, start, new, bs)
    gpu.sync()
    assert np.array_equal(dpk.read(np.uint16, pk.shape), want_k)
    assert np.array_equal(dpv.read(np.uint16, pv.shape), want_v)


def test_paged_append_f16_then_gather_round_trip(gpu, oracle):
    """append (half source, token-major) -> gather gives the source back bit
    for bit and equals the oracle's gather; untouched pool rows keep their
    sentinel."""
    rng = np.random.default_rng(8)
    hkv, d, bs, total, pool_blocks, max_seq = 8, 128, 16, 1000, 100, 1024
    nblk = (total + bs - 1) // bs
    table = rng.permutation(pool_blocks)[:nblk].astype(np.int32)
    src_k = rng.integers(0, 65536, (total, hkv, d)).astype(np.uint16)   # [tok, Hkv, D]
    src_v = rng.integers(0, 65536, (total, hkv, d)).astype(np.uint16)
    pk = np.full((pool_blocks * bs, hkv, d), SENT, np.uint16)
    dpk, dpv, dt = dev(pk), dev(pk), dev(table)
    # a table declared one block too short is refused before anything is written
    with pytest.raises(GraniteHipError) as e:
        gpu.paged_kv_cache_append_ex(dev(src_k), dev(src_v), F16, hkv * d, d, dpk, dpv, dt, hkv, d, 0, total, bs,
                                     max_blocks=nblk - 1)
    assert e.value.code == _capi.EOVERFLOW
    gpu.sync()
    assert np.all(dpk.read(np.uint16, pk.shape) == SENT)
    gpu.paged_kv_cache_append_ex(dev(src_k), dev(src_v), F16, hkv * d, d, dpk, dpv, dt, hkv, d, 0, total, bs,
                                 max_blocks=nblk)
    want_pool = pk.copy()
    oracle.lib.go_paged_kv_cache_append_f16(want_pool.reshape(-1), src_k.reshape(-1), table, hkv, d, 0,
                                            total, bs, hkv * d, d)
    gpu.sync()
    assert np.array_equal(dpk.read(np.uint16, pk.shape), want_pool)
    gk, gv = dev(np.zeros((hkv, max_seq, d), np.uint16)), dev(np.zeros((hkv, max_seq, d), np.uint16))
    gpu.paged_kv_gather(gk, gv, dpk, dpv, dt, hkv, d, total, bs, max_seq)
    gpu.sync()
    got_k = gk.read(np.uint16, (hkv, max_seq, d))
    got_v = gv.read(np.uint16, (hkv, max_seq, d))
    assert np.array_equal(got_k[:, :total], np.transpose(src_k, (1, 0, 2)))
    assert np.array_equal(got_v[:, :total], np.transpose(src_v, (1, 0, 2)))
    assert np.all(got_k[:, total:] == 0)
    want = np.zeros((hkv, max_seq, d), np.uint16)
    oracle.lib.go_paged_gather_f16(want.reshape(-1), want_pool.reshape(-1), table, hkv, d, total, bs, max_seq)
    assert np.array_equal(got_k, want)


def test_paged_with_identity_table_equals_contiguous(gpu):
    rng = np.random.default_rng(9)
    hkv, d, bs, new = 4, 128, 16, 48
    src = (rng.standard_normal((new, hkv, d)) * 2).astype(np.float32)
    table = np.arange(3, dtype=np.int32)
    dpk, dpv = dev(np.zeros((new, hkv, d), np.uint16)), dev(np.zeros((new, hkv, d), np.uint16))
    gpu.paged_kv_cache_append_ex(dev(src), dev(src), F32, hkv * d, d, dpk, dpv, dev(table), hkv, d, 0, new, bs,
                                 ROUND_TRUNCATE)
    dck, dcv = dev(np.zeros((hkv, new, d), np.uint16)), dev(np.zeros((hkv, new, d), np.uint16))
    gpu.kv_cache_append(dck, dcv, dev(src), dev(src), hkv, d, 0, new, new)
    gpu.sync()
    pool = dpk.read(np.uint16, (new, hkv, d))
    cache = dck.read(np.uint16, (hkv, new, d))
    assert np.array_equal(np.transpose(pool, (1, 0, 2)), cache)


def test_null_and_bad_arguments(gpu):
    buf = dev(np.zeros(1024, np.uint16))
    with pytest.raises(GraniteHipError) as e:
        gpu.kv_cache_append(None, buf, buf, buf, 1, 128, 0, 1, 4)
    assert e.value.code == _capi.ENULL
    with pytest.raises(GraniteHipError) as e:
        gpu.paged_kv_cache_append(buf, buf, buf, buf, None, 1, 128, 0, 1, 16)
    assert e.value.code == _capi.ENULL
    with pytest.raises(GraniteHipError) as e:
        gpu.paged_kv_cache_append(buf, buf, buf, buf, buf, 1, 128, 0, 1, 0)
    assert e.value.code == _capi.EINVAL


@pytest.mark.parametrize("paged", [False, True])
@pytest.mark.parametrize("src_dtype", [F16, F32])
def test_kv_commit_accepted_path(gpu, oracle, paged, src_dtype):
    """Commit of a speculation tree's accepted path: cache rows start_pos.. receive the accepted
    nodes' K/V in path order.  The reference leaves this step unwritten (its runner only
    truncates, src/llm/speculative_runner.cpp:871-882), so the semantics are this build's:
    the expected cache is the oracle's append of the gathered rows."""
    hkv, d, n_nodes, bs, start = 4, 128, 64, 16, 45
    say(f"kv commit accepted paged={paged} src_dtype={src_dtype}")
    rng = np.random.default_rng(91)
    accepted = np.array([0, 3, 9, 10, 41, 63], np.int32)
    tree_f32_k = (rng.standard_normal((hkv, n_nodes, d)) * 2).astype(np.float32)
    tree_f32_v = (rng.standard_normal((hkv, n_nodes, d)) * 2).astype(np.float32)
    if src_dtype == F16:
        tk, tv = tree_f32_k.astype(np.float16).view(np.uint16), tree_f32_v.astype(np.float16).view(np.uint16)
        rows_k, rows_v = tk[:, accepted], tv[:, accepted]                  # bit copy
    else:
        tk, tv = tree_f32_k, tree_f32_v
        rows_k, rows_v = oracle.fp32_to_fp16(tk[:, accepted]), oracle.fp32_to_fp16(tv[:, accepted])
    n = len(accepted)
    if paged:
        nblk = (start + n + bs - 1) // bs + 3
        table = rng.permutation(nblk).astype(np.int32)
        ck = np.full((nblk * bs, hkv, d), SENT, np.uint16)
        cv = np.full((nblk * bs, hkv, d), SENT + 1, np.uint16)
        want_k, want_v = ck.copy(), cv.copy()
        for i in range(n):
            pos = start + i
            row = table[pos // bs] * bs + pos % bs
            want_k[row], want_v[row] = rows_k[:, i], rows_v[:, i]
        extra = dict(block_table=dev(table), block_size=bs)
    else:
        max_seq = 64
        ck = np.full((hkv, max_seq, d), SENT, np.uint16)
        cv = np.full((hkv, max_seq, d), SENT + 1, np.uint16)
        want_k, want_v = ck.copy(), cv.copy()
        want_k[:, start:start + n], want_v[:, start:start + n] = rows_k, rows_v
        extra = dict(max_seq_len=max_seq)
    dck, dcv, dtk, dtv, dacc = dev(ck), dev(cv), dev(tk), dev(tv), dev(accepted)
    gpu.kv_commit_accepted(dtk, dtv, src_dtype, d, n_nodes * d, n_nodes, dacc, n, dck, dcv, hkv, d, start, **extra)
    gpu.sync()
    assert np.array_equal(dck.read(np.uint16, ck.shape), want_k)
    assert np.array_equal(dcv.read(np.uint16, cv.shape), want_v)
    # a node index outside the tree leaves its row unwritten; an empty path does nothing
    bad = dev(np.array([1, -1, 64, 2], np.int32))
    dck2, dcv2 = dev(ck), dev(cv)
    gpu.kv_commit_accepted(dtk, dtv, src_dtype, d, n_nodes * d, n_nodes, bad, 4, dck2, dcv2, hkv, d, start, **extra)
    gpu.kv_commit_accepted(dtk, dtv, src_dtype, d, n_nodes * d, n_nodes, bad, 0, dck2, dcv2, hkv, d, start, **extra)
    gpu.sync()
    got = dck2.read(np.uint16, ck.shape)
    changed = (got != ck).any(axis=-1)
    assert int(changed.sum()) == 2 * hkv   # only the two valid nodes' rows, one per head
    if not paged:
        with pytest.raises(GraniteHipError) as e:
            gpu.kv_commit_accepted(dtk, dtv, src_dtype, d, n_nodes * d, n_nodes, dacc, n, dck, dcv, hkv, d, 60, **extra)
        assert e.value.code == _capi.EOVERFLOW


def test_calibration_library_runs_and_checks_arguments(gpu):
    """The matrix-core rate kernel (libgranite_hip_calibration.so, a measurement aid beside
    the attention library): finishes, reports its flops and its time, and refuses what its
    launches do not cover."""
    import ctypes as C
    from granite_amd import calibration
    say("calibration library")
    n = 16384
    buf = dev(np.ones(n, np.float16))
    units = gpu.device_info().compute_units
    for shape, waves, mix in ((32, 2, (0, 0, 0)), (16, 2, (0, 0, 0)), (32, 1, (3, 1, 1)), (32, 2, (3, 1, 1))):
        flops, ms = calibration.mfma_rate(buf, n, 10, shape=shape, waves_per_simd=waves, mix=mix)
        assert flops == units * 4 * waves * 10 * 16 * 2 * 32 * 32 * 16 and ms > 0
    for kwargs in (dict(n_halves=12), dict(iterations=0), dict(shape=8), dict(waves_per_simd=3),
                   dict(mix=(5, 0, 0)), dict(shape=16, mix=(3, 1, 1))):
        args = dict(n_halves=n, iterations=10, shape=32, waves_per_simd=2, mix=(0, 0, 0))
        args.update(kwargs)
        with pytest.raises(RuntimeError):
            calibration.mfma_rate(buf, args["n_halves"], args["iterations"], shape=args["shape"],
                                  waves_per_simd=args["waves_per_simd"], mix=args["mix"])


@pytest.mark.parametrize("rows,d,dp,esz", [(1, 4, 64, 4), (37, 80, 128, 2), (300, 24, 64, 2), (5, 100, 128, 4)])
def test_copy_rows_pads_and_slices(gpu, rows, d, dp, esz):
    """granite_hip_copy_rows: pad [rows, d] to [rows, dp] with zeros, slice it back; bit exact,
    nothing written beyond the rows' fill range."""
    say(f"copy_rows rows={rows} d={d} dp={dp} esz={esz}")
    dt = np.uint16 if esz == 2 else np.uint32
    rng = np.random.default_rng(rows + d)
    src = rng.integers(1, np.iinfo(dt).max, size=(rows, d), dtype=dt)
    padded = dev(np.full((rows, dp), 0x5A5A, dt))
    gpu.copy_rows(padded, dp * esz, dev(src), d * esz, rows, d * esz, dp * esz)
    gpu.sync()
    got = padded.read(dt, (rows, dp))
    assert np.array_equal(got[:, :d], src) and not got[:, d:].any()
    back = dev(np.full((rows, d + 2), 0x77, dt))   # a destination with a wider pitch than the copy
    gpu.copy_rows(back, (d + 2) * esz, padded, dp * esz, rows, d * esz, d * esz)
    gpu.sync()
    got = back.read(dt, (rows, d + 2))
    assert np.array_equal(got[:, :d], src) and (got[:, d:] == 0x77).all()
    with pytest.raises(GraniteHipError):
        gpu.copy_rows(back, d * esz, padded, dp * esz, rows, dp * esz, d * esz)   # copy > fill
