"""GPU parity: decode attention (contiguous and paged, single and batched)
against the oracle's restatement of src/llm/transformer.mm:1779-1840.
Tolerances: outputs |d| <= 2e-3 or <= 1e-2 |ref|; log-sum-exp 1e-4 absolute."""
import numpy as np
import pytest

from granite_amd import F16, F32, DeviceBuffer, GraniteHipError, _capi
from granite_amd import workloads as W
from gpu_util import assert_close, assert_lse, dev, say
import ref64

pytestmark = pytest.mark.gpu


def test_decode_contiguous_config(gpu, oracle):
    """batch 1, 32 q heads, 8 KV heads, D=128, 512 cached tokens, Q fp32."""
    case = W.make_decode_contiguous()
    say("decode contiguous ctx=512")
    want, want_lse = oracle.attention_cached(case.q[None, None], case.k_cache, case.v_cache, case.seq_kv,
                                             case.seq_kv - 1, case.scale)
    out, lse = dev(np.zeros((32, 128), np.float32)), dev(np.zeros(32, np.float32))
    dq, dk, dv = dev(case.q), dev(case.k_cache), dev(case.v_cache)
    gpu.decode_attention(q=dq, q_dtype=F32, k_cache=dk, v_cache=dv, out=out, lse=lse, batch_size=1,
                         num_heads=32, num_kv_heads=8, head_dim=128, scale=case.scale, max_seq=case.max_seq,
                         fixed_seq_len=case.seq_kv)
    gpu.sync()
    assert_close(out.read(np.float32, (32, 128)), want[0, 0], "decode out")
    assert_lse(lse.read(np.float32, (32,)), want_lse[0, :, 0], "decode lse")
    # the reference-shaped entry point gives the same bits
    out2 = dev(np.zeros((32, 128), np.float32))
    gpu.multihead_attention(dq, dk, dv, out2, 32, 8, 1, case.seq_kv, 128, case.scale, case.max_seq)
    gpu.sync()
    assert np.array_equal(out2.read(np.float32, (32, 128)), out.read(np.float32, (32, 128)))


@pytest.mark.parametrize("seq_kv,max_seq,hq,hkv", [(1, 64, 8, 8), (31, 64, 8, 2), (33, 64, 32, 8),
                                                   (257, 300, 4, 1), (1000, 1000, 64, 8), (700, 4096, 40, 2)])
def test_decode_contiguous_shapes(gpu, oracle, seq_kv, max_seq, hq, hkv):
    say(f"decode contiguous seq_kv={seq_kv} max_seq={max_seq} hq={hq} hkv={hkv}")
    case = W.make_decode_contiguous(seed=seq_kv, num_heads=hq, num_kv_heads=hkv, seq_kv=seq_kv, max_seq=max_seq)
    want, want_lse = oracle.attention_cached(case.q[None, None], case.k_cache, case.v_cache, seq_kv, seq_kv - 1,
                                             case.scale)
    out, lse = dev(np.zeros((hq, 128), np.float32)), dev(np.zeros(hq, np.float32))
    gpu.decode_attention(q=dev(case.q), q_dtype=F32, k_cache=dev(case.k_cache), v_cache=dev(case.v_cache),
                         out=out, lse=lse, batch_size=1, num_heads=hq, num_kv_heads=hkv, head_dim=128,
                         scale=case.scale, max_seq=max_seq, fixed_seq_len=seq_kv)
    gpu.sync()
    assert_close(out.read(np.float32, (hq, 128)), want[0, 0], "out")
    assert_lse(lse.read(np.float32, (hq,)), want_lse[0, :, 0], "lse")


def _run_batched(gpu, case, q_dtype, chunk_tokens=0, with_lse=True):
    B, hq = case.batch, case.num_heads
    q_host = case.q if q_dtype == F16 else case.q.astype(np.float32)
    out = dev(np.full((B, hq, 128), -7.0, np.float32))
    lse = dev(np.full((B, hq), -7.0, np.float32)) if with_lse else None
    bufs = (dev(q_host), dev(case.k_pool), dev(case.v_pool), dev(case.block_tables), dev(case.seq_lens))
    gpu.decode_attention(q=bufs[0], q_dtype=q_dtype, k_cache=bufs[1], v_cache=bufs[2], block_tables=bufs[3],
                         seq_lens=bufs[4], out=out, lse=lse, batch_size=B, num_heads=hq,
                         num_kv_heads=case.num_kv_heads, head_dim=128, scale=case.scale,
                         block_size=case.block_size, max_blocks_per_seq=case.max_blocks,
                         chunk_tokens=chunk_tokens)
    gpu.sync()
    return out.read(np.float32, (B, hq, 128)), (lse.read(np.float32, (B, hq)) if with_lse else None)


@pytest.mark.parametrize("q_dtype", [F16, F32])
@pytest.mark.parametrize("bs", [16, 32, 1, 12])
def test_batched_paged_decode_small(gpu, oracle, q_dtype, bs):
    lens = np.array([1, 17, 64, 0, 255, 256, 257, 700, 33, 5], np.int32)
    case = W.make_paged_decode(seed=bs, block_size=bs, ctx_max=768, seq_lens=lens)
    say(f"batched paged decode small bs={bs} q_dtype={q_dtype}")
    want, want_lse = oracle.batched_paged_decode(case.q.astype(np.float32), case.k_pool, case.v_pool,
                                                 case.block_tables, case.seq_lens, bs, case.scale)
    got, got_lse = _run_batched(gpu, case, q_dtype)
    live = lens > 0
    assert_close(got[live], want[live], "out")
    assert_lse(got_lse[live], want_lse[live], "lse")
    assert np.all(got[~live] == -7.0) and np.all(got_lse[~live] == -7.0)   # empty sequence untouched


@pytest.mark.parametrize("hq,hkv", [(12, 3), (64, 16), (40, 2), (160, 8), (8, 8), (6, 1)])
def test_batched_paged_decode_head_shapes(gpu, oracle, hq, hkv):
    """Head counts on both sides of the kernel's two list shapes (heads in groups of 8 or
    not), with more than 16 query heads per KV head among them."""
    lens = np.array([40, 1300, 0, 31, 513, 2100, 64, 9], np.int32)
    case = W.make_paged_decode(seed=hq, num_heads=hq, num_kv_heads=hkv, ctx_max=2112, seq_lens=lens)
    say(f"batched paged decode heads hq={hq} hkv={hkv}")
    want, want_lse = oracle.batched_paged_decode(case.q.astype(np.float32), case.k_pool, case.v_pool,
                                                 case.block_tables, case.seq_lens, 16, case.scale)
    got, got_lse = _run_batched(gpu, case, F16)
    live = lens > 0
    assert_close(got[live], want[live], "out")
    assert_lse(got_lse[live], want_lse[live], "lse")
    assert np.all(got[~live] == -7.0)


@pytest.mark.parametrize("trial", range(12))
def test_batched_paged_decode_random_shapes(gpu, oracle, trial):
    """Seeded random batches: head counts, group sizes, block sizes and length mixes (empty,
    single-token, tile edges, long) that move the workers' range boundaries around."""
    rng = np.random.default_rng(1000 + trial)
    hkv = int(rng.choice([8, 16, 4, 2, 1, 3]))
    hq = hkv * int(rng.choice([1, 2, 4, 8, 20]))
    B = int(rng.integers(1, 24))
    kind = trial % 4
    if kind == 0:
        lens = rng.integers(0, 200, B)
    elif kind == 1:
        lens = rng.integers(1, 2500, B)
    elif kind == 2:
        lens = np.where(rng.random(B) < 0.3, 0, rng.integers(1, 900, B))
    else:
        lens = rng.choice([1, 31, 32, 33, 63, 64, 65, 1024], B)
    lens = lens.astype(np.int32)
    lens[0] = max(lens[0], 3)
    bs = int(rng.choice([16, 32, 8, 12]))
    case = W.make_paged_decode(seed=trial, num_heads=hq, num_kv_heads=hkv, block_size=bs,
                               ctx_max=int(max(lens.max(), 64)), seq_lens=lens)
    say(f"batched paged decode random trial={trial} hq={hq} hkv={hkv} B={B} bs={bs} tokens={int(lens.sum())}")
    want, want_lse = oracle.batched_paged_decode(case.q.astype(np.float32), case.k_pool, case.v_pool,
                                                 case.block_tables, case.seq_lens, bs, case.scale)
    got, got_lse = _run_batched(gpu, case, F16 if trial % 3 else F32)
    live = lens > 0
    assert_close(got[live], want[live], "out")
    assert_lse(got_lse[live], want_lse[live], "lse")
    assert np.all(got[~live] == -7.0)


@pytest.mark.parametrize("chunk", [32, 128, 512, 1024])
def test_batched_paged_decode_chunk_sizes_agree(gpu, oracle, chunk):
    lens = np.array([900, 31, 1500, 1024], np.int32)
    case = W.make_paged_decode(seed=77, ctx_max=1536, seq_lens=lens)
    say(f"batched paged decode chunk={chunk}")
    want, want_lse = oracle.batched_paged_decode(case.q.astype(np.float32), case.k_pool, case.v_pool,
                                                 case.block_tables, case.seq_lens, 16, case.scale)
    got, got_lse = _run_batched(gpu, case, F16, chunk_tokens=chunk)
    assert_close(got, want, "out")
    assert_lse(got_lse, want_lse, "lse")


def test_batched_paged_decode_reference_entry_point(gpu, oracle):
    """MetalCompute::batched_paged_attention_decode shape: Q/out fp32, no lse."""
    lens = np.array([300, 0, 77, 513], np.int32)
    case = W.make_paged_decode(seed=5, ctx_max=640, seq_lens=lens)
    want, _ = oracle.batched_paged_decode(case.q.astype(np.float32), case.k_pool, case.v_pool,
                                          case.block_tables, case.seq_lens, 16, case.scale)
    out = dev(np.zeros((4, 32, 128), np.float32))
    gpu.batched_paged_attention_decode(dev(case.q.astype(np.float32)), dev(case.k_pool), dev(case.v_pool),
                                       dev(case.block_tables), dev(case.seq_lens), out, 4, 32, 8, 128, 16,
                                       case.max_blocks, case.scale)
    gpu.sync()
    got = out.read(np.float32, (4, 32, 128))
    assert_close(got[lens > 0], want[lens > 0], "out")
    assert np.all(got[1] == 0)
    # single-sequence entry point, sequence 3
    out1 = dev(np.zeros((32, 128), np.float32))
    gpu.paged_attention_decode(dev(case.q[3].astype(np.float32)), dev(case.k_pool), dev(case.v_pool),
                               dev(case.block_tables[3]), out1, 32, 8, int(lens[3]), 128, 16, case.scale)
    gpu.sync()
    assert_close(out1.read(np.float32, (32, 128)), want[3], "single")


def test_batched_paged_decode_full_config(gpu, oracle):
    """64 sequences, ctx ~ U[256, 8192], block 16, shuffled tables, Q fp16."""
    case = W.make_paged_decode()
    say(f"batched paged decode full: tokens={int(case.seq_lens.sum())} blocks={case.num_blocks}")
    want, want_lse = oracle.batched_paged_decode(case.q.astype(np.float32), case.k_pool, case.v_pool,
                                                 case.block_tables, case.seq_lens, 16, case.scale)
    got, got_lse = _run_batched(gpu, case, F16)
    err = assert_close(got, want, "out")
    lerr = assert_lse(got_lse, want_lse, "lse")
    say(f"  max abs err {err:.2e}, lse err {lerr:.2e}")


def test_paged_decode_equals_contiguous_decode(gpu):
    """Same tokens through a shuffled pool and through a contiguous cache."""
    rng = np.random.default_rng(3)
    hq, hkv, total, bs = 32, 8, 777, 16
    case = W.make_paged_decode(seed=9, ctx_max=1024, seq_lens=np.array([total], np.int32))
    kc = np.transpose(ref64.gather_paged(case.k_pool, case.block_tables[0], bs, total), (1, 0, 2)).copy()
    vc = np.transpose(ref64.gather_paged(case.v_pool, case.block_tables[0], bs, total), (1, 0, 2)).copy()
    got, got_lse = _run_batched(gpu, case, F16)
    out, lse = dev(np.zeros((hq, 128), np.float32)), dev(np.zeros(hq, np.float32))
    gpu.decode_attention(q=dev(case.q[0]), q_dtype=F16, k_cache=dev(kc), v_cache=dev(vc), out=out, lse=lse,
                         batch_size=1, num_heads=hq, num_kv_heads=hkv, head_dim=128, scale=case.scale,
                         max_seq=total, fixed_seq_len=total)
    gpu.sync()
    assert np.array_equal(out.read(np.float32, (hq, 128)), got[0])
    assert np.array_equal(lse.read(np.float32, (hq,)), got_lse[0])


def test_decode_rejects_bad_arguments(gpu):
    buf = dev(np.zeros(4096, np.float32))
    base = dict(q=buf, q_dtype=F32, k_cache=buf, v_cache=buf, out=buf, batch_size=1, num_heads=8,
                num_kv_heads=2, head_dim=128, scale=0.1, max_seq=16, fixed_seq_len=4)
    for bad, code in ((dict(head_dim=96), _capi.EUNSUPPORTED), (dict(num_kv_heads=3), _capi.EINVAL),
                      (dict(q=None), _capi.ENULL), (dict(fixed_seq_len=0), _capi.EINVAL),
                      (dict(fixed_seq_len=17), _capi.EINVAL), (dict(chunk_tokens=48), _capi.EINVAL),
                      (dict(q_dtype=7), _capi.EINVAL)):
        with pytest.raises(GraniteHipError) as e:
            gpu.decode_attention(**{**base, **bad})
        assert e.value.code == code, bad


# ---- head size 64 (the reference's d64 decode kernels, metal_shaders_attention.h:2769-2977, 3202-3422) ----

def _run_batched_d(gpu, case, q_dtype, D, chunk_tokens=0):
    B, hq = case.batch, case.num_heads
    q_host = case.q if q_dtype == F16 else case.q.astype(np.float32)
    out = dev(np.full((B, hq, D), -7.0, np.float32))
    lse = dev(np.full((B, hq), -7.0, np.float32))
    bufs = (dev(q_host), dev(case.k_pool), dev(case.v_pool), dev(case.block_tables), dev(case.seq_lens))
    gpu.decode_attention(q=bufs[0], q_dtype=q_dtype, k_cache=bufs[1], v_cache=bufs[2], block_tables=bufs[3],
                         seq_lens=bufs[4], out=out, lse=lse, batch_size=B, num_heads=hq,
                         num_kv_heads=case.num_kv_heads, head_dim=D, scale=case.scale,
                         block_size=case.block_size, max_blocks_per_seq=case.max_blocks, chunk_tokens=chunk_tokens)
    gpu.sync()
    return out.read(np.float32, (B, hq, D)), lse.read(np.float32, (B, hq))


@pytest.mark.parametrize("q_dtype", [F16, F32])
@pytest.mark.parametrize("hq,hkv,bs,ctx", [(32, 8, 16, 768), (12, 3, 12, 2112), (64, 16, 32, 2112), (40, 2, 16, 600),
                                           (8, 8, 16, 5000)])
def test_batched_paged_decode_head_dim_64(gpu, oracle, q_dtype, hq, hkv, bs, ctx):
    """Both kernels (one workgroup per short context, the persistent one for long ones) and
    both list shapes of the persistent kernel at head size 64."""
    lens = np.array([1, 17, 64, 0, 255, 256, 257, ctx, 33, ctx // 2 + 1], np.int32)
    case = W.make_paged_decode(seed=hq + bs, num_heads=hq, num_kv_heads=hkv, head_dim=64, block_size=bs,
                               ctx_max=ctx, seq_lens=lens)
    say(f"batched paged decode d64 hq={hq} hkv={hkv} bs={bs} ctx={ctx} q_dtype={q_dtype}")
    want, want_lse = oracle.batched_paged_decode(case.q.astype(np.float32), case.k_pool, case.v_pool,
                                                 case.block_tables, case.seq_lens, bs, case.scale)
    got, got_lse = _run_batched_d(gpu, case, q_dtype, 64)
    live = lens > 0
    assert_close(got[live], want[live], "out")
    assert_lse(got_lse[live], want_lse[live], "lse")
    assert np.all(got[~live] == -7.0) and np.all(got_lse[~live] == -7.0)
    if ctx > 768:   # the chunk kernel with its merge launch as well
        got, got_lse = _run_batched_d(gpu, case, q_dtype, 64, chunk_tokens=256)
        assert_close(got[live], want[live], "out (chunk kernel)")
        assert_lse(got_lse[live], want_lse[live], "lse (chunk kernel)")


@pytest.mark.parametrize("seq_kv,max_seq,hq,hkv", [(1, 64, 8, 8), (33, 64, 32, 8), (700, 4096, 40, 2), (3000, 3000, 16, 4)])
def test_decode_contiguous_head_dim_64(gpu, oracle, seq_kv, max_seq, hq, hkv):
    say(f"decode contiguous d64 seq_kv={seq_kv} max_seq={max_seq} hq={hq} hkv={hkv}")
    case = W.make_decode_contiguous(seed=seq_kv, num_heads=hq, num_kv_heads=hkv, head_dim=64, seq_kv=seq_kv,
                                    max_seq=max_seq)
    want, want_lse = oracle.attention_cached(case.q[None, None], case.k_cache, case.v_cache, seq_kv, seq_kv - 1,
                                             case.scale)
    out, lse = dev(np.zeros((hq, 64), np.float32)), dev(np.zeros(hq, np.float32))
    gpu.decode_attention(q=dev(case.q), q_dtype=F32, k_cache=dev(case.k_cache), v_cache=dev(case.v_cache),
                         out=out, lse=lse, batch_size=1, num_heads=hq, num_kv_heads=hkv, head_dim=64,
                         scale=case.scale, max_seq=max_seq, fixed_seq_len=seq_kv)
    gpu.sync()
    assert_close(out.read(np.float32, (hq, 64)), want[0, 0], "out")
    assert_lse(lse.read(np.float32, (hq,)), want_lse[0, :, 0], "lse")
