"""GPU parity of the projections on Q4_K weights (MetalCompute::fused_qkv_matvec_q4k and
matvec_q4k, include/granite/metal_compute.h:683-694, 73-79) against the oracle's
dequantise-and-multiply (src/model/gguf.cpp:952-1020).

Tolerance.  Both sides sum K products in float, in different orders (the kernel also
applies the minima to sums of inputs, as the reference kernel does), so a result may differ
from the exact value by a few K * 2^-24 of sum |x_k w_k|; the bound asserted is
8 * 2^-24 * sqrt(K) * sum |x_k w_k| + 1e-6 against the oracle.  The reference's CPU path
multiplies by weights it truncated to half at load time; the distance to that path is
asserted too, at the size of that truncation (2^-10 of sum |x_k w_k|)."""
import numpy as np
import pytest

from granite_amd import GraniteHipError, _capi
from granite_amd import workloads as W
from gpu_util import dev, say

pytestmark = pytest.mark.gpu


def _abs_dot(oracle, x, blocks):
    w32, _ = oracle.q4k_dequantize(blocks)
    w = np.abs(w32.astype(np.float64)).reshape(blocks.shape[0], -1)
    return np.abs(x).astype(np.float64) @ w.T


def _check(oracle, got, x, blocks, what):
    want = oracle.matvec_q4k(x, blocks)
    mag = _abs_dot(oracle, x, blocks)
    K = x.shape[1]
    bound = 8 * 2.0 ** -24 * np.sqrt(K) * mag + 1e-6
    err = np.abs(got.astype(np.float64) - want)
    assert np.isfinite(got).all() and np.all(err <= bound), \
        f"{what}: max err {err.max():.3e}, worst ratio to bound {np.max(err / bound):.2f}"
    # and the CPU path: the same product with the weights it stored as half
    _, w16 = oracle.q4k_dequantize(blocks)
    cpu = oracle.matmul_transb_fp16(x, w16.reshape(blocks.shape[0], K))
    assert np.all(np.abs(got - cpu) <= 2.0 ** -10 * mag + 2 * bound), f"{what}: off the CPU path"
    return float(err.max())


@pytest.mark.parametrize("K,heads,kv_heads,head_dim,batch", [(256, 1, 1, 8, 1), (512, 3, 1, 24, 1),
                                                            (2304, 4, 2, 64, 1), (4096, 32, 8, 128, 1),
                                                            (1024, 5, 1, 64, 2), (2048, 8, 2, 128, 3),
                                                            (1024, 4, 4, 32, 4), (768, 2, 1, 40, 7),
                                                            # batches of tokens: the matrix-core kernel
                                                            (256, 1, 1, 8, 5), (4096, 32, 8, 128, 64),
                                                            (1280, 3, 1, 88, 33), (2048, 8, 2, 128, 32), (512, 2, 2, 16, 300),
                                                            # workgroups of two token tiles: ragged second tile, ragged
                                                            # last workgroup, K not a multiple of the staged chunk
                                                            (768, 2, 1, 40, 65), (1280, 3, 1, 88, 97), (2304, 4, 2, 64, 129),
                                                            # rows longer than one staged slice of the inputs (4096
                                                            # columns with one vector, 2048 with two): several trips,
                                                            # the last one ragged
                                                            (8448, 2, 1, 32, 1), (4352, 2, 1, 32, 2), (14336, 1, 1, 64, 1),
                                                            (6144, 3, 3, 16, 2)])
def test_fused_qkv_matvec_q4k(gpu, oracle, K, heads, kv_heads, head_dim, batch):
    say(f"fused qkv q4k K={K} heads={heads} kv_heads={kv_heads} head_dim={head_dim} batch={batch}")
    case = W.make_qkv_projection(seed=K + heads + batch, K=K, num_heads=heads, num_kv_heads=kv_heads,
                                 head_dim=head_dim, batch=batch)
    yq = dev(np.full((batch, case.Nq), np.nan, np.float32))
    yk = dev(np.full((batch, case.Nkv), np.nan, np.float32))
    yv = dev(np.full((batch, case.Nkv), np.nan, np.float32))
    gpu.fused_qkv_matvec_q4k(dev(case.x), dev(case.wq), dev(case.wk), dev(case.wv), yq, yk, yv, K, case.Nq,
                             case.Nkv, batch=batch)
    gpu.sync()
    _check(oracle, yq.read(np.float32, (batch, case.Nq)), case.x, case.wq, "yq")
    _check(oracle, yk.read(np.float32, (batch, case.Nkv)), case.x, case.wk, "yk")
    _check(oracle, yv.read(np.float32, (batch, case.Nkv)), case.x, case.wv, "yv")


@pytest.mark.parametrize("trial", range(12))
def test_random_projection_shapes(gpu, oracle, trial):
    """Seeded random shapes across both kernels: K any multiple of 256 up to 9216, row counts
    that are not multiples of a wave's or a workgroup's rows, 1 to 140 tokens."""
    rng = np.random.default_rng(9100 + trial)
    K = 256 * int(rng.integers(1, 37))
    head_dim = int(rng.choice([8, 24, 40, 64, 88, 128]))
    kv_heads = int(rng.integers(1, 4))
    heads = kv_heads * int(rng.integers(1, 4))
    batch = int(rng.choice([1, 2, int(rng.integers(3, 33)), int(rng.integers(33, 65)), int(rng.integers(65, 141))]))
    say(f"q4k random trial={trial} K={K} heads={heads} kv_heads={kv_heads} head_dim={head_dim} batch={batch}")
    case = W.make_qkv_projection(seed=9200 + trial, K=K, num_heads=heads, num_kv_heads=kv_heads,
                                 head_dim=head_dim, batch=batch)
    yq = dev(np.full((batch, case.Nq), np.nan, np.float32))
    yk = dev(np.full((batch, case.Nkv), np.nan, np.float32))
    yv = dev(np.full((batch, case.Nkv), np.nan, np.float32))
    gpu.fused_qkv_matvec_q4k(dev(case.x), dev(case.wq), dev(case.wk), dev(case.wv), yq, yk, yv, case.K, case.Nq,
                             case.Nkv, batch=batch)
    gpu.sync()
    _check(oracle, yq.read(np.float32, (batch, case.Nq)), case.x, case.wq, "yq")
    _check(oracle, yk.read(np.float32, (batch, case.Nkv)), case.x, case.wk, "yk")
    _check(oracle, yv.read(np.float32, (batch, case.Nkv)), case.x, case.wv, "yv")


def test_matvec_q4k_output_projection(gpu, oracle):
    """y = Wo x with K = num_heads * head_dim: MetalCompute::matvec_q4k behind attention."""
    rng = np.random.default_rng(3)
    K, N = 4096, 1000   # a row count that is no multiple of the rows a workgroup takes
    x = rng.standard_normal((1, K), dtype=np.float32)
    w = W.random_q4k(rng, N, K)
    y = dev(np.full((1, N), np.nan, np.float32))
    gpu.matvec_q4k(dev(x), dev(w), y, K, N)
    gpu.sync()
    _check(oracle, y.read(np.float32, (1, N)), x, w, "y")
    x5 = rng.standard_normal((5, K), dtype=np.float32)
    y5 = dev(np.full((5, N), np.nan, np.float32))
    gpu.matvec_q4k(dev(x5), dev(w), y5, K, N, batch=5)
    gpu.sync()
    _check(oracle, y5.read(np.float32, (5, N)), x5, w, "y batch 5")


def test_known_blocks(gpu):
    """Hand-built blocks with closed-form results: d = 1, scales 1, no minimum -> the weights
    are the nibbles; x = 1 -> y = sum of the nibbles; then the minimum alone."""
    K = 512
    q = (np.arange(2 * K) * 7 % 16).reshape(4, 256)          # 2 rows x 2 blocks
    ones, zeros = np.ones(4, np.float16), np.zeros(4, np.float16)
    w = W.pack_q4k(ones, zeros, np.ones((4, 8)), np.zeros((4, 8)), q).reshape(2, 2, 144)
    x = np.ones((1, K), np.float32)
    y = dev(np.zeros((1, 2), np.float32))
    gpu.matvec_q4k(dev(x), dev(w), y, K, 2)
    gpu.sync()
    assert np.array_equal(y.read(np.float32, (1, 2))[0], q.reshape(2, 512).sum(axis=1).astype(np.float32))
    mins = np.arange(32).reshape(4, 8) % 64
    w = W.pack_q4k(zeros, np.full(4, 0.5, np.float16), np.ones((4, 8)), mins, q).reshape(2, 2, 144)
    gpu.matvec_q4k(dev(x), dev(w), y, K, 2)
    gpu.sync()
    want = -(0.5 * 32 * mins.reshape(2, 16).sum(axis=1)).astype(np.float32)
    assert np.array_equal(y.read(np.float32, (1, 2))[0], want)


def test_rejects_bad_arguments(gpu):
    buf = dev(np.zeros(1 << 14, np.float32))
    lib = _capi.load()
    assert lib.granite_hip_matvec_q4k(buf.ptr, buf.ptr, buf.ptr, 300, 4) == _capi.EINVAL   # K % 256
    assert lib.granite_hip_matvec_q4k(None, buf.ptr, buf.ptr, 256, 4) == _capi.ENULL
    assert lib.granite_hip_matvec_q4k(buf.ptr, None, buf.ptr, 256, 4) == _capi.ENULL
    assert lib.granite_hip_matvec_q4k(buf.ptr + 4, buf.ptr, buf.ptr, 256, 4) == _capi.EINVAL  # alignment
    assert lib.granite_hip_matvec_q4k(buf.ptr, buf.ptr, buf.ptr, 256, 0) == _capi.OK
    gpu.sync()


def test_batched_projection_scratch_can_be_reserved(gpu, oracle):
    """The matrix-core path keeps its chunk sums in library scratch: the stated requirement,
    reserved once, is enough (no growth during the call)."""
    lib = _capi.load()
    case = W.make_qkv_projection(seed=77, K=1024, num_heads=4, num_kv_heads=2, head_dim=64, batch=40)
    rows = case.Nq + 2 * case.Nkv
    assert lib.granite_hip_q4k_workspace_required(case.K, rows, 2) == 0
    need = lib.granite_hip_q4k_workspace_required(case.K, rows, 40)
    assert need == 2 * 64 * rows * 4        # two chunks of K, two tiles of 32 tokens
    gpu.reserve_workspace(need)
    held = gpu.workspace_bytes()
    yq, yk, yv = (dev(np.zeros((40, n), np.float32)) for n in (case.Nq, case.Nkv, case.Nkv))
    gpu.fused_qkv_matvec_q4k(dev(case.x), dev(case.wq), dev(case.wk), dev(case.wv), yq, yk, yv, case.K, case.Nq,
                             case.Nkv, batch=40)
    gpu.sync()
    assert gpu.workspace_bytes() == held
    _check(oracle, yq.read(np.float32, (40, case.Nq)), case.x, case.wq, "yq")


@pytest.mark.parametrize("batch", [1, 2, 3, 64, 256])
def test_scale_fields_known_answer_on_gpu(gpu, batch):
    """The hand-worked super-block of tests/golden/q4k_scales_kat.json through the kernels: with
    one-hot inputs every output is one weight, and every weight of the block is a multiple of
    0.25 below 2^11, so the results must be exact -- in the vector kernel (batch <= 2) and in
    the matrix-core kernel (batch > 2), for all eight (scale, minimum) pairs."""
    from test_oracle_q4k import kat_block
    say(f"q4k scale-field known answer batch={batch}")
    block, want = kat_block()
    rows = 4
    w = np.ascontiguousarray(np.tile(block[None, None], (rows, 1, 1)))        # [rows, 1, 144]
    picks = (np.arange(batch) * 37 + 5) % 256 if batch < 256 else np.arange(256)
    x = np.zeros((batch, 256), np.float32)
    x[np.arange(batch), picks] = 1.0
    y = dev(np.full((batch, rows), np.nan, np.float32))
    gpu.matvec_q4k(dev(x), dev(w), y, 256, rows, batch=batch)
    gpu.sync()
    got = y.read(np.float32, (batch, rows))
    assert np.array_equal(got, np.repeat(want[picks].astype(np.float32)[:, None], rows, axis=1))


@pytest.mark.parametrize("magnitudes", ["large", "tiny", "mixed"])
@pytest.mark.parametrize("batch", [3, 40])
def test_batched_projection_input_magnitudes(gpu, oracle, magnitudes, batch):
    """The matrix-core kernel (batch > 2) on inputs far outside the half range on either side:
    thousands (a sub-block's sum of 32 exceeds 65504), millionths (below the smallest normal
    half), and both in one batch and one row.  The bound has no absolute floor: it scales
    with sum |x w|, as a float summation's does."""
    say(f"q4k batched magnitudes={magnitudes} batch={batch}")
    K, rows = 1024, 96
    rng = np.random.default_rng({"large": 11, "tiny": 22, "mixed": 33}[magnitudes] + batch)
    blocks = W.random_q4k(rng, rows, K)
    x = rng.standard_normal((batch, K), dtype=np.float32)
    if magnitudes == "large":
        x = x * 3000.0 + 2500.0            # sub-block sums around 80000
    elif magnitudes == "tiny":
        x = x * 1e-6
    else:
        x[0::2] *= 1e-6                    # every other token tiny ...
        x[1::2] *= 3000.0                  # ... the rest large,
        x[:, K // 2:] *= 1e-3              # and the second chunk of K a thousand times smaller than the first
    x = np.ascontiguousarray(x.astype(np.float32))
    y = dev(np.full((batch, rows), np.nan, np.float32))
    gpu.matvec_q4k(dev(x), dev(blocks), y, K, rows, batch=batch)
    gpu.sync()
    got = y.read(np.float32, (batch, rows))
    want = oracle.matvec_q4k(x, blocks)
    mag = _abs_dot(oracle, x, blocks)
    bound = 8 * 2.0 ** -24 * np.sqrt(K) * mag
    err = np.abs(got.astype(np.float64) - want)
    assert np.isfinite(got).all() and np.all(err <= bound), \
        f"max err {err.max():.3e}, worst ratio to bound {np.max(err / np.maximum(bound, 1e-300)):.2f}"
