"""Pins the oracle's Q4_K dequantisation (src/model/gguf.cpp:952-1020) and projections
(src/llm/math_ops.cpp:67-103) without the GPU: the sizes the reference's own tests hold,
ggml's packing of the 6-bit fields run backwards, hand-built blocks with closed-form
values, an independent float64 dequantisation, and the reference's math_ops.cpp."""
import json
from pathlib import Path

import numpy as np
import pytest

import oracle_bind
from granite_amd import workloads as W

KAT = json.loads((Path(__file__).parent / "golden" / "q4k_scales_kat.json").read_text())


def kat_block():
    """The fixture's super-block (144 bytes) and its 256 weights by the fixture's own rule,
    from the hand-typed sc / m lists (not from any unpacking code)."""
    scale_bytes = np.array([int(h, 16) for h in KAT["scale_bytes_hex"]], np.uint8)
    qs = ((7 * np.arange(128) + 3) & 255).astype(np.uint8)
    block = np.zeros(144, np.uint8)
    block[0:2] = np.array([int(KAT["block"]["d_bits_hex"], 16)], np.uint16).view(np.uint8)
    block[2:4] = np.array([int(KAT["block"]["dmin_bits_hex"], 16)], np.uint16).view(np.uint8)
    block[4:16] = scale_bytes
    block[16:] = qs
    d, dmin, sc, m = KAT["block"]["d"], KAT["block"]["dmin"], KAT["sc"], KAT["m"]
    w = np.zeros(256, np.float64)
    for g in range(4):
        for l in range(32):
            w[64 * g + l] = d * sc[2 * g] * (int(qs[32 * g + l]) & 15) - dmin * m[2 * g]
            w[64 * g + 32 + l] = d * sc[2 * g + 1] * (int(qs[32 * g + l]) >> 4) - dmin * m[2 * g + 1]
    return block, w


def dequant64(blocks: np.ndarray) -> np.ndarray:
    """Vectorised float64 dequantisation of Q4_K super-blocks [nb, 144] -> [nb, 256]."""
    nb = blocks.shape[0]
    d = blocks[:, 0:2].copy().view(np.float16).astype(np.float64)        # [nb, 1]
    dmin = blocks[:, 2:4].copy().view(np.float16).astype(np.float64)
    s = blocks[:, 4:16].astype(np.int64)
    sc = np.concatenate([s[:, 0:4] & 63, (s[:, 8:12] & 15) | ((s[:, 0:4] >> 6) << 4)], axis=1)
    mn = np.concatenate([s[:, 4:8] & 63, (s[:, 8:12] >> 4) | ((s[:, 4:8] >> 6) << 4)], axis=1)
    qs = blocks[:, 16:].astype(np.int64).reshape(nb, 4, 32)
    q = np.stack([qs & 15, qs >> 4], axis=2).reshape(nb, 8, 32)
    return ((d * sc)[:, :, None] * q - (dmin * mn)[:, :, None]).reshape(nb, 256)


def test_block_geometry_matches_the_reference_tests():
    # tests/test_gguf.cpp:78 and :106: 256 values and 144 bytes per Q4_K block
    assert W.QK_K == 256 and W.Q4K_BLOCK_BYTES == 144
    blocks = W.random_q4k(np.random.default_rng(0), 3, 512)
    assert blocks.shape == (3, 2, 144)


def test_scale_and_minimum_unpacking_inverts_the_packing(oracle):
    """Every 6-bit value in every one of the 8 positions, packed as ggml's quantiser packs
    it, comes back out of go_q4k_scale_min; the other positions hold the complement so a
    wrong shift or index shows."""
    sc, m = np.zeros(1, np.uint8), np.zeros(1, np.uint8)
    for j in range(8):
        for value in range(64):
            scales = np.full((1, 8), 63 - value)
            mins = np.full((1, 8), (value * 7 + 3) % 64)
            scales[0, j] = value
            mins[0, j] = 63 - value
            block = W.pack_q4k(np.ones(1, np.float16), np.ones(1, np.float16), scales, mins,
                               np.zeros((1, 256), np.int64))
            for jj in range(8):
                oracle.lib.go_q4k_scale_min(jj, np.ascontiguousarray(block[0, 4:16]), sc, m)
                assert (int(sc[0]), int(m[0])) == (int(scales[0, jj]), int(mins[0, jj])), (j, value, jj)


def test_closed_form_blocks(oracle):
    ones, zeros = np.ones(1, np.float16), np.zeros(1, np.float16)
    # d = 1, every scale 1, no minimum: the weights are the nibbles, in order
    q = (np.arange(256) * 5 % 16).reshape(1, 256)
    block = W.pack_q4k(ones, zeros, np.ones((1, 8)), np.zeros((1, 8)), q)
    w32, w16 = oracle.q4k_dequantize(block)
    assert np.array_equal(w32, q[0].astype(np.float32))
    assert np.array_equal(w16.view(np.float16).astype(np.float32), q[0].astype(np.float32))
    # q = 0: weight = -dmin * min of its sub-block of 32
    mins = np.arange(8).reshape(1, 8) * 9
    block = W.pack_q4k(ones, np.full(1, 0.5, np.float16), np.ones((1, 8)), mins, np.zeros((1, 256)))
    w32, _ = oracle.q4k_dequantize(block)
    assert np.array_equal(w32.reshape(8, 32), np.repeat(-0.5 * mins.reshape(8, 1), 32, axis=1).astype(np.float32))
    # sub-block j scaled by j: weight = 2 * j * q
    block = W.pack_q4k(np.full(1, 2.0, np.float16), zeros, np.arange(8).reshape(1, 8) * 8 + 1, np.zeros((1, 8)),
                       np.full((1, 256), 3))
    w32, _ = oracle.q4k_dequantize(block)
    assert np.array_equal(w32.reshape(8, 32)[:, 0], (2.0 * (np.arange(8) * 8 + 1) * 3).astype(np.float32))
    # the first 32 weights of every 64 are the low nibbles of 32 bytes, the next 32 the high ones
    block = np.zeros((1, 144), np.uint8)
    block[0, 0:2] = np.array([1.0], np.float16).view(np.uint8)
    block[0, 4:8] = 1                     # scales of sub-blocks 0..3 = 1 (4..7 stay 0)
    block[0, 16] = 0xA3                   # byte 0 of the nibbles: weight 0 = 3, weight 32 = 10
    w32, _ = oracle.q4k_dequantize(block)
    assert w32[0] == 3 and w32[32] == 10 and np.count_nonzero(w32) == 2


def test_dequantisation_against_float64(oracle):
    rng = np.random.default_rng(5)
    blocks = W.random_q4k(rng, 7, 1024).reshape(-1, 144)
    w32, w16 = oracle.q4k_dequantize(blocks)
    want = dequant64(blocks).reshape(-1)
    # one product and one subtraction in float: within an ulp or so of the float64 value
    assert np.all(np.abs(w32 - want) <= 2.0 ** -22 * np.maximum(np.abs(want), 1e-3))
    # what the reference stores: the float value through its truncating conversion
    assert np.array_equal(w16, oracle.fp32_to_fp16(w32))


def test_projection_against_float64_and_the_reference_routine(oracle):
    case = W.make_qkv_projection(seed=9, K=1024, num_heads=3, num_kv_heads=1, head_dim=32, batch=3)
    w64 = dequant64(case.wq.reshape(-1, 144)).reshape(case.Nq, case.K)
    want = case.x.astype(np.float64) @ w64.T
    bound = (np.abs(case.x).astype(np.float64) @ np.abs(w64).T) * case.K * 2.0 ** -24
    got = oracle.matvec_q4k(case.x, case.wq)
    assert got.shape == (3, case.Nq)
    assert np.all(np.abs(got - want) <= bound)
    # the CPU path multiplies by the half weights it stored at load time (math_ops.cpp:95-103)
    _, w16 = oracle.q4k_dequantize(case.wq)
    cpu = oracle.matmul_transb_fp16(case.x, w16.reshape(case.Nq, case.K))
    w16_64 = w16.view(np.float16).astype(np.float64).reshape(case.Nq, case.K)
    assert np.all(np.abs(cpu - case.x.astype(np.float64) @ w16_64.T) <= bound)
    # truncation to half moves a weight by less than 2^-10 of itself (half subnormals aside)
    assert np.all(np.abs(cpu - got) <= 2.0 ** -10 * (np.abs(case.x).astype(np.float64) @ np.abs(w64).T) + 2 * bound)
    ref = oracle_bind.load_ref()
    if ref is None:
        pytest.skip("oracle/_ref not built (no reference tree here)")
    c = np.empty_like(cpu)
    ref.ref_matmul_transb_fp16(case.x, w16.reshape(case.Nq, case.K), c, 3, case.Nq, case.K)
    assert np.array_equal(c, cpu)   # same loop, same order: bit for bit


def test_scale_fields_known_answer(oracle):
    """tests/golden/q4k_scales_kat.json: twelve hand-typed scale bytes and the eight (scale,
    minimum) pairs worked out by hand from src/model/gguf.cpp:963-971.  Pins the j >= 4
    branch (two bits from one byte, four from another) without any packing code of this
    repository in the loop."""
    q = np.array([int(h, 16) for h in KAT["scale_bytes_hex"]], np.uint8)
    sc, m = np.zeros(1, np.uint8), np.zeros(1, np.uint8)
    for j in range(8):
        oracle.lib.go_q4k_scale_min(j, q, sc, m)
        assert (int(sc[0]), int(m[0])) == (KAT["sc"][j], KAT["m"][j]), j
    # the same bytes through the vectorised restatement used elsewhere in this file
    block, want = kat_block()
    assert np.array_equal(dequant64(block[None]), want[None])
    # and the whole block through the oracle's dequantisation: every value exact
    w32, w16 = oracle.q4k_dequantize(block[None, None])
    assert np.array_equal(w32.astype(np.float64).reshape(-1), want)
    assert np.array_equal(w16.view(np.float16).astype(np.float64).reshape(-1), want)
