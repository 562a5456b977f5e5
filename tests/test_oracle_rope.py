"""Pins the oracle's rotary embedding (oracle/granite_oracle.c: go_rope_table, go_rope_apply)
without retyping it: the reference's own table tests (tests/test_llm.cpp:14-63), a float64
evaluation, and the properties any plane rotation has."""
import numpy as np
import pytest

import oracle_bind


@pytest.fixture(scope="module")
def oracle():
    return oracle_bind.load()


def test_table_shape_and_position_zero(oracle):
    # tests/test_llm.cpp:14-40: 2048 x 32 entries for head_dim 64; at position 0 cos = 1, sin = 0
    cos, sin = oracle.rope_table(2048, 64, 10000.0)
    assert cos.shape == (2048, 32) and sin.shape == (2048, 32)
    cos8, sin8 = oracle.rope_table(1024, 8, 10000.0)
    assert np.all(np.abs(cos8[0] - 1.0) <= 1e-5) and np.all(np.abs(sin8[0]) <= 1e-5)


def test_table_position_one_against_libm(oracle):
    # tests/test_llm.cpp:42-63: position 1, head_dim 8, theta 10000, within 1e-5
    cos, sin = oracle.rope_table(1024, 8, 10000.0)
    for i in range(4):
        angle = 1.0 / np.float32(10000.0) ** (np.float32(2 * i) / np.float32(8))
        assert abs(cos[1, i] - np.cos(angle)) <= 1e-5
        assert abs(sin[1, i] - np.sin(angle)) <= 1e-5


@pytest.mark.parametrize("head_dim,theta", [(128, 10000.0), (64, 500000.0), (8, 10000.0)])
def test_table_against_float64_of_the_fp32_angle(oracle, head_dim, theta):
    """The angle is formed in fp32 (pos * freq); given that angle, cos and sin must be the
    correctly rounded ones to within an ulp or two."""
    n = 4096
    cos, sin = oracle.rope_table(n, head_dim, theta)
    i = np.arange(head_dim // 2)
    freq64 = 1.0 / np.float64(theta) ** (2.0 * i / head_dim)
    # fp32 freq may differ from the float64 one in its last place; allow for it through the angle
    pos = np.arange(n, dtype=np.float64)[:, None]
    angle = pos * freq64[None, :]
    slack = 1e-6 + pos * freq64[None, :] * 2.0 ** -22  # angle error of an fp32 freq and product
    assert np.all(np.abs(cos - np.cos(angle)) <= slack)
    assert np.all(np.abs(sin - np.sin(angle)) <= slack)
    assert np.all(np.abs(cos.astype(np.float64) ** 2 + sin.astype(np.float64) ** 2 - 1.0) <= 1e-6)


def test_apply_is_a_rotation(oracle):
    rng = np.random.default_rng(1)
    cos, sin = oracle.rope_table(512, 64)
    x = rng.standard_normal((37, 5, 64)).astype(np.float32)
    y = oracle.rope_apply(x, 100, cos, sin)
    # pair norms are kept
    nx = x[..., 0::2].astype(np.float64) ** 2 + x[..., 1::2].astype(np.float64) ** 2
    ny = y[..., 0::2].astype(np.float64) ** 2 + y[..., 1::2].astype(np.float64) ** 2
    assert np.all(np.abs(nx - ny) <= 1e-5 * (1 + nx))
    # position 0 is the identity (cos = 1, sin = 0 exactly)
    assert np.array_equal(oracle.rope_apply(x[:1], 0, cos, sin), x[:1])
    # heads are treated alike: rotating one head alone gives the same numbers
    assert np.array_equal(oracle.rope_apply(x[:, 2:3], 100, cos, sin), y[:, 2:3])


def test_apply_against_float64_and_sign_convention(oracle):
    """(1, 0) at position p maps to (cos, sin), (0, 1) to (-sin, cos): fixes which of the
    two outputs carries the minus sign; random data against a float64 complex multiply."""
    cos, sin = oracle.rope_table(300, 16)
    e0 = np.zeros((1, 1, 16), np.float32); e0[..., 0::2] = 1.0
    e1 = np.zeros((1, 1, 16), np.float32); e1[..., 1::2] = 1.0
    y0 = oracle.rope_apply(e0, 7, cos, sin)[0, 0]
    y1 = oracle.rope_apply(e1, 7, cos, sin)[0, 0]
    assert np.array_equal(y0[0::2], cos[7]) and np.array_equal(y0[1::2], sin[7])
    assert np.array_equal(y1[0::2], -sin[7]) and np.array_equal(y1[1::2], cos[7])
    rng = np.random.default_rng(2)
    x = rng.standard_normal((50, 3, 16)).astype(np.float32)
    y = oracle.rope_apply(x, 250, cos, sin)
    z = (x[..., 0::2] + 1j * x[..., 1::2]).astype(np.complex128)
    rot = (cos[250:300] + 1j * sin[250:300]).astype(np.complex128)[:, None, :]
    want = z * rot
    assert np.all(np.abs(y[..., 0::2] - want.real) <= 1e-6 * (1 + np.abs(want)))
    assert np.all(np.abs(y[..., 1::2] - want.imag) <= 1e-6 * (1 + np.abs(want)))


def test_two_rotations_compose(oracle):
    """Rotating by position a and then by position b equals rotating by a + b (to rounding)."""
    cos, sin = oracle.rope_table(64, 32)
    rng = np.random.default_rng(3)
    x = rng.standard_normal((1, 4, 32)).astype(np.float32)
    ab = oracle.rope_apply(oracle.rope_apply(x, 5, cos, sin), 9, cos, sin)
    direct = oracle.rope_apply(x, 14, cos, sin)
    assert np.all(np.abs(ab - direct) <= 2e-5)


def test_apply_range_error(oracle):
    # rope.cpp:34-38: start_pos + seq_len > max_seq_len is refused
    cos, sin = oracle.rope_table(16, 8)
    x = np.zeros((4, 1, 8), np.float32)
    oracle.rope_apply(x, 12, cos, sin)
    with pytest.raises(ValueError):
        oracle.rope_apply(x, 13, cos, sin)
