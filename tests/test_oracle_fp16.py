"""Pins the oracle's half<->float conversions (src/llm/math_ops.cpp:18-54)."""
import json
from pathlib import Path

import numpy as np
import pytest

import oracle_bind

GOLDEN = Path(__file__).parent / "golden"


def _bits32(x: np.ndarray) -> np.ndarray:
    return np.ascontiguousarray(x, np.float32).view(np.uint32)


def test_fp16_to_fp32_all_65536_match_ieee(oracle):
    h = np.arange(65536, dtype=np.uint16)
    got = oracle.fp16_to_fp32(h)
    want = h.view(np.float16).astype(np.float32)  # IEEE widening is exact
    nan = np.isnan(want)
    assert np.array_equal(_bits32(got)[~nan], _bits32(want)[~nan])
    # NaNs: sign | 0x7F800000 | mant << 13 (math_ops.cpp:33-38)
    hn = h[nan].astype(np.uint32)
    expect = ((hn >> 15) << 31) | 0x7F800000 | ((hn & 0x3FF) << 13)
    assert np.array_equal(_bits32(got)[nan], expect)


def test_fp32_to_fp16_closed_form_random(oracle):
    rng = np.random.default_rng(7)
    bits = rng.integers(0, 2**32, size=400000, dtype=np.uint64).astype(np.uint32)
    f = bits.view(np.float32)
    got = oracle.fp32_to_fp16(f)
    sign = (bits >> 16) & 0x8000
    e = ((bits >> 23) & 0xFF).astype(np.int64) - 127 + 15
    mant = (bits >> 13) & 0x3FF
    want = np.where(e <= 0, sign, np.where(e >= 31, sign | 0x7C00, sign | (e.clip(0, 31) << 10) | mant))
    assert np.array_equal(got, want.astype(np.uint16))


def test_fp32_to_fp16_is_truncation_toward_zero(oracle):
    """For values inside the normal half range the result is the nearest half
    whose magnitude does not exceed |x| -- a property, not the formula."""
    rng = np.random.default_rng(11)
    f = (rng.standard_normal(200000) * 8).astype(np.float32)
    f = f[np.abs(f) >= 2.0**-14]
    got = oracle.fp32_to_fp16(f).view(np.float16).astype(np.float64)
    assert np.all(np.abs(got) <= np.abs(f.astype(np.float64)))
    rne = f.astype(np.float16).astype(np.float64)
    ulp = np.spacing(np.abs(got).astype(np.float16)).astype(np.float64)
    assert np.all(np.abs(f.astype(np.float64)) - np.abs(got) < ulp)
    assert np.all(np.abs(rne - got) <= ulp)  # never further than one ulp from RNE


def test_known_answers(oracle):
    kat = json.loads((GOLDEN / "fp16_kat.json").read_text())
    for row in kat["fp32_to_fp16"]:
        f = np.array([int(row["f32_bits"], 16)], dtype=np.uint32).view(np.float32)
        assert int(oracle.fp32_to_fp16(f)[0]) == int(row["half"], 16), row
        if "NaN" not in row["value"]:
            with np.errstate(over="ignore"):
                assert int(f.astype(np.float16).view(np.uint16)[0]) == int(row["rne"], 16), row
    for row in kat["fp16_to_fp32"]:
        h = np.array([int(row["half"], 16)], dtype=np.uint16)
        assert int(_bits32(oracle.fp16_to_fp32(h))[0]) == int(row["f32_bits"], 16), row


def test_round_trip_is_identity_on_normals(oracle):
    h = np.arange(65536, dtype=np.uint16)
    e = (h >> 10) & 0x1F
    normal = (e > 0) & (e < 31)
    back = oracle.fp32_to_fp16(oracle.fp16_to_fp32(h[normal]))
    assert np.array_equal(back, h[normal])
    # subnormals flush to signed zero on the way back (exp <= 0 branch)
    sub = (e == 0)
    back = oracle.fp32_to_fp16(oracle.fp16_to_fp32(h[sub]))
    assert np.array_equal(back, h[sub] & 0x8000)


def test_against_reference_build(oracle):
    """oracle/_ref holds the reference's own math_ops.cpp when it was built."""
    ref = oracle_bind.load_ref()
    if ref is None:
        pytest.skip("oracle/_ref not built (reference tree absent)")
    h = np.arange(65536, dtype=np.uint16)
    want = np.empty(65536, np.float32)
    ref.ref_fp16_to_fp32_array(h, want, h.size)
    assert np.array_equal(_bits32(oracle.fp16_to_fp32(h)), _bits32(want))
    rng = np.random.default_rng(3)
    bits = rng.integers(0, 2**32, size=100000, dtype=np.uint64).astype(np.uint32)
    f = bits.view(np.float32)
    got = oracle.fp32_to_fp16(f)
    want16 = np.array([ref.ref_fp32_to_fp16(float(x)) if np.isfinite(x) else ref.ref_fp32_to_fp16(x)
                       for x in f[:20000]], dtype=np.uint16)
    finite = np.isfinite(f[:20000])  # ctypes passes NaN payloads through double; compare finite only
    assert np.array_equal(got[:20000][finite], want16[finite])


def test_parallel_for_partition_matches_reference(oracle):
    """Thread partition of math_ops.h:41-69: chunk = ceil(n/threads), index i
    belongs to chunk i // chunk; serial when n < threads."""
    ref = oracle_bind.load_ref()
    if ref is None:
        pytest.skip("oracle/_ref not built (reference tree absent)")
    for n, t in [(10, 4), (100, 8), (7, 8), (64, 64), (1000, 3), (1, 1), (9, 4), (13, 5), (1001, 16), (33, 32)]:
        visited = np.zeros(n, np.uint8)
        calls = ref.ref_parallel_for_count(n, t, visited)
        assert calls == n and np.all(visited == 1)
        # the partition as executed: which thread ran which index, on both sides
        ref_owner, own_owner = np.full(n, -1, np.int32), np.full(n, -1, np.int32)
        ref.ref_parallel_for_owner(n, t, ref_owner)
        oracle.lib.go_parallel_for_owner(n, t, own_owner)
        assert np.array_equal(ref_owner, own_owner), (n, t)
        # and against the closed form: serial below one item per thread, else chunks of ceil(n / t)
        chunk = -(-n // t)
        want = np.zeros(n, np.int32) if (t <= 1 or n < t) else (np.arange(n) // chunk * chunk).astype(np.int32)
        assert np.array_equal(own_owner, want), (n, t)
