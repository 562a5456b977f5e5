"""The decode entry point that allocates nothing (granite_hip_decode_attention_static):
called through the C ABI, twice in a row, the second time on a smaller batch, and compared
bit for bit with granite_hip_decode_attention, which runs the same kernels on the library's
growable scratch.  Sizes beyond the static scratch are refused before anything is launched."""
import ctypes as C

import numpy as np
import pytest

from granite_amd import F16, F32, GraniteHipError, _capi
from granite_amd import workloads as W
from gpu_util import assert_close, dev, say

pytestmark = pytest.mark.gpu


def _args(case, q_dtype, out, lse):
    q = case.q if q_dtype == F16 else case.q.astype(np.float32)
    keep = [dev(q), dev(case.k_pool), dev(case.v_pool), dev(case.block_tables), dev(case.seq_lens)]
    a = _capi.DecodeArgs(q=keep[0].ptr, q_dtype=q_dtype, k_cache=keep[1].ptr, v_cache=keep[2].ptr,
                         block_tables=keep[3].ptr, seq_lens=keep[4].ptr, out=out.ptr, lse=lse.ptr,
                         batch_size=case.batch, num_heads=case.num_heads, num_kv_heads=case.num_kv_heads,
                         head_dim=128, block_size=case.block_size, max_blocks_per_seq=case.max_blocks,
                         max_seq=0, scale=case.scale, fixed_seq_len=0, chunk_tokens=0)
    return a, keep


def _free_device_bytes(hip) -> int:
    free, total = C.c_size_t(), C.c_size_t()
    assert hip.hipMemGetInfo(C.byref(free), C.byref(total)) == 0
    return free.value


def _timing_names(lib) -> list:
    buf = C.create_string_buffer(4096)
    lib.granite_hip_kernel_timing_names(buf, len(buf))
    return sorted(n for n in buf.value.decode().split(",") if n)


def test_static_scratch_decode_matches_the_allocating_entry_point(gpu, oracle):
    lib = _capi.load()
    hip = C.CDLL("libamdhip64.so")
    limit = lib.granite_hip_static_scratch_bytes()
    assert limit == 32 << 20
    rng = np.random.default_rng(77)
    # first call: 24 sequences of mixed lengths (stream kernel, partials and plan in scratch);
    # second call: a smaller batch with other lengths, so stale partials of the first call lie
    # in the array where the second reads only what it wrote itself
    shapes = [(rng.integers(800, 4097, size=24).astype(np.int32), F16),
              (np.array([3000, 1, 950, 2048, 777], np.int32), F32)]
    for call, (lens, q_dtype) in enumerate(shapes):
        say(f"static-scratch decode call {call}: batch={len(lens)} q_dtype={q_dtype}")
        case = W.make_paged_decode(seed=300 + call, ctx_max=4096, seq_lens=lens)
        b = case.batch
        out_ref, lse_ref = dev(np.zeros((b, 32, 128), np.float32)), dev(np.zeros((b, 32), np.float32))
        out_new, lse_new = dev(np.full((b, 32, 128), 7.0, np.float32)), dev(np.full((b, 32), 7.0, np.float32))
        a_ref, keep_ref = _args(case, q_dtype, out_ref, lse_ref)
        a_new, keep_new = _args(case, q_dtype, out_new, lse_new)
        need = C.c_size_t()
        _capi.check(lib.granite_hip_decode_workspace_required(C.byref(a_ref), C.byref(need)), "required")
        assert 0 < need.value <= limit
        _capi.check(lib.granite_hip_decode_attention(C.byref(a_ref)), "decode_attention")
        gpu.sync()
        held = lib.granite_hip_workspace_bytes()
        # the device's free memory, to the byte, before and after: a hipMalloc or hipFree inside
        # the call (or one pair of them that does not net out) would show
        free_before = _free_device_bytes(hip)
        _capi.check(lib.granite_hip_decode_attention_static(C.byref(a_new)), "decode_attention_static")
        assert _free_device_bytes(hip) == free_before
        gpu.sync()
        assert _free_device_bytes(hip) == free_before
        assert lib.granite_hip_workspace_bytes() == held
        got, ref = out_new.read(np.uint32, (b, 32, 128)), out_ref.read(np.uint32, (b, 32, 128))
        assert np.array_equal(got, ref), "outputs differ from granite_hip_decode_attention"
        assert np.array_equal(lse_new.read(np.uint32, (b, 32)), lse_ref.read(np.uint32, (b, 32)))
        want, _ = oracle.batched_paged_decode(case.q.astype(np.float32), case.k_pool, case.v_pool,
                                              case.block_tables, case.seq_lens, case.block_size, case.scale)
        assert_close(got.view(np.float32), want, "static-scratch decode vs oracle")
        if call == 1:
            # with kernel timing on, the allocating entry point records its launches (and creates
            # events for that); the static one must record nothing
            _capi.check(lib.granite_hip_reset_kernel_timing(), "reset timing")
            _capi.check(lib.granite_hip_enable_kernel_timing(1), "enable timing")
            try:
                _capi.check(lib.granite_hip_decode_attention_static(C.byref(a_new)), "decode_attention_static")
                gpu.sync()
                assert _timing_names(lib) == [], "the static entry point recorded timing events"
                _capi.check(lib.granite_hip_decode_attention(C.byref(a_ref)), "decode_attention")
                gpu.sync()
                assert _timing_names(lib) != []     # (the switch does work)
            finally:
                _capi.check(lib.granite_hip_enable_kernel_timing(0), "disable timing")
                _capi.check(lib.granite_hip_reset_kernel_timing(), "reset timing")
            assert np.array_equal(out_new.read(np.uint32, (b, 32, 128)), ref)
        del keep_ref, keep_new


def test_static_scratch_decode_refuses_what_does_not_fit(gpu):
    lib = _capi.load()
    buf = dev(np.zeros(1 << 16, np.float32))
    # 4096 sequences x 64 heads: far more partial slots than 32 MiB hold.  Nothing is launched,
    # so the (too small) buffers are never touched.
    a = _capi.DecodeArgs(q=buf.ptr, q_dtype=F16, k_cache=buf.ptr, v_cache=buf.ptr, block_tables=buf.ptr,
                         seq_lens=buf.ptr, out=buf.ptr, lse=None, batch_size=4096, num_heads=64,
                         num_kv_heads=8, head_dim=128, block_size=16, max_blocks_per_seq=512, max_seq=0,
                         scale=0.1, fixed_seq_len=0, chunk_tokens=0)
    need = C.c_size_t()
    _capi.check(lib.granite_hip_decode_workspace_required(C.byref(a), C.byref(need)), "required")
    assert need.value > lib.granite_hip_static_scratch_bytes()
    rc = lib.granite_hip_decode_attention_static(C.byref(a))
    assert rc == _capi.ESCRATCH
    assert b"scratch" in lib.granite_hip_error_string(rc)
    gpu.sync()
