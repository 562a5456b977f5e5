"""Python mirror of the HipCompute class (the MetalCompute-shaped API of the
HIP backend).  Method names, argument order and meaning follow
include/granite/metal_compute.h:752-920 of the reference; every call goes
straight to the C ABI in libgranite_hip.so.  Used by the tests and the
benchmark; the C++ host layer in granite_amd/host is the same surface for C++
callers.
"""
from __future__ import annotations

import ctypes as C
from typing import Optional

import numpy as np

from . import _capi
from ._capi import (F16, F32, MASK_CAUSAL, MASK_NONE, MASK_TREE, MEM_DEVICE, ROUND_NEAREST,
                    ROUND_TRUNCATE, AttentionArgs, RopeArgs, DecodeArgs, check)


class DeviceBuffer:
    """A device allocation owned by the caller (Granite's MTL::Buffer stand-in)."""

    def __init__(self, nbytes: int, kind: int = MEM_DEVICE):
        self.nbytes = int(nbytes)
        self.kind = kind
        ptr = C.c_void_p()
        check(_capi.load().granite_hip_malloc(C.byref(ptr), max(self.nbytes, 16), kind), "malloc")
        self.ptr = ptr.value

    @classmethod
    def from_numpy(cls, arr: np.ndarray) -> "DeviceBuffer":
        arr = np.ascontiguousarray(arr)
        buf = cls(arr.nbytes)
        buf.write(arr)
        return buf

    def write(self, arr: np.ndarray, offset: int = 0) -> None:
        arr = np.ascontiguousarray(arr)
        if offset + arr.nbytes > self.nbytes:
            raise ValueError("write beyond the end of the buffer")
        check(_capi.load().granite_hip_memcpy_h2d(self.ptr + offset, arr.ctypes.data, arr.nbytes),
              "memcpy_h2d")

    def read(self, dtype, shape, offset: int = 0) -> np.ndarray:
        out = np.empty(shape, dtype=dtype)
        if offset + out.nbytes > self.nbytes:
            raise ValueError("read beyond the end of the buffer")
        check(_capi.load().granite_hip_memcpy_d2h(out.ctypes.data, self.ptr + offset, out.nbytes),
              "memcpy_d2h")
        return out

    def fill(self, byte: int) -> None:
        check(_capi.load().granite_hip_memset(self.ptr, byte, self.nbytes), "memset")

    def free(self) -> None:
        if self.ptr:
            check(_capi.load().granite_hip_free(self.ptr, self.kind), "free")
            self.ptr = None

    def __del__(self):
        try:
            if getattr(self, "ptr", None) and _capi.load().granite_hip_is_initialized():
                _capi.load().granite_hip_free(self.ptr, self.kind)
        except Exception:
            pass


def _p(buf) -> Optional[int]:
    if buf is None:
        return None
    return buf.ptr if isinstance(buf, DeviceBuffer) else int(buf)


class HipCompute:
    """One in-order queue of attention / KV work on one MI355X."""

    def __init__(self, device: int = 0):
        self.lib = _capi.load()
        self.device = device
        self.initialize()

    # ---- lifecycle (MetalCompute::initialize / shutdown / sync / commit)
    def initialize(self) -> None:
        check(self.lib.granite_hip_init(self.device), "init")

    def shutdown(self) -> None:
        check(self.lib.granite_hip_shutdown(), "shutdown")

    def is_initialized(self) -> bool:
        return bool(self.lib.granite_hip_is_initialized())

    def sync(self) -> None:
        check(self.lib.granite_hip_sync(), "sync")

    def commit(self) -> None:
        """Launches are submitted as they are made; nothing to flush."""

    def device_info(self) -> _capi.DeviceInfo:
        info = _capi.DeviceInfo()
        check(self.lib.granite_hip_get_device_info(C.byref(info)), "get_device_info")
        return info

    def create_buffer(self, size: int, shared: bool = False) -> DeviceBuffer:
        return DeviceBuffer(size, _capi.MEM_SHARED if shared else MEM_DEVICE)

    # ---- timing
    def event(self) -> int:
        ev = C.c_void_p()
        check(self.lib.granite_hip_event_create(C.byref(ev)), "event_create")
        return ev.value

    def record(self, ev: int) -> None:
        check(self.lib.granite_hip_event_record(ev), "event_record")

    def elapsed_ms(self, start: int, stop: int) -> float:
        check(self.lib.granite_hip_event_synchronize(stop), "event_synchronize")
        ms = C.c_float()
        check(self.lib.granite_hip_event_elapsed_ms(start, stop, C.byref(ms)), "event_elapsed")
        return ms.value

    def destroy_event(self, ev: int) -> None:
        check(self.lib.granite_hip_event_destroy(ev), "event_destroy")

    # ---- per-kernel timing (MetalCompute::enable_kernel_timing & co.)
    def enable_kernel_timing(self, enable: bool) -> None:
        check(self.lib.granite_hip_enable_kernel_timing(int(enable)), "enable_kernel_timing")

    def reset_kernel_timing(self) -> None:
        check(self.lib.granite_hip_reset_kernel_timing(), "reset_kernel_timing")

    def get_kernel_timing_stats(self) -> dict:
        """{kernel name: (total GPU milliseconds, dispatches)}"""
        buf = C.create_string_buffer(4096)
        check(self.lib.granite_hip_kernel_timing_names(buf, len(buf)), "kernel_timing_names")
        stats = {}
        for name in filter(None, buf.value.decode().split(",")):
            ms, n = C.c_double(), C.c_uint64()
            check(self.lib.granite_hip_get_kernel_timing(name.encode(), C.byref(ms), C.byref(n)),
                  "get_kernel_timing")
            stats[name] = (ms.value, n.value)
        return stats

    # ---- KV cache
    def kv_cache_append(self, cache_k, cache_v, new_k, new_v, num_kv_heads, head_dim,
                        current_len, new_len, max_seq_len) -> None:
        check(self.lib.granite_hip_kv_cache_append(_p(cache_k), _p(cache_v), _p(new_k), _p(new_v),
                                                   num_kv_heads, head_dim, current_len, new_len,
                                                   max_seq_len), "kv_cache_append")

    def kv_cache_append_ex(self, cache_k, cache_v, new_k, new_v, src_dtype, src_tok_stride,
                           src_head_stride, num_kv_heads, head_dim, current_len, new_len,
                           max_seq_len, rounding=ROUND_TRUNCATE) -> None:
        check(self.lib.granite_hip_kv_cache_append_ex(
            _p(cache_k), _p(cache_v), _p(new_k), _p(new_v), src_dtype, src_tok_stride,
            src_head_stride, num_kv_heads, head_dim, current_len, new_len, max_seq_len, rounding),
            "kv_cache_append_ex")

    def paged_kv_cache_append(self, new_k, new_v, k_cache, v_cache, block_table, num_kv_heads,
                              head_dim, start_pos, new_len, block_size) -> None:
        check(self.lib.granite_hip_paged_kv_cache_append(
            _p(new_k), _p(new_v), _p(k_cache), _p(v_cache), _p(block_table), num_kv_heads,
            head_dim, start_pos, new_len, block_size), "paged_kv_cache_append")

    def paged_kv_cache_append_ex(self, new_k, new_v, src_dtype, src_tok_stride, src_head_stride,
                                 k_cache, v_cache, block_table, num_kv_heads, head_dim, start_pos,
                                 new_len, block_size, rounding=ROUND_TRUNCATE, max_blocks=0) -> None:
        """max_blocks: entries of block_table (0: not stated); an append that would run past
        them fails with EOVERFLOW instead of reading beyond the table."""
        check(self.lib.granite_hip_paged_kv_cache_append_ex(
            _p(new_k), _p(new_v), src_dtype, src_tok_stride, src_head_stride, _p(k_cache),
            _p(v_cache), _p(block_table), num_kv_heads, head_dim, start_pos, new_len, block_size,
            rounding, max_blocks), "paged_kv_cache_append_ex")

    def paged_kv_gather(self, dst_k, dst_v, k_cache, v_cache, block_table, num_kv_heads, head_dim,
                        length, block_size, max_seq_len) -> None:
        check(self.lib.granite_hip_paged_kv_gather(
            _p(dst_k), _p(dst_v), _p(k_cache), _p(v_cache), _p(block_table), num_kv_heads,
            head_dim, length, block_size, max_seq_len), "paged_kv_gather")

    def copy_rows(self, dst, dst_row_bytes, src, src_row_bytes, rows, copy_bytes, fill_bytes) -> None:
        """Strided row copy with the tail of every destination row zeroed (granite_hip_copy_rows)."""
        check(self.lib.granite_hip_copy_rows(_p(dst), dst_row_bytes, _p(src), src_row_bytes, rows, copy_bytes,
                                             fill_bytes), "copy_rows")

    # ---- attention (reference-shaped entry points)
    def multihead_attention(self, Q, K, V, output, num_heads, num_kv_heads, seq_q, seq_kv,
                            head_dim, scale, max_seq=0) -> None:
        check(self.lib.granite_hip_multihead_attention(
            _p(Q), _p(K), _p(V), _p(output), num_heads, num_kv_heads, seq_q, seq_kv, head_dim,
            scale, max_seq), "multihead_attention")

    def attention_tree(self, Q, K_cache, V_cache, K_tree, V_tree, parent_indices, output,
                       num_heads, num_kv_heads, num_nodes, cache_len, head_dim, scale) -> None:
        check(self.lib.granite_hip_attention_tree(
            _p(Q), _p(K_cache), _p(V_cache), _p(K_tree), _p(V_tree), _p(parent_indices),
            _p(output), num_heads, num_kv_heads, num_nodes, cache_len, head_dim, scale),
            "attention_tree")

    def paged_attention_decode(self, Q, K_cache, V_cache, block_table, output, num_heads,
                               num_kv_heads, seq_len, head_dim, block_size, scale) -> None:
        check(self.lib.granite_hip_paged_attention_decode(
            _p(Q), _p(K_cache), _p(V_cache), _p(block_table), _p(output), num_heads, num_kv_heads,
            seq_len, head_dim, block_size, scale), "paged_attention_decode")

    def batched_paged_attention_decode(self, Q, K_cache, V_cache, block_tables, seq_lens, output,
                                       batch_size, num_heads, num_kv_heads, head_dim, block_size,
                                       max_blocks_per_seq, scale) -> None:
        check(self.lib.granite_hip_batched_paged_attention_decode(
            _p(Q), _p(K_cache), _p(V_cache), _p(block_tables), _p(seq_lens), _p(output),
            batch_size, num_heads, num_kv_heads, head_dim, block_size, max_blocks_per_seq, scale),
            "batched_paged_attention_decode")

    # ---- attention (general forms)
    def decode_attention(self, *, q, q_dtype, k_cache, v_cache, out, batch_size, num_heads,
                         num_kv_heads, head_dim, scale, block_tables=None, seq_lens=None,
                         lse=None, block_size=0, max_blocks_per_seq=0, max_seq=0,
                         fixed_seq_len=0, chunk_tokens=0, workspace=None, workspace_bytes=None,
                         query_workspace=False, static_scratch=False):
        """workspace: a DeviceBuffer (or pointer + workspace_bytes) the launch takes its scratch
        from instead of the library's buffer.  query_workspace: launch nothing, return the
        scratch bytes the launch would need."""
        a = DecodeArgs(q=_p(q), q_dtype=q_dtype, k_cache=_p(k_cache), v_cache=_p(v_cache),
                       block_tables=_p(block_tables), seq_lens=_p(seq_lens), out=_p(out),
                       lse=_p(lse), batch_size=batch_size, num_heads=num_heads,
                       num_kv_heads=num_kv_heads, head_dim=head_dim, block_size=block_size,
                       max_blocks_per_seq=max_blocks_per_seq, max_seq=max_seq, scale=scale,
                       fixed_seq_len=fixed_seq_len, chunk_tokens=chunk_tokens)
        if query_workspace:
            need = C.c_size_t()
            check(self.lib.granite_hip_decode_workspace_required(C.byref(a), C.byref(need)),
                  "decode_workspace_required")
            return need.value
        if static_scratch:  # the entry point that allocates nothing
            check(self.lib.granite_hip_decode_attention_static(C.byref(a)), "decode_attention_static")
            return None
        if workspace is not None:
            nbytes = workspace.nbytes if workspace_bytes is None else workspace_bytes
            check(self.lib.granite_hip_decode_attention_ws(C.byref(a), _p(workspace), nbytes),
                  "decode_attention_ws")
        else:
            check(self.lib.granite_hip_decode_attention(C.byref(a)), "decode_attention")

    def attention(self, *, q, q_dtype, q_tok_stride, q_head_stride, out, out_dtype,
                  out_tok_stride, out_head_stride, seq_q, num_heads, num_kv_heads, head_dim, scale,
                  k_cache=None, v_cache=None, cache_len=0, max_seq=0, block_table=None,
                  block_size=0, k_extra=None, v_extra=None, extra_len=0, parents=None,
                  mask_mode=MASK_CAUSAL, start_pos=0, lse=None, workspace=None, workspace_bytes=None,
                  query_workspace=False):
        a = AttentionArgs(q=_p(q), q_dtype=q_dtype, q_tok_stride=q_tok_stride,
                          q_head_stride=q_head_stride, out=_p(out), out_dtype=out_dtype,
                          out_tok_stride=out_tok_stride, out_head_stride=out_head_stride,
                          lse=_p(lse), k_cache=_p(k_cache), v_cache=_p(v_cache),
                          block_table=_p(block_table), block_size=block_size, max_seq=max_seq,
                          cache_len=cache_len, k_extra=_p(k_extra), v_extra=_p(v_extra),
                          extra_len=extra_len, parents=_p(parents), mask_mode=mask_mode,
                          start_pos=start_pos, seq_q=seq_q, num_heads=num_heads,
                          num_kv_heads=num_kv_heads, head_dim=head_dim, scale=scale)
        if query_workspace:
            need = C.c_size_t()
            check(self.lib.granite_hip_attention_workspace_required(C.byref(a), C.byref(need)),
                  "attention_workspace_required")
            return need.value
        if workspace is not None:
            nbytes = workspace.nbytes if workspace_bytes is None else workspace_bytes
            check(self.lib.granite_hip_attention_ws(C.byref(a), _p(workspace), nbytes), "attention_ws")
        else:
            check(self.lib.granite_hip_attention(C.byref(a)), "attention")

    # ---- scratch memory
    def workspace_bytes(self) -> int:
        return int(self.lib.granite_hip_workspace_bytes())

    def reserve_workspace(self, nbytes: int) -> None:
        """Grow the library's scratch now, so that later launches needing no more never allocate."""
        check(self.lib.granite_hip_reserve_workspace(nbytes), "reserve_workspace")

    def kv_commit_accepted(self, k_tree, v_tree, src_dtype, src_tok_stride, src_head_stride, num_nodes,
                           accepted_nodes, num_accepted, k_cache, v_cache, num_kv_heads, head_dim,
                           start_pos, block_table=None, block_size=0, max_seq_len=0,
                           rounding=ROUND_TRUNCATE) -> None:
        """Writes the accepted tree nodes' K/V rows, in path order, to cache positions
        start_pos .. (the step src/llm/speculative_runner.cpp:871-882 presumes done)."""
        check(self.lib.granite_hip_kv_commit_accepted(
            _p(k_tree), _p(v_tree), src_dtype, src_tok_stride, src_head_stride, num_nodes,
            _p(accepted_nodes), num_accepted, _p(k_cache), _p(v_cache), _p(block_table), num_kv_heads,
            head_dim, start_pos, block_size, max_seq_len, rounding), "kv_commit_accepted")

    def rope_multihead(self, q, k, num_heads_q, num_heads_k, seq_len, head_dim, start_pos,
                       freq_base=10000.0) -> None:
        """MetalCompute::rope_multihead (include/granite/metal_compute.h:728-739): q
        [seq, Hq, D] and k [seq, Hkv, D] float, rotated in place."""
        check(self.lib.granite_hip_rope_multihead(_p(q), _p(k), num_heads_q, num_heads_k, seq_len,
                                                  head_dim, start_pos, freq_base), "rope_multihead")

    def rope_append(self, *, seq_len, head_dim, start_pos, q=None, num_heads_q=0, q_f16=None, k=None,
                    num_heads_k=0, v=None, cache_k=None, cache_v=None, block_table=None, block_size=0,
                    max_seq_len=0, cos_table=None, sin_table=None, table_positions=0,
                    freq_base=10000.0, write_k_back=True, rounding=ROUND_TRUNCATE, positions=None,
                    table_stride=0, max_blocks_per_seq=0) -> None:
        """Rotation of Q and K and, in the same pass, the append of the rotated K and of V to
        the (contiguous or paged) half cache; with RoPECache's tables the rotation is
        bit-identical to RoPECache::apply (src/llm/rope.cpp:24-92)."""
        a = RopeArgs(q=_p(q), q_f16=_p(q_f16), k=_p(k), v=_p(v), cache_k=_p(cache_k),
                     cache_v=_p(cache_v), block_table=_p(block_table), cos_table=_p(cos_table),
                     sin_table=_p(sin_table), table_positions=table_positions,
                     num_heads_q=num_heads_q, num_heads_k=num_heads_k, seq_len=seq_len,
                     head_dim=head_dim, start_pos=start_pos, max_seq_len=max_seq_len,
                     block_size=block_size, freq_base=freq_base, write_k_back=int(write_k_back),
                     rounding=rounding, positions=_p(positions), table_stride=table_stride,
                     max_blocks_per_seq=max_blocks_per_seq)
        check(self.lib.granite_hip_rope_append(C.byref(a)), "rope_append")

    # ---- projections on Q4_K weights
    def fused_qkv_matvec_q4k(self, x, Wq, Wk, Wv, yq, yk, yv, K, Nq, Nkv, batch=1, x_stride=None,
                             yq_stride=None, ykv_stride=None) -> None:
        """MetalCompute::fused_qkv_matvec_q4k (include/granite/metal_compute.h:683-694): the
        three attention projections of one token (or of `batch` tokens) in one launch."""
        if batch == 1 and x_stride is None and yq_stride is None and ykv_stride is None:
            check(self.lib.granite_hip_fused_qkv_matvec_q4k(_p(x), _p(Wq), _p(Wk), _p(Wv), _p(yq), _p(yk),
                                                            _p(yv), K, Nq, Nkv), "fused_qkv_matvec_q4k")
            return
        check(self.lib.granite_hip_fused_qkv_matvec_q4k_batched(
            _p(x), K if x_stride is None else x_stride, _p(Wq), _p(Wk), _p(Wv), _p(yq), _p(yk), _p(yv),
            Nq if yq_stride is None else yq_stride, Nkv if ykv_stride is None else ykv_stride, K, Nq, Nkv,
            batch), "fused_qkv_matvec_q4k_batched")

    def matvec_q4k(self, x, W, y, K, N, batch=1) -> None:
        """MetalCompute::matvec_q4k (metal_compute.h:73-79): y = W x on Q4_K weights."""
        if batch == 1:
            check(self.lib.granite_hip_matvec_q4k(_p(x), _p(W), _p(y), K, N), "matvec_q4k")
        else:
            check(self.lib.granite_hip_matvec_q4k_batched(_p(x), K, _p(W), _p(y), N, K, N, batch),
                  "matvec_q4k_batched")

    def build_tree_mask(self, parent_indices, mask_words, num_nodes) -> None:
        check(self.lib.granite_hip_build_tree_mask(_p(parent_indices), _p(mask_words), num_nodes),
              "build_tree_mask")


_instance: Optional[HipCompute] = None


def get_hip_compute(device: int = 0) -> HipCompute:
    """Process-wide instance, created on first use (get_metal_compute() analogue,
    src/backend/metal/metal_compute.mm:2721-2745)."""
    global _instance
    if _instance is None:
        _instance = HipCompute(device)
    return _instance


__all__ = ["DeviceBuffer", "HipCompute", "get_hip_compute", "F16", "F32", "MASK_CAUSAL",
           "MASK_NONE", "MASK_TREE", "ROUND_NEAREST", "ROUND_TRUNCATE"]
