"""ctypes access to the CPU oracle (oracle/libgranite_oracle.so) and, where it
was built, to the reference's own math_ops.cpp (oracle/_ref).  Test-only."""
from __future__ import annotations

import ctypes as C
import subprocess
from pathlib import Path

import numpy as np

ROOT = Path(__file__).resolve().parent.parent
ORACLE_SO = ROOT / "oracle" / "libgranite_oracle.so"
REF_SO = ROOT / "oracle" / "_ref" / "libgranite_ref_mathops.so"

_f32p = np.ctypeslib.ndpointer(np.float32, flags="C_CONTIGUOUS")
_u16p = np.ctypeslib.ndpointer(np.uint16, flags="C_CONTIGUOUS")
_i32p = np.ctypeslib.ndpointer(np.int32, flags="C_CONTIGUOUS")
_u8p = np.ctypeslib.ndpointer(np.uint8, flags="C_CONTIGUOUS")
_int, _flt, _long, _vp = C.c_int, C.c_float, C.c_long, C.c_void_p


def _opt(arr):
    return None if arr is None else arr.ctypes.data_as(C.c_void_p)


class Oracle:
    def __init__(self, lib: C.CDLL):
        self.lib = lib
        L = lib
        L.go_fp16_to_fp32.restype = _flt
        L.go_fp16_to_fp32.argtypes = [C.c_uint16]
        L.go_fp32_to_fp16.restype = C.c_uint16
        L.go_fp32_to_fp16.argtypes = [_flt]
        L.go_fp16_to_fp32_array.argtypes = [_u16p, _f32p, C.c_size_t]
        L.go_fp32_to_fp16_array.argtypes = [_f32p, _u16p, C.c_size_t]
        L.go_set_num_threads.argtypes = [_int]
        L.go_get_num_threads.restype = _int
        L.go_parallel_for_owner.argtypes = [C.c_size_t, C.c_size_t, _i32p]
        L.go_kv_cache_append_f16.restype = _int
        L.go_kv_cache_append_f16.argtypes = [_u16p, _u16p, _int, _int, _int, _int, _int]
        L.go_kv_cache_append_f32.restype = _int
        L.go_kv_cache_append_f32.argtypes = [_u16p, _f32p, _int, _int, _int, _int, _int]
        L.go_paged_kv_cache_append_f32.argtypes = [_u16p, _f32p, _i32p, _int, _int, _int, _int, _int]
        L.go_paged_kv_cache_append_f16.argtypes = [_u16p, _u16p, _i32p, _int, _int, _int, _int,
                                                   _int, _long, _long]
        L.go_paged_gather_f16.argtypes = [_u16p, _u16p, _i32p, _int, _int, _int, _int, _int]
        L.go_attention_core.argtypes = [_f32p, _f32p, _f32p, _f32p, _vp, _int, _int, _int, _int,
                                        _int, _int, _int, _flt]
        L.go_attention_cached.argtypes = [_f32p, _u16p, _u16p, _f32p, _vp, _int, _int, _int, _int,
                                          _int, _int, _int, _int, _flt]
        L.go_attention_paged.argtypes = [_f32p, _u16p, _u16p, _i32p, _int, _f32p, _vp, _int, _int,
                                         _int, _int, _int, _int, _int, _flt]
        L.go_batched_paged_decode.argtypes = [_f32p, _u16p, _u16p, _i32p, _i32p, _f32p, _vp, _int,
                                              _int, _int, _int, _int, _int, _flt]
        L.go_tree_mask.restype = _int
        L.go_tree_mask.argtypes = [_i32p, _int, _u8p]
        L.go_attention_tree.restype = _int
        L.go_attention_tree.argtypes = [_f32p, _vp, _vp, _vp, _int, _int, _f32p, _f32p, _i32p,
                                        _f32p, _vp, _int, _int, _int, _int, _int, _int, _flt]
        L.go_block_manager_new.restype = _vp
        L.go_rope_table.argtypes = [_f32p, _f32p, _int, _int, _flt]
        L.go_rope_apply.argtypes = [_f32p, _int, _int, _int, _int, _f32p, _f32p, _int]
        L.go_rope_apply.restype = _int
        L.go_q4k_scale_min.argtypes = [_int, _u8p, _u8p, _u8p]
        L.go_q4k_dequantize.argtypes = [_u8p, C.c_size_t, _vp, _vp]
        L.go_matmul_transb_fp16.argtypes = [_f32p, _u16p, _f32p, _int, _int, _int]
        L.go_matvec_q4k.argtypes = [_f32p, _u8p, _f32p, _int, _int, _int]
        L.go_block_manager_new.argtypes = [_int, _int]
        L.go_block_manager_delete.argtypes = [_vp]
        L.go_block_manager_allocate.restype = _int
        L.go_block_manager_allocate.argtypes = [_vp]
        L.go_block_manager_free.argtypes = [_vp, _int]
        L.go_block_manager_num_free.restype = _int
        L.go_block_manager_num_free.argtypes = [_vp]
        L.go_paged_cache_new.restype = _vp
        L.go_paged_cache_new.argtypes = [_vp]
        L.go_paged_cache_delete.argtypes = [_vp]
        L.go_paged_cache_append_tokens.restype = _int
        L.go_paged_cache_append_tokens.argtypes = [_vp, _int]
        L.go_paged_cache_truncate.argtypes = [_vp, _int]
        L.go_paged_cache_release.argtypes = [_vp]
        L.go_paged_cache_seq_len.restype = _int
        L.go_paged_cache_seq_len.argtypes = [_vp]
        L.go_paged_cache_num_blocks.restype = _int
        L.go_paged_cache_num_blocks.argtypes = [_vp]
        L.go_paged_cache_table.restype = C.POINTER(C.c_int)
        L.go_paged_cache_table.argtypes = [_vp]
        L.go_paged_cache_physical_block.restype = _int
        L.go_paged_cache_physical_block.argtypes = [_vp, _int]
        L.go_paged_cache_block_offset.restype = _int
        L.go_paged_cache_block_offset.argtypes = [_vp, _int]

    # ---- conversions
    def fp16_to_fp32(self, h: np.ndarray) -> np.ndarray:
        h = np.ascontiguousarray(h, dtype=np.uint16)
        out = np.empty(h.shape, dtype=np.float32)
        self.lib.go_fp16_to_fp32_array(h.reshape(-1), out.reshape(-1), h.size)
        return out

    def fp32_to_fp16(self, f: np.ndarray) -> np.ndarray:
        f = np.ascontiguousarray(f, dtype=np.float32)
        out = np.empty(f.shape, dtype=np.uint16)
        self.lib.go_fp32_to_fp16_array(f.reshape(-1), out.reshape(-1), f.size)
        return out

    # ---- attention
    def attention_core(self, q, k_all, v_all, start_pos, scale, want_lse=True):
        """q [B,Sq,Hq,D] f32; k_all/v_all [T,Hkv,D] f32 -> ctx [B,Sq,Hq,D], lse [B,Hq,Sq]."""
        q = np.ascontiguousarray(q, np.float32)
        k_all = np.ascontiguousarray(k_all, np.float32)
        v_all = np.ascontiguousarray(v_all, np.float32)
        B, Sq, Hq, D = q.shape
        T, Hkv, _ = k_all.shape
        ctx = np.empty((B, Sq, Hq, D), np.float32)
        lse = np.empty((B, Hq, Sq), np.float32) if want_lse else None
        self.lib.go_attention_core(q, k_all, v_all, ctx, _opt(lse), B, Sq, Hq, Hkv, D, T,
                                   start_pos, scale)
        return ctx, lse

    def attention_cached(self, q, cache_k, cache_v, total_seq, start_pos, scale, want_lse=True):
        """cache_k/v [Hkv,max_seq,D] half bits."""
        q = np.ascontiguousarray(q, np.float32)
        ck = np.ascontiguousarray(cache_k).view(np.uint16)
        cv = np.ascontiguousarray(cache_v).view(np.uint16)
        B, Sq, Hq, D = q.shape
        Hkv, max_seq, _ = ck.shape
        ctx = np.empty((B, Sq, Hq, D), np.float32)
        lse = np.empty((B, Hq, Sq), np.float32) if want_lse else None
        self.lib.go_attention_cached(q, ck, cv, ctx, _opt(lse), B, Sq, Hq, Hkv, D, total_seq,
                                     max_seq, start_pos, scale)
        return ctx, lse

    def attention_paged(self, q, pool_k, pool_v, table, block_size, total_seq, start_pos, scale,
                        want_lse=True):
        q = np.ascontiguousarray(q, np.float32)
        pk = np.ascontiguousarray(pool_k).view(np.uint16)
        pv = np.ascontiguousarray(pool_v).view(np.uint16)
        table = np.ascontiguousarray(table, np.int32)
        B, Sq, Hq, D = q.shape
        Hkv = pk.shape[1]
        ctx = np.empty((B, Sq, Hq, D), np.float32)
        lse = np.empty((B, Hq, Sq), np.float32) if want_lse else None
        self.lib.go_attention_paged(q, pk, pv, table, block_size, ctx, _opt(lse), B, Sq, Hq, Hkv,
                                    D, total_seq, start_pos, scale)
        return ctx, lse

    def batched_paged_decode(self, q, pool_k, pool_v, tables, seq_lens, block_size, scale):
        q = np.ascontiguousarray(q, np.float32)
        pk = np.ascontiguousarray(pool_k).view(np.uint16)
        pv = np.ascontiguousarray(pool_v).view(np.uint16)
        tables = np.ascontiguousarray(tables, np.int32)
        seq_lens = np.ascontiguousarray(seq_lens, np.int32)
        B, Hq, D = q.shape
        Hkv = pk.shape[1]
        out = np.zeros((B, Hq, D), np.float32)
        lse = np.zeros((B, Hq), np.float32)
        self.lib.go_batched_paged_decode(q, pk, pv, tables, seq_lens, out, _opt(lse), B, Hq, Hkv,
                                         D, block_size, tables.shape[1], scale)
        return out, lse

    def rope_table(self, max_seq_len: int, head_dim: int, theta: float = 10000.0):
        """(cos, sin), each [max_seq_len, head_dim // 2] float32 (RoPECache::initialize)."""
        cos = np.zeros((max_seq_len, head_dim // 2), np.float32)
        sin = np.zeros((max_seq_len, head_dim // 2), np.float32)
        self.lib.go_rope_table(cos, sin, max_seq_len, head_dim, theta)
        return cos, sin

    def rope_apply(self, x: np.ndarray, start_pos: int, cos: np.ndarray, sin: np.ndarray) -> np.ndarray:
        """Rotated copy of x [seq, heads, D] float32 (RoPECache::apply); raises on its range error."""
        out = np.ascontiguousarray(x, np.float32).copy()
        seq, heads, d = out.shape
        rc = self.lib.go_rope_apply(out, seq, heads, d, start_pos, np.ascontiguousarray(cos),
                                    np.ascontiguousarray(sin), cos.shape[0])
        if rc != 0:
            raise ValueError("RoPE position out of range")
        return out

    # ---- Q4_K weights and projections
    def q4k_dequantize(self, blocks: np.ndarray):
        """blocks [..., 144] uint8 -> (float32 weights, what the reference stores: half bits)."""
        blocks = np.ascontiguousarray(blocks, np.uint8)
        numel = blocks.size // 144 * 256
        w32, w16 = np.empty(numel, np.float32), np.empty(numel, np.uint16)
        self.lib.go_q4k_dequantize(blocks.reshape(-1), numel, _opt(w32), _opt(w16))
        return w32, w16

    def matvec_q4k(self, x: np.ndarray, w_blocks: np.ndarray) -> np.ndarray:
        """x [batch, K] float32, w_blocks [N, K/256, 144] -> y [batch, N] float32."""
        x = np.ascontiguousarray(x, np.float32)
        w = np.ascontiguousarray(w_blocks, np.uint8)
        batch, K = x.shape
        N = w.shape[0]
        y = np.empty((batch, N), np.float32)
        self.lib.go_matvec_q4k(x, w.reshape(-1), y, K, N, batch)
        return y

    def matmul_transb_fp16(self, a: np.ndarray, b_half_bits: np.ndarray) -> np.ndarray:
        """a [M, K] float32, b [N, K] half bits -> a @ b.T (the CPU path's projection)."""
        a = np.ascontiguousarray(a, np.float32)
        b = np.ascontiguousarray(b_half_bits, np.uint16)
        M, K = a.shape
        N = b.shape[0]
        c = np.empty((M, N), np.float32)
        self.lib.go_matmul_transb_fp16(a, b, c, M, N, K)
        return c

    def tree_mask(self, parents) -> np.ndarray:
        parents = np.ascontiguousarray(parents, np.int32)
        n = parents.shape[0]
        mask = np.zeros((n, n), np.uint8)
        rc = self.lib.go_tree_mask(parents, n, mask.reshape(-1))
        if rc != 0:
            raise ValueError("parent index out of range")
        return mask

    def attention_tree(self, q, cache_k, cache_v, k_tree, v_tree, parents, cached_len, scale,
                       table=None, block_size=1, max_seq=0):
        """q [B,N,Hq,D] f32; k_tree/v_tree [B,N,Hkv,D] f32; cache contiguous
        [Hkv,max_seq,D] or paged [rows,Hkv,D] half bits."""
        q = np.ascontiguousarray(q, np.float32)
        k_tree = np.ascontiguousarray(k_tree, np.float32)
        v_tree = np.ascontiguousarray(v_tree, np.float32)
        parents = np.ascontiguousarray(parents, np.int32)
        B, N, Hq, D = q.shape
        Hkv = k_tree.shape[2]
        ck = None if cache_k is None else np.ascontiguousarray(cache_k).view(np.uint16)
        cv = None if cache_v is None else np.ascontiguousarray(cache_v).view(np.uint16)
        tb = None if table is None else np.ascontiguousarray(table, np.int32)
        ctx = np.empty((B, N, Hq, D), np.float32)
        lse = np.empty((B, Hq, N), np.float32)
        rc = self.lib.go_attention_tree(q, _opt(ck), _opt(cv), _opt(tb), block_size, max_seq,
                                        k_tree, v_tree, parents, ctx, _opt(lse), B, N, Hq, Hkv, D,
                                        cached_len, scale)
        if rc != 0:
            raise ValueError("parent index out of range")
        return ctx, lse


_oracle = None


def load() -> Oracle:
    global _oracle
    if _oracle is None:
        if not ORACLE_SO.exists():
            subprocess.run(["make", "-C", str(ROOT / "oracle"), "libgranite_oracle.so"], check=True)
        _oracle = Oracle(C.CDLL(str(ORACLE_SO)))
    return _oracle


def load_ref():
    """The reference's own math_ops.cpp, when oracle/_ref was built; else None."""
    if not REF_SO.exists():
        return None
    lib = C.CDLL(str(REF_SO))
    lib.ref_fp16_to_fp32.restype = _flt
    lib.ref_fp16_to_fp32.argtypes = [C.c_uint16]
    lib.ref_fp32_to_fp16.restype = C.c_uint16
    lib.ref_fp32_to_fp16.argtypes = [_flt]
    lib.ref_fp16_to_fp32_array.argtypes = [_u16p, _f32p, C.c_size_t]
    lib.ref_get_num_threads.restype = C.c_size_t
    lib.ref_parallel_for_owner.argtypes = [C.c_size_t, C.c_size_t, _i32p]
    lib.ref_parallel_for_count.restype = C.c_size_t
    lib.ref_parallel_for_count.argtypes = [C.c_size_t, C.c_size_t, _u8p]
    lib.ref_matmul_transb_fp16.argtypes = [_f32p, _u16p, _f32p, _int, _int, _int]
    return lib
