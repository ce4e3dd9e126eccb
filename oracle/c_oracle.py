"""numpy-facing wrapper over liboracle.so (oracle/litekv_oracle.c). TEST INFRASTRUCTURE.

fp16 tensors travel as ``np.float16`` arrays (viewed as uint16 at the C
boundary); attention results come back as unrounded float32.
"""

from __future__ import annotations

import ctypes
from ctypes import c_float, c_int, c_int64, c_uint16, c_void_p

import numpy as np

from .build import LIB_PATH, build_oracle

_lib = None


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not LIB_PATH.exists():
            build_oracle()
        _lib = ctypes.CDLL(str(LIB_PATH))
        _lib.oracle_half_to_float.restype = c_float
        _lib.oracle_half_to_float.argtypes = [c_uint16]
    return _lib


def _h(a: np.ndarray) -> np.ndarray:
    a = np.ascontiguousarray(a)
    assert a.dtype == np.float16, a.dtype
    return a


def _i32(a) -> np.ndarray:
    return np.ascontiguousarray(np.asarray(a, dtype=np.int32))


def _p(a):
    return None if a is None else a.ctypes.data_as(c_void_p)


def half_to_float(bits: int) -> float:
    return float(lib().oracle_half_to_float(bits))


def kv_append(kv_values: np.ndarray, select_index, kv_buffer: np.ndarray) -> None:
    """In place: kv_buffer[select_index[i]] = kv_values[i]; arrays are [*, 2*Hkv, D] float16."""
    kv_values = _h(kv_values)
    assert kv_buffer.dtype == np.float16 and kv_buffer.flags.c_contiguous
    idx = _i32(select_index)
    row = int(np.prod(kv_buffer.shape[1:]))
    assert int(np.prod(kv_values.shape[1:])) == row
    f = lib().oracle_kv_append
    f.restype = None
    f.argtypes = [c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64]
    f(_p(kv_values), _p(idx), _p(kv_buffer), idx.shape[0], row, kv_buffer.shape[0])


def page_gather(src_pool: np.ndarray, dst_pool: np.ndarray, src_ids, dst_ids=None, page_size: int = 16) -> None:
    """In place: dst_pool[page dst_ids[i]] = src_pool[page src_ids[i]] (pools [slots, 2*Hkv, D])."""
    src_pool = _h(src_pool)
    assert dst_pool.dtype == np.float16 and dst_pool.flags.c_contiguous
    s = _i32(src_ids)
    d = None if dst_ids is None else _i32(dst_ids)
    page_elems = page_size * int(np.prod(src_pool.shape[1:]))
    f = lib().oracle_page_gather
    f.restype = None
    f.argtypes = [c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64, c_int64]
    f(_p(src_pool), _p(dst_pool), _p(s), _p(d), s.shape[0], page_elems,
      src_pool.shape[0] // page_size, dst_pool.shape[0] // page_size)


def paged_decode(q, pool, block_table, seq_lens, scale: float, page_size: int = 16, wide: bool = False,
                 return_lse: bool = False):
    """out float32 [B, Hq, D] of decode attention through the block table."""
    q, pool = _h(q), _h(pool)
    bt, sl = _i32(block_table), _i32(seq_lens)
    b, hq, d = q.shape
    hkv = pool.shape[1] // 2
    out = np.zeros((b, hq, d), dtype=np.float32)
    lse = np.zeros((b, hq), dtype=np.float32) if return_lse else None
    f = lib().oracle_paged_decode
    f.restype = None
    f.argtypes = [c_void_p, c_void_p, c_void_p, c_int64, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int,
                  c_int, c_int, c_float, c_int]
    f(_p(q), _p(pool), _p(bt), bt.shape[1], _p(sl), _p(out), _p(lse), b, hq, hkv, d, page_size, scale,
      int(wide))
    return (out, lse) if return_lse else out


def lse_merge(mid_o: np.ndarray, mid_lse: np.ndarray) -> np.ndarray:
    """Merge [n, D] partial outputs with [n] log-sum-exps in index order."""
    mid_o = np.ascontiguousarray(mid_o, dtype=np.float32)
    mid_lse = np.ascontiguousarray(mid_lse, dtype=np.float32)
    n, d = mid_o.shape
    out = np.zeros(d, dtype=np.float32)
    f = lib().oracle_lse_merge
    f.restype = None
    f.argtypes = [c_void_p, c_void_p, c_int, c_int, c_void_p]
    f(_p(mid_o), _p(mid_lse), n, d, _p(out))
    return out


def decode_partitioned(q, pool, block_table, seq_lens, scale: float, partition: int = 128, page_size: int = 16):
    """(out, mid_o, mid_lse) of the two-stage flash-decoding with fixed token partitions."""
    q, pool = _h(q), _h(pool)
    bt, sl = _i32(block_table), _i32(seq_lens)
    b, hq, d = q.shape
    hkv = pool.shape[1] // 2
    parts = max(1, (int(sl.max(initial=0)) + partition - 1) // partition)
    out = np.zeros((b, hq, d), dtype=np.float32)
    mid_o = np.zeros((b, hq, parts, d), dtype=np.float32)
    mid_lse = np.full((b, hq, parts), -np.inf, dtype=np.float32)
    f = lib().oracle_decode_partitioned
    f.restype = None
    f.argtypes = [c_void_p, c_void_p, c_void_p, c_int64, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int,
                  c_int, c_int, c_int, c_int, c_int, c_float]
    f(_p(q), _p(pool), _p(bt), bt.shape[1], _p(sl), _p(out), _p(mid_o), _p(mid_lse), b, hq, hkv, d, page_size,
      partition, parts, scale)
    return out, mid_o, mid_lse


def paged_prefill(q, pool, block_table, cu_q_lens, context_lens, scale: float, page_size: int = 16,
                  wide: bool = False) -> np.ndarray:
    """out float32 [T, Hq, D]: causal chunk attention over paged KV (history + chunk)."""
    q, pool = _h(q), _h(pool)
    bt, cu = _i32(block_table), _i32(cu_q_lens)
    ctx = None if context_lens is None else _i32(context_lens)
    t, hq, d = q.shape
    hkv = pool.shape[1] // 2
    out = np.zeros((t, hq, d), dtype=np.float32)
    f = lib().oracle_paged_prefill
    f.restype = None
    f.argtypes = [c_void_p, c_void_p, c_void_p, c_int64, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int,
                  c_int, c_int, c_float, c_int]
    f(_p(q), _p(pool), _p(bt), bt.shape[1], _p(cu), _p(ctx), _p(out), cu.shape[0] - 1, hq, hkv, d, page_size,
      scale, int(wide))
    return out


def varlen_prefill(q, k, v, seq_starts, seq_lens, scale: float, wide: bool = False) -> np.ndarray:
    """out float32 [T, Hq, D]: per-sequence causal attention over packed k, v [T, Hkv, D]."""
    q, k, v = _h(q), _h(k), _h(v)
    st, sl = _i32(seq_starts), _i32(seq_lens)
    t, hq, d = q.shape
    hkv = k.shape[1]
    out = np.zeros((t, hq, d), dtype=np.float32)
    f = lib().oracle_varlen_prefill
    f.restype = None
    f.argtypes = [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int,
                  c_float, c_int]
    f(_p(q), _p(k), _p(v), _p(st), _p(sl), _p(out), sl.shape[0], hq, hkv, d, scale, int(wide))
    return out
