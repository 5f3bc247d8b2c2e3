"""ctypes access to oracle/liboracle.so (C part of the CPU oracle).  TEST INFRASTRUCTURE ONLY."""
import ctypes
import os
import subprocess
from ctypes import c_float, c_int, c_int64, c_void_p

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_PATH = os.path.join(_HERE, "liboracle.so")


def build() -> str:
    subprocess.check_call(["make", "-C", _HERE, "-s", "-B"])
    return _PATH


def _load():
    if not os.path.exists(_PATH):
        build()
    lib = ctypes.CDLL(_PATH)
    lib.ref_k_elem_offset.restype = c_int64
    lib.ref_k_elem_offset.argtypes = [c_int64] * 7 + [c_int]
    lib.ref_v_elem_offset.restype = c_int64
    lib.ref_v_elem_offset.argtypes = [c_int64] * 7 + [c_int]
    lib.ref_apply_llama_rope.restype = None
    lib.ref_apply_llama_rope.argtypes = [c_void_p, c_int64, c_int64, c_float, c_float, c_void_p]
    lib.ref_single_mha.restype = None
    lib.ref_single_mha.argtypes = [c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64,
                                   c_int64, c_int, c_void_p]
    lib.ref_selected_single_mha.restype = None
    lib.ref_selected_single_mha.argtypes = [c_void_p, c_void_p, c_void_p, c_void_p, c_int64,
                                            c_int64, c_int64, c_int64, c_int64, c_int64, c_int,
                                            c_void_p]
    lib.ref_append_paged_kv_cache.restype = None
    lib.ref_append_paged_kv_cache.argtypes = [c_void_p, c_void_p, c_int64, c_void_p, c_void_p,
                                              c_int64, c_int64, c_int64, c_int64, c_int]
    lib.ref_stable_topk.restype = None
    lib.ref_stable_topk.argtypes = [c_void_p, c_int64, c_int64, c_int64, c_void_p]
    return lib


lib = _load()


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def _i32(a):
    return np.ascontiguousarray(a, dtype=np.int32)


def apply_llama_rope(x, offset, rope_scale=1.0, rope_theta=1e4):
    """x [D] -> rotated [D] (float32)."""
    x = _f32(x)
    out = np.empty_like(x)
    lib.ref_apply_llama_rope(x.ctypes.data, x.shape[0], int(offset), rope_scale, rope_theta,
                             out.ctypes.data)
    return out


def single_mha(q, k, v, layout=0):
    """q [Hq, D]; k, v [N, Hkv, D] (NHD) or [Hkv, N, D] (HND) -> o [Hq, D]."""
    q, k, v = _f32(q), _f32(k), _f32(v)
    hq, d = q.shape
    n, hkv = (k.shape[0], k.shape[1]) if layout == 0 else (k.shape[1], k.shape[0])
    o = np.empty((hq, d), dtype=np.float32)
    lib.ref_single_mha(q.ctypes.data, k.ctypes.data, v.ctypes.data, n, hq, hkv, d, layout,
                       o.ctypes.data)
    return o


def selected_single_mha(q, k, v, selected, last_len, page_size, layout=0):
    """selected [H, page_budget] logical pages, last column = partially filled last page."""
    q, k, v, selected = _f32(q), _f32(k), _f32(v), _i32(selected)
    h, d = q.shape
    n = k.shape[0] if layout == 0 else k.shape[1]
    o = np.empty((h, d), dtype=np.float32)
    lib.ref_selected_single_mha(q.ctypes.data, k.ctypes.data, v.ctypes.data, selected.ctypes.data,
                                selected.shape[1], int(last_len), n, int(page_size), h, d, layout,
                                o.ctypes.data)
    return o


def append_paged_kv_cache(pool, page_indices, seq_len, keys, values, layout=0):
    """pool float32 (modified in place), keys/values [n, H, D]."""
    assert pool.dtype == np.float32 and pool.flags["C_CONTIGUOUS"]
    keys, values, page_indices = _f32(keys), _f32(values), _i32(page_indices)
    n, h, d = keys.shape
    page_size = pool.shape[3] if layout == 1 else pool.shape[2]
    lib.ref_append_paged_kv_cache(pool.ctypes.data, page_indices.ctypes.data, int(seq_len),
                                  keys.ctypes.data, values.ctypes.data, n, h, page_size, d, layout)


def stable_topk(values, k):
    values = _f32(values)
    rows, n = values.shape
    k = min(int(k), n)
    out = np.empty((rows, k), dtype=np.int32)
    lib.ref_stable_topk(values.ctypes.data, rows, n, k, out.ctypes.data)
    return out
