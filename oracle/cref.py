"""ctypes access to the scalar C restatement (oracle/c/tdist_oracle.c). Test infrastructure only."""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "_build", "libtdist_oracle.so")
_lib = None


def build(force=False):
    src = os.path.join(_HERE, "c", "tdist_oracle.c")
    if force or not os.path.exists(LIB_PATH) or os.path.getmtime(src) > os.path.getmtime(LIB_PATH):
        subprocess.run(["make", "-C", _HERE] + (["-B"] if force else []), check=True, stdout=subprocess.DEVNULL)
    return LIB_PATH


def load():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            build()
        _lib = ctypes.CDLL(LIB_PATH)
        _lib.oc_e4m3_to_f32.restype = ctypes.c_float
        _lib.oc_e4m3_to_f32.argtypes = [ctypes.c_uint8]
        _lib.oc_post_process.restype = ctypes.c_int64
    return _lib


def _p(a):
    return None if a is None else a.ctypes.data_as(ctypes.c_void_p)


def _c(a, dtype):
    return None if a is None else np.ascontiguousarray(a, dtype=dtype)


def e4m3_table():
    out = np.empty(256, dtype=np.float32)
    load().oc_e4m3_table(_p(out))
    return out


def reduce_slices_bf16(c_u16, first):
    """c_u16: uint16 [R, n] (bf16 bit patterns). Returns uint16 [n]."""
    c_u16 = _c(c_u16, np.uint16)
    R, n = c_u16.shape
    out = np.empty(n, dtype=np.uint16)
    load().oc_reduce_slices_bf16(_p(c_u16), ctypes.c_int64(n), ctypes.c_int(R), ctypes.c_int(first), ctypes.c_int64(n),
                                 _p(out))
    return out


def gemm_nt_f64(a_f32, b_f32):
    a_f32, b_f32 = _c(a_f32, np.float32), _c(b_f32, np.float32)
    M, K = a_f32.shape
    N = b_f32.shape[0]
    out = np.empty((M, N), dtype=np.float64)
    load().oc_gemm_nt_f64(_p(a_f32), _p(b_f32), _p(out), ctypes.c_int(M), ctypes.c_int(N), ctypes.c_int(K))
    return out


def gemm_e4m3_nt_f64(a_u8, b_u8, row_scale, col_scale):
    a_u8, b_u8 = _c(a_u8, np.uint8), _c(b_u8, np.uint8)
    rs, cs = _c(row_scale, np.float32), _c(col_scale, np.float32)
    M, K = a_u8.shape
    N = b_u8.shape[0]
    out = np.empty((M, N), dtype=np.float64)
    load().oc_gemm_e4m3_nt_f64(_p(a_u8), _p(b_u8), _p(rs), _p(cs), _p(out), ctypes.c_int(M), ctypes.c_int(N),
                               ctypes.c_int(K))
    return out


def moe_preprocess(ids_i32, topk, num_experts):
    ids = _c(ids_i32, np.int32).reshape(-1)
    n = ids.size
    splits = np.empty(num_experts, dtype=np.int32)
    cumsum = np.empty(num_experts + 1, dtype=np.int32)
    scatter = np.empty(n, dtype=np.int32)
    gather = np.empty(n, dtype=np.int32)
    topk_idx = np.empty(n, dtype=np.int32)
    load().oc_moe_preprocess(_p(ids), ctypes.c_int64(n), ctypes.c_int(topk), ctypes.c_int(num_experts), _p(splits),
                             _p(cumsum), _p(scatter), _p(gather), _p(topk_idx))
    return splits, cumsum, scatter.reshape(-1, topk), gather, topk_idx


def dispatch_slots(rows_u8, scales, gather_idx, cumsum, W, Er, max_m, fill_byte=0):
    rows_u8 = _c(rows_u8, np.uint8)
    row_bytes = rows_u8.shape[1]
    sc = _c(scales, np.float32)
    gi = _c(gather_idx, np.int32)
    cs = _c(cumsum, np.int32)
    slot_rows = np.full((W * max_m, row_bytes), fill_byte, dtype=np.uint8)
    slot_scales = np.zeros(W * max_m, dtype=np.float32) if sc is not None else None
    splits = np.empty(W * Er, dtype=np.int32)
    load().oc_dispatch_slots(_p(rows_u8), ctypes.c_int64(row_bytes), _p(sc), _p(gi), _p(cs), ctypes.c_int(W),
                             ctypes.c_int(Er), ctypes.c_int(max_m), _p(slot_rows), _p(slot_scales), _p(splits))
    return splits, slot_rows, slot_scales


def post_process(slot_rows_u8, slot_scales, splits, W, Er, max_m):
    slot_rows_u8 = _c(slot_rows_u8, np.uint8)
    row_bytes = slot_rows_u8.shape[1]
    sp = _c(splits, np.int32)
    total = int(sp.sum())
    sc = _c(slot_scales, np.float32)
    out_rows = np.empty((total, row_bytes), dtype=np.uint8)
    out_scales = np.empty(total, dtype=np.float32) if sc is not None else None
    n = load().oc_post_process(_p(slot_rows_u8), ctypes.c_int64(row_bytes), _p(sc), _p(sp), ctypes.c_int(W),
                               ctypes.c_int(Er), ctypes.c_int(max_m), _p(out_rows), _p(out_scales))
    assert n == total
    return out_rows, out_scales


def combine_e4m3(sorted_rows_u8, sorted_scales, scatter_idx, topk_w):
    rows = _c(sorted_rows_u8, np.uint8)
    H = rows.shape[1]
    si = _c(scatter_idx, np.int32)
    T, topk = si.shape
    sc, w = _c(sorted_scales, np.float32), _c(topk_w, np.float32)
    out = np.empty((T, H), dtype=np.float32)
    load().oc_combine_e4m3(_p(rows), _p(sc), _p(si), _p(w), ctypes.c_int64(T), ctypes.c_int(topk), ctypes.c_int(H),
                           _p(out))
    return out


def decode_range(q_f32, k_cache_f32, v_cache_f32, table_i32, lo, hi, scale, soft_cap=0.0):
    q, k, v = _c(q_f32, np.float32), _c(k_cache_f32, np.float32), _c(v_cache_f32, np.float32)
    tb = _c(table_i32, np.int32)
    lo, hi = _c(lo, np.int32), _c(hi, np.int32)
    B, Hq, D = q.shape
    _, page_size, Hkv, _ = k.shape
    Dv = v.shape[-1]
    out = np.empty((B, Hq, Dv), dtype=np.float64)
    lse = np.empty((B, Hq), dtype=np.float64)
    load().oc_decode_range(_p(q), _p(k), _p(v), _p(tb), ctypes.c_int64(tb.shape[1]), _p(lo), _p(hi), ctypes.c_int(B),
                           ctypes.c_int(Hq), ctypes.c_int(Hkv), ctypes.c_int(D), ctypes.c_int(Dv), ctypes.c_int(page_size),
                           ctypes.c_double(scale), ctypes.c_double(soft_cap), _p(out), _p(lse))
    return out, lse
