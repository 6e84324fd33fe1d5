"""CPU oracle of the sparse-decode path — TEST INFRASTRUCTURE, not part of the product.

Thin ctypes/numpy front end of ``tka_oracle.c``.  Only tests, the smoke check and the CPU leg of the
benchmark may import this package; the shipped library never does.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "_build", "libtka_oracle.so")

F16, BF16 = 0, 1


def build(force=False):
    """Compile tka_oracle.c with gcc (seconds)."""
    if force or not os.path.exists(_SO) or os.path.getmtime(_SO) < os.path.getmtime(
            os.path.join(_HERE, "tka_oracle.c")):
        subprocess.check_call(["make", "-s", "-B", "-C", _HERE])
    return _SO


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        L = ctypes.CDLL(_SO)
        c_i, c_i64, c_f, c_d, c_p = ctypes.c_int, ctypes.c_int64, ctypes.c_float, ctypes.c_double, ctypes.c_void_p
        L.orc_half_to_float.restype = c_f
        L.orc_half_to_float.argtypes = [ctypes.c_uint16]
        L.orc_bf16_to_float.restype = c_f
        L.orc_bf16_to_float.argtypes = [ctypes.c_uint16]
        L.orc_score_key.restype = ctypes.c_uint32
        L.orc_score_key.argtypes = [c_f]
        L.orc_key_score.restype = c_f
        L.orc_key_score.argtypes = [ctypes.c_uint32]
        L.orc_group_query.restype = None
        L.orc_group_query.argtypes = [c_p, c_i, c_i, c_p]
        L.orc_scores_canonical.restype = None
        L.orc_scores_canonical.argtypes = [c_p, c_i, c_i64, c_i64, c_p, c_f, c_p]
        L.orc_scores_f64.restype = None
        L.orc_scores_f64.argtypes = [c_p, c_i, c_i64, c_i64, c_p, c_i, c_d, c_p]
        L.orc_topk_stable.restype = c_i
        L.orc_topk_stable.argtypes = [c_p, c_i64, c_i, c_p, c_p]
        L.orc_center_expand.restype = None
        L.orc_center_expand.argtypes = [c_p, c_i, c_i, c_p]
        L.orc_center_topk_expand.restype = c_i
        L.orc_center_topk_expand.argtypes = [c_p, c_p, c_i, c_i, c_i, c_i, c_f, c_p, c_p, c_p]
        L.orc_cluster_topk.restype = c_i
        L.orc_cluster_topk.argtypes = [c_p, c_p, c_p, c_i, c_i, c_i, c_i, c_i, c_i64, c_f, c_p]
        L.orc_index_union.restype = c_i
        L.orc_index_union.argtypes = [c_p, c_i, c_i, c_i, c_i64, c_p]
        L.orc_attention_f64.restype = None
        L.orc_attention_f64.argtypes = [c_p, c_p, c_p, c_i, c_i64, c_p, c_i64, c_p, c_d, c_p, c_p]
        L.orc_lse_combine.restype = None
        L.orc_lse_combine.argtypes = [c_p, c_p, c_p, c_i, c_p, c_p]
        L.orc_retrieval_attention.restype = c_i
        L.orc_retrieval_attention.argtypes = [c_p, c_p, c_p, c_i, c_i64, c_i64, c_i, c_i, c_f, c_p, c_p, c_p]
        L.orc_sparse_decode_step.restype = c_i
        L.orc_sparse_decode_step.argtypes = [c_p, c_p, c_p, c_i, c_i, c_i64, c_i64, c_i, c_i, c_i, c_f,
                                             c_p, c_p, c_p, c_p]
        _lib = L
    return _lib


# ---- helpers: 16-bit element arrays are carried as numpy uint16 bit patterns ---------------------

def to_bits(x, dtype):
    """float array -> uint16 bit patterns of fp16 (round-to-nearest-even) or bf16 (RNE)."""
    x = np.asarray(x)
    if dtype == F16:
        return np.ascontiguousarray(x.astype(np.float16)).view(np.uint16)
    u = np.ascontiguousarray(x.astype(np.float32)).view(np.uint32)
    rounded = u + 0x7FFF + ((u >> 16) & 1)
    return (rounded >> 16).astype(np.uint16)


def from_bits(b, dtype):
    b = np.asarray(b, dtype=np.uint16)
    if dtype == F16:
        return b.view(np.float16).astype(np.float32)
    return (b.astype(np.uint32) << 16).view(np.float32)


def _p(a):
    return a.ctypes.data_as(ctypes.c_void_p) if a is not None else None


def _c16(a):
    a = np.ascontiguousarray(a)
    assert a.dtype == np.uint16
    return a


def group_query(q_bits, dtype, group):
    """q_bits [group,128] -> fp32 [128] summed query."""
    q_bits = _c16(q_bits)
    out = np.empty(128, np.float32)
    lib().orc_group_query(_p(q_bits), dtype, group, _p(out))
    return out


def scores_canonical(keys_bits, dtype, qf, scale=1.0):
    """keys_bits [n,128] (any row stride, last dim contiguous) -> fp32 [n] canonical scores."""
    assert keys_bits.dtype == np.uint16 and keys_bits.ndim == 2 and keys_bits.shape[1] == 128
    assert keys_bits.strides[1] == 2 and keys_bits.strides[0] % 2 == 0
    n = keys_bits.shape[0]
    qf = np.ascontiguousarray(qf, np.float32)
    out = np.empty(n, np.float32)
    lib().orc_scores_canonical(keys_bits.ctypes.data, dtype, n, keys_bits.strides[0] // 2, _p(qf),
                               np.float32(scale), _p(out))
    return out


def scores_f64(keys_bits, dtype, q_bits, scale=1.0):
    assert keys_bits.dtype == np.uint16 and keys_bits.ndim == 2 and keys_bits.shape[1] == 128
    assert keys_bits.strides[1] == 2
    q_bits = _c16(q_bits).reshape(-1, 128)
    n = keys_bits.shape[0]
    out = np.empty(n, np.float64)
    lib().orc_scores_f64(keys_bits.ctypes.data, dtype, n, keys_bits.strides[0] // 2, _p(q_bits),
                         q_bits.shape[0], float(scale), _p(out))
    return out


def topk_stable(scores, k):
    scores = np.ascontiguousarray(scores, np.float32)
    idx = np.empty(k, np.int32)
    val = np.empty(k, np.float32)
    rc = lib().orc_topk_stable(_p(scores), scores.shape[0], k, _p(idx), _p(val))
    if rc != 0:
        raise ValueError("bad k")
    return idx, val


def score_keys(scores):
    """Vectorised orc_score_key (numpy) — used by tests to pin the C version."""
    x = np.asarray(scores, np.float32)
    x = np.where(x == 0, np.float32(0.0), x)
    u = x.view(np.uint32)
    key = np.where(u & 0x80000000, ~u, u | np.uint32(0x80000000)).astype(np.uint32)
    return np.where(np.isnan(x), np.uint32(0), key)


def center_topk_expand(q_bits, centers_bits, dtype, top_c, cluster_len, scale=1.0):
    q_bits, centers_bits = _c16(q_bits), _c16(centers_bits)
    nc = centers_bits.shape[0]
    out = np.empty(top_c * cluster_len, np.int32)
    cen = np.empty(top_c, np.int32)
    val = np.empty(top_c, np.float32)
    rc = lib().orc_center_topk_expand(_p(q_bits), _p(centers_bits), dtype, nc, top_c, cluster_len,
                                      np.float32(scale), _p(out), _p(cen), _p(val))
    if rc != 0:
        raise ValueError("bad top_c")
    return out, cen, val


def cluster_topk(q_bits, centers_bits, keys_bits, dtype, top_c, cluster_len, k, scale=1.0):
    """keys_bits [num_centers*cluster_len, 128] view with arbitrary row stride."""
    q_bits, centers_bits = _c16(q_bits), _c16(centers_bits)
    assert keys_bits.strides[1] == 2
    out = np.empty(top_c * k, np.int32)
    rc = lib().orc_cluster_topk(_p(q_bits), _p(centers_bits), keys_bits.ctypes.data, dtype,
                                centers_bits.shape[0], top_c, cluster_len, k, keys_bits.strides[0] // 2,
                                np.float32(scale), _p(out))
    if rc != 0:
        raise ValueError("bad sizes")
    return out


def index_union(ids, sink, local, n):
    ids = np.ascontiguousarray(ids, np.int32)
    out = np.full(ids.shape[0] + sink + local, -1, np.int32)
    cnt = lib().orc_index_union(_p(ids), ids.shape[0], sink, local, n, _p(out))
    return out, cnt


def attention_f64(q_bits, keys_bits, values_bits, dtype, idx=None, count=None, logit=None, scale=1.0):
    """One query head [128]; keys/values [n,128] views sharing one row stride. Returns (out[128], lse)."""
    q_bits = _c16(q_bits)
    assert keys_bits.strides == values_bits.strides and keys_bits.strides[1] == 2
    if idx is not None:
        idx = np.ascontiguousarray(idx, np.int32)
        if count is None:
            count = idx.shape[0]
    elif count is None:
        count = keys_bits.shape[0]
    if logit is not None:
        logit = np.ascontiguousarray(logit, np.float32)
    out = np.empty(128, np.float64)
    lse = ctypes.c_double()
    lib().orc_attention_f64(_p(q_bits), keys_bits.ctypes.data, values_bits.ctypes.data, dtype,
                            keys_bits.strides[0] // 2, _p(idx), count, _p(logit), float(scale), _p(out),
                            ctypes.byref(lse))
    return out, lse.value


def lse_combine(m, l, acc):
    m = np.ascontiguousarray(m, np.float32)
    l = np.ascontiguousarray(l, np.float32)
    acc = np.ascontiguousarray(acc, np.float32)
    out = np.empty(128, np.float64)
    lse = ctypes.c_double()
    lib().orc_lse_combine(_p(m), _p(l), _p(acc), m.shape[0], _p(out), ctypes.byref(lse))
    return out, lse.value


def retrieval_attention(q_bits, keys_bits, values_bits, dtype, num_chunks, k, scale=1.0):
    """One (batch entry, head). keys/values [seq_len,128] strided views. Returns (out, idx, val)."""
    q_bits = _c16(q_bits)
    assert keys_bits.strides == values_bits.strides and keys_bits.strides[1] == 2
    n = keys_bits.shape[0]
    out = np.empty(128, np.float64)
    idx = np.empty(num_chunks * k, np.int32)
    val = np.empty(num_chunks * k, np.float32)
    rc = lib().orc_retrieval_attention(_p(q_bits), keys_bits.ctypes.data, values_bits.ctypes.data, dtype, n,
                                       keys_bits.strides[0] // 2, num_chunks, k, np.float32(scale), _p(out),
                                       _p(idx), _p(val))
    if rc != 0:
        raise ValueError("bad sizes")
    return out, idx, val


def sparse_decode_step(q_bits, keys_bits, values_bits, dtype, group, k, sink, local, scale):
    """One (batch entry, KV head). q_bits [group,128]. Returns (out[group,128], topk_idx, topk_val, union)."""
    q_bits = _c16(q_bits)
    assert keys_bits.strides == values_bits.strides and keys_bits.strides[1] == 2
    n = keys_bits.shape[0]
    out = np.empty((group, 128), np.float64)
    tidx = np.empty(k, np.int32)
    tval = np.empty(k, np.float32)
    uni = np.full(k + sink + local, -1, np.int32)
    cnt = lib().orc_sparse_decode_step(_p(q_bits), keys_bits.ctypes.data, values_bits.ctypes.data, dtype, group,
                                       n, keys_bits.strides[0] // 2, k, sink, local, np.float32(scale), _p(out),
                                       _p(tidx), _p(tval), _p(uni))
    if cnt < 0:
        raise ValueError("bad sizes")
    return out, tidx, tval, uni[:cnt]
