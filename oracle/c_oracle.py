"""ctypes view of the scalar C restatement (oracle/kvx_oracle.c). TEST INFRASTRUCTURE ONLY."""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libkvx_oracle.so")


def build(force: bool = False) -> str:
    if force or not os.path.exists(_SO):
        subprocess.check_call(["make", "-C", _HERE, "-B" if force else "-s"])
    return _SO


def _lib():
    lib = ctypes.CDLL(build())
    return lib


def _p(a, t):
    return a.ctypes.data_as(ctypes.POINTER(t))


def quantize_rows(x: np.ndarray):
    x = np.ascontiguousarray(x, dtype=np.float32)
    rows, D = x.shape
    codes = np.empty((rows, D), np.uint8)
    scale = np.empty(rows, np.float32)
    zp = np.empty(rows, np.int32)
    _lib().kvxo_quantize_rows(_p(x, ctypes.c_float), ctypes.c_int64(rows), ctypes.c_int32(D),
                              _p(codes, ctypes.c_uint8), _p(scale, ctypes.c_float), _p(zp, ctypes.c_int32))
    return codes, scale, zp


def dequantize_rows(codes: np.ndarray, scale: np.ndarray, zp: np.ndarray):
    codes = np.ascontiguousarray(codes, dtype=np.uint8)
    scale = np.ascontiguousarray(scale, dtype=np.float32)
    zp = np.ascontiguousarray(zp, dtype=np.int32)
    rows, D = codes.shape
    out = np.empty((rows, D), np.float32)
    _lib().kvxo_dequantize_rows(_p(codes, ctypes.c_uint8), _p(scale, ctypes.c_float), _p(zp, ctypes.c_int32),
                                ctypes.c_int64(rows), ctypes.c_int32(D), _p(out, ctypes.c_float))
    return out


def quantize_blocks4(x: np.ndarray):
    x = np.ascontiguousarray(x, dtype=np.float32)
    blocks, E = x.shape
    packed = np.empty((blocks, E // 2), np.uint8)
    scale = np.empty(blocks, np.float32)
    zp = np.empty(blocks, np.int32)
    _lib().kvxo_quantize_blocks4(_p(x, ctypes.c_float), ctypes.c_int64(blocks), ctypes.c_int32(E),
                                 _p(packed, ctypes.c_uint8), _p(scale, ctypes.c_float), _p(zp, ctypes.c_int32))
    return packed, scale, zp


def dequantize_blocks4(packed: np.ndarray, scale: np.ndarray, zp: np.ndarray):
    packed = np.ascontiguousarray(packed, dtype=np.uint8)
    scale = np.ascontiguousarray(scale, dtype=np.float32)
    zp = np.ascontiguousarray(zp, dtype=np.int32)
    blocks, half = packed.shape
    out = np.empty((blocks, 2 * half), np.float32)
    _lib().kvxo_dequantize_blocks4(_p(packed, ctypes.c_uint8), _p(scale, ctypes.c_float), _p(zp, ctypes.c_int32),
                                   ctypes.c_int64(blocks), ctypes.c_int32(2 * half), _p(out, ctypes.c_float))
    return out


def sdpa_weights(q, k, v, tp, input_pos, scale):
    q = np.ascontiguousarray(q, dtype=np.float32)
    k = np.ascontiguousarray(k, dtype=np.float32)
    v = np.ascontiguousarray(v, dtype=np.float32)
    B, Hq, q_len, D = q.shape
    Hkv, T = k.shape[1], k.shape[2]
    tp_p = None
    if tp is not None:
        tp = np.ascontiguousarray(np.broadcast_to(tp, (B, Hkv, T)), dtype=np.int32)
        tp_p = _p(tp, ctypes.c_int32)
    o = np.empty((B, Hq, q_len, D), np.float32)
    w = np.empty((B, Hkv, T), np.float32)
    lse = np.empty((B, q_len, Hq), np.float32)
    _lib().kvxo_sdpa_weights(_p(q, ctypes.c_float), _p(k, ctypes.c_float), _p(v, ctypes.c_float), tp_p,
                             ctypes.c_int32(B), ctypes.c_int32(Hq), ctypes.c_int32(Hkv), ctypes.c_int32(q_len),
                             ctypes.c_int32(T), ctypes.c_int32(D), ctypes.c_int32(input_pos), ctypes.c_float(scale),
                             _p(o, ctypes.c_float), _p(w, ctypes.c_float), _p(lse, ctypes.c_float))
    return o, w, lse


def h2o_update_select(scores, w, kv_len, limit, k):
    assert scores.dtype == np.float32 and scores.flags.c_contiguous
    B, Hkv, L = scores.shape
    w_p = None
    if w is not None:
        w = np.ascontiguousarray(w, dtype=np.float32)
        w_p = _p(w, ctypes.c_float)
    nxt = np.empty((B, Hkv, k), np.int32)
    _lib().kvxo_h2o_update_select(_p(scores, ctypes.c_float), w_p, ctypes.c_int32(B), ctypes.c_int32(Hkv),
                                  ctypes.c_int32(L), ctypes.c_int32(kv_len), ctypes.c_int32(limit),
                                  ctypes.c_int32(k), _p(nxt, ctypes.c_int32))
    return nxt
