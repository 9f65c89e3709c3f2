"""ctypes binding of oracle/libuv_oracle.so (checker only)."""
from __future__ import annotations

import ctypes as C
import os

import numpy as np

from .build import LIB, build

_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB):
            build()
        _lib = C.CDLL(LIB)
        _lib.uvo_h2f.restype = C.c_float
        _lib.uvo_h2f.argtypes = [C.c_uint16]
        _lib.uvo_f2h.restype = C.c_uint16
        _lib.uvo_f2h.argtypes = [C.c_float]
    return _lib


def _p(a):
    return a.ctypes.data_as(C.c_void_p)


def quantize_rows(x: np.ndarray):
    x = np.ascontiguousarray(x, dtype=np.float32)
    hd = x.shape[-1]
    n = x.size // hd
    q = np.empty(x.shape, dtype=np.int8)
    s = np.empty(x.shape[:-1], dtype=np.float16)
    lib().uvo_quantize_rows(_p(x), C.c_int64(n), C.c_int(hd), _p(q), _p(s))
    return q, s


def decode_attn_i8(q, kc, vc, ks, vs, pos, starts, scale, window=0, ring=None, rows=None):
    q = np.ascontiguousarray(q, dtype=np.float32)
    kc, vc = np.ascontiguousarray(kc), np.ascontiguousarray(vc)
    ks, vs = np.ascontiguousarray(ks, dtype=np.float16), np.ascontiguousarray(vs, dtype=np.float16)
    pos, starts = np.ascontiguousarray(pos, dtype=np.int64), np.ascontiguousarray(starts, dtype=np.int64)
    B, H, hd = q.shape
    KH, S = kc.shape[1], kc.shape[2]
    if ring is None:
        ring = window > 0
    out = np.zeros((B, H, hd), dtype=np.float32)
    b0, b1 = rows if rows is not None else (0, B)
    lib().uvo_decode_attn_i8(_p(q), _p(kc), _p(vc), _p(ks), _p(vs), _p(pos), _p(starts), _p(out), C.c_int(B), C.c_int(H),
                             C.c_int(KH), C.c_int(S), C.c_int(hd), C.c_float(scale), C.c_int(window), C.c_int(int(ring)),
                             C.c_int(b0), C.c_int(b1))
    return out


def fused_sample(x, u, sc, T):
    x = np.ascontiguousarray(x, dtype=np.float32)
    u = np.ascontiguousarray(u, dtype=np.float32)
    B, V = x.shape
    tok = np.empty(B, dtype=np.int64)
    lp = np.empty(B, dtype=np.float32)
    lib().uvo_fused_sample(_p(x), _p(u), C.c_int(B), C.c_int(V), C.c_float(sc[0]), C.c_float(sc[1]), C.c_float(sc[2]),
                           C.c_float(T), _p(tok), _p(lp))
    return tok, lp


def philox(ctr, key):
    c = np.asarray(ctr, dtype=np.uint32)
    k = np.asarray(key, dtype=np.uint32)
    o = np.empty(4, dtype=np.uint32)
    lib().uvo_philox4x32_10(_p(c), _p(k), _p(o))
    return o
