"""ctypes front-end for oracle/brute_force.c (double precision loops). TEST INFRASTRUCTURE ONLY."""

from __future__ import annotations

import ctypes
import os
import subprocess
from typing import Optional

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libaxl_oracle.so")
_lib = None


def build(force: bool = False) -> str:
    """Compiles brute_force.c with gcc (via the Makefile next to it)."""
    if force and os.path.exists(_LIB_PATH):
        os.remove(_LIB_PATH)
    subprocess.run(["make", "-s", "-C", _HERE], check=True)
    return _LIB_PATH


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = ctypes.CDLL(_LIB_PATH)
    return _lib


def _p(a: Optional[np.ndarray], ctype):
    if a is None:
        return ctypes.POINTER(ctype)()
    return a.ctypes.data_as(ctypes.POINTER(ctype))


def _f64(a) -> np.ndarray:
    return np.ascontiguousarray(np.asarray(a, dtype=np.float64))


MASK_NONE, MASK_CAUSAL, MASK_SLIDING = 0, 1, 2


def attention_fwd(q, k, v, *, scale=1.0, mask_kind=MASK_NONE, window=0, segment_ids=None,
                  q_offset=None):
    """q [B,T,Hq,D], k/v [B,S,Hkv,D] -> (out [B,T,Hq,D], lse [B,Hq,T]) as float64 numpy."""
    q, k, v = _f64(q), _f64(k), _f64(v)
    b, t, hq, d = q.shape
    s, hkv = k.shape[1], k.shape[2]
    out = np.empty_like(q)
    lse = np.empty((b, hq, t), dtype=np.float64)
    seg = None if segment_ids is None else np.ascontiguousarray(segment_ids, dtype=np.int32)
    off = None if q_offset is None else np.ascontiguousarray(q_offset, dtype=np.int64)
    lib().axl_oracle_attention_fwd(
        _p(q, ctypes.c_double), _p(k, ctypes.c_double), _p(v, ctypes.c_double),
        _p(out, ctypes.c_double), _p(lse, ctypes.c_double), _p(seg, ctypes.c_int32),
        _p(off, ctypes.c_int64), b, t, s, hq, hkv, d, ctypes.c_double(scale), mask_kind,
        int(window))
    return out, lse


def attention_bwd(q, k, v, dout, *, scale=1.0, mask_kind=MASK_NONE, window=0, segment_ids=None,
                  q_offset=None):
    """Returns (dq, dk, dv) of sum(out * dout), float64 numpy."""
    q, k, v, dout = _f64(q), _f64(k), _f64(v), _f64(dout)
    b, t, hq, d = q.shape
    s, hkv = k.shape[1], k.shape[2]
    dq, dk, dv = np.empty_like(q), np.empty_like(k), np.empty_like(v)
    seg = None if segment_ids is None else np.ascontiguousarray(segment_ids, dtype=np.int32)
    off = None if q_offset is None else np.ascontiguousarray(q_offset, dtype=np.int64)
    lib().axl_oracle_attention_bwd(
        _p(q, ctypes.c_double), _p(k, ctypes.c_double), _p(v, ctypes.c_double),
        _p(dout, ctypes.c_double), _p(dq, ctypes.c_double), _p(dk, ctypes.c_double),
        _p(dv, ctypes.c_double), _p(seg, ctypes.c_int32), _p(off, ctypes.c_int64), b, t, s, hq,
        hkv, d, ctypes.c_double(scale), mask_kind, int(window))
    return dq, dk, dv


def paged_decode(q, kpool, vpool, page_tables, lengths, *, scale=1.0, window=-1):
    """q [B,Hq,D]; pools [Hkv,P,page,D]; page_tables [B,pps]; lengths [B] -> out [B,Hq,D]."""
    q, kpool, vpool = _f64(q), _f64(kpool), _f64(vpool)
    b, hq, d = q.shape
    hkv, p, page, _ = kpool.shape
    pt = np.ascontiguousarray(page_tables, dtype=np.int32)
    ln = np.ascontiguousarray(lengths, dtype=np.int32)
    out = np.empty_like(q)
    lib().axl_oracle_paged_decode(
        _p(q, ctypes.c_double), _p(kpool, ctypes.c_double), _p(vpool, ctypes.c_double),
        _p(pt, ctypes.c_int32), _p(ln, ctypes.c_int32), _p(out, ctypes.c_double), b, hq, hkv, d, p,
        page, pt.shape[1], ctypes.c_double(scale), int(window))
    return out
