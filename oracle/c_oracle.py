"""ctypes loader for oracle/libfa_oracle.so (plain-C restatement, oracle/fa_oracle.c).  TEST INFRASTRUCTURE ONLY."""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libfa_oracle.so")


def build() -> str:
    subprocess.run(["make", "-s", "-B", "-C", _HERE, "libfa_oracle.so"], check=True)
    return LIB_PATH


def _lib() -> ctypes.CDLL:
    if not os.path.exists(LIB_PATH):
        build()
    L = ctypes.CDLL(LIB_PATH)
    fp = ctypes.POINTER(ctypes.c_float)
    ip = ctypes.POINTER(ctypes.c_int32)
    L.fa_oracle_forward_dense.restype = ctypes.c_int
    L.fa_oracle_forward_dense.argtypes = [fp, fp, fp, fp, fp] + [ctypes.c_int] * 6 + [ctypes.c_float, ctypes.c_int]
    L.fa_oracle_forward_packed.restype = ctypes.c_int
    L.fa_oracle_forward_packed.argtypes = [fp, fp, fp, fp, fp, ip, ip] + [ctypes.c_int] * 4 + [
        ctypes.c_int64, ctypes.c_float, ctypes.c_int]
    return L


def _f(a):
    return a.ctypes.data_as(ctypes.POINTER(ctypes.c_float))


def dense(q, k, v, is_causal=False, scale=None):
    """q [B,Hq,Sq,D], k/v [B,Hk,Sk,D] float arrays -> (out fp32, lse fp32)."""
    q, k, v = (np.ascontiguousarray(np.asarray(x, dtype=np.float32)) for x in (q, k, v))
    B, Hq, Sq, D = q.shape
    Hk, Sk = k.shape[1], k.shape[2]
    scale = float(scale) if scale is not None else 1.0 / np.sqrt(D)
    out = np.empty_like(q)
    lse = np.empty((B, Hq, Sq), dtype=np.float32)
    rc = _lib().fa_oracle_forward_dense(_f(q), _f(k), _f(v), _f(out), _f(lse), B, Hq, Hk, Sq, Sk, D, scale,
                                        1 if is_causal else 0)
    assert rc == 0
    return out, lse


def packed(q, k, v, cu_q, cu_k, is_causal=False, scale=None):
    """q [Tq,Hq,D], k/v [Tk,Hk,D], cu_seqlens [B+1] -> (out [Tq,Hq,D], lse [Hq,Tq])."""
    q, k, v = (np.ascontiguousarray(np.asarray(x, dtype=np.float32)) for x in (q, k, v))
    cu_q = np.ascontiguousarray(np.asarray(cu_q, dtype=np.int32))
    cu_k = np.ascontiguousarray(np.asarray(cu_k, dtype=np.int32))
    Tq, Hq, D = q.shape
    Hk = k.shape[1]
    scale = float(scale) if scale is not None else 1.0 / np.sqrt(D)
    out = np.zeros_like(q)
    lse = np.full((Hq, Tq), np.inf, dtype=np.float32)
    ip = ctypes.POINTER(ctypes.c_int32)
    rc = _lib().fa_oracle_forward_packed(_f(q), _f(k), _f(v), _f(out), _f(lse), cu_q.ctypes.data_as(ip),
                                         cu_k.ctypes.data_as(ip), len(cu_q) - 1, Hq, Hk, D, Tq, scale,
                                         1 if is_causal else 0)
    assert rc == 0
    return out, lse
