"""ctypes binding of oracle/libksa_oracle.so (built by oracle/Makefile).
TEST INFRASTRUCTURE ONLY, like everything under oracle/."""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libksa_oracle.so")
_lib = None


def build(force=False):
    if force or not os.path.exists(_SO):
        subprocess.check_call(["make", "-C", _HERE, "-B" if force else "-s", "all"])
    return _SO


def lib():
    global _lib
    if _lib is None:
        build()
        L = ctypes.CDLL(_SO)
        i32p = ctypes.POINTER(ctypes.c_int32)
        f32p = ctypes.POINTER(ctypes.c_float)
        L.ksa_oracle_visible.restype = ctypes.c_int
        L.ksa_oracle_visible.argtypes = [ctypes.c_int64, ctypes.c_int64] + [ctypes.c_int] * 5
        L.ksa_oracle_block_index.restype = ctypes.c_int64
        L.ksa_oracle_block_index.argtypes = [ctypes.c_int] * 9 + [i32p] * 4
        L.ksa_oracle_attention_rows.restype = None
        L.ksa_oracle_attention_rows.argtypes = (
            [f32p] * 3 + [ctypes.c_int] * 10 + [ctypes.c_float, i32p, ctypes.c_int, f32p, f32p])
        L.ksa_oracle_decode.restype = None
        L.ksa_oracle_decode.argtypes = (
            [f32p] * 3 + [ctypes.c_int] * 5 + [ctypes.c_int64] * 2 + [i32p, i32p, ctypes.c_float, f32p])
        _lib = L
    return _lib


def _p(a, t):
    return a.ctypes.data_as(ctypes.POINTER(t))


def block_index(Sq, Sk, C, S, W, P, skip_old=False, tile_m=128, tile_n=64):
    M = -(-Sq // tile_m)
    N = -(-Sk // tile_n)
    mc = np.empty(M, np.int32)
    fc = np.empty(M, np.int32)
    mi = np.empty((M, N), np.int32)
    fi = np.empty((M, N), np.int32)
    pairs = lib().ksa_oracle_block_index(Sq, Sk, C, S, W, P, int(skip_old), tile_m, tile_n,
                                         _p(mc, ctypes.c_int32), _p(mi, ctypes.c_int32),
                                         _p(fc, ctypes.c_int32), _p(fi, ctypes.c_int32))
    return mc, mi, fc, fi, int(pairs)


def attention_rows(q, k, v, C, S, W, summary_pos=None, skip_old=False, scale=None, rows=None):
    """q [Sq,Hq,D], k/v [Sq,Hkv,D] float32.  Returns (out [R,Hq,D], lse [Hq,R]) float32."""
    q = np.ascontiguousarray(q, np.float32)
    k = np.ascontiguousarray(k, np.float32)
    v = np.ascontiguousarray(v, np.float32)
    Sq, Hq, D = q.shape
    Hkv = k.shape[1]
    if summary_pos is not None:
        sp = np.asarray(summary_pos, bool)
        k = np.ascontiguousarray(np.concatenate([k[sp], k], axis=0))
        v = np.ascontiguousarray(np.concatenate([v[sp], v], axis=0))
    Sk = k.shape[0]
    P = Sk - Sq
    if scale is None:
        scale = 1.0 / np.sqrt(D)
    rows = np.arange(Sq, dtype=np.int32) if rows is None else np.ascontiguousarray(rows, np.int32)
    out = np.empty((len(rows), Hq, D), np.float32)
    lse = np.empty((Hq, len(rows)), np.float32)
    f = ctypes.c_float
    lib().ksa_oracle_attention_rows(_p(q, f), _p(k, f), _p(v, f), Sq, Sk, Hq, Hkv, D, C, S, W, P,
                                    int(skip_old), float(scale), _p(rows, ctypes.c_int32),
                                    len(rows), _p(out, f), _p(lse, f))
    return out, lse


def decode(q, k, v, start, end, scale=None):
    """q [B,Hq,Q,D]; k/v [B,Hkv,L,D] float32 contiguous; start/end int32 [B]."""
    q = np.ascontiguousarray(q, np.float32)
    k = np.ascontiguousarray(k, np.float32)
    v = np.ascontiguousarray(v, np.float32)
    Bz, Hq, Q, D = q.shape
    Hkv, L = k.shape[1], k.shape[2]
    if scale is None:
        scale = 1.0 / np.sqrt(D)
    start = np.ascontiguousarray(np.broadcast_to(np.asarray(start, np.int32), (Bz,)))
    end = np.ascontiguousarray(np.broadcast_to(np.asarray(end, np.int32), (Bz,)))
    out = np.empty((Bz, Q, Hq, D), np.float32)
    f = ctypes.c_float
    lib().ksa_oracle_decode(_p(q, f), _p(k, f), _p(v, f), Bz, Hq, Hkv, Q, D, Hkv * L * D, L * D,
                            _p(start, ctypes.c_int32), _p(end, ctypes.c_int32), float(scale),
                            _p(out, f))
    return out
