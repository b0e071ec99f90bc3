"""ctypes access to oracle/libmep_oracle.so (the scalar C checker) on numpy
arrays.  TEST INFRASTRUCTURE ONLY -- see oracle/mep_oracle.c."""

from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libmep_oracle.so")
_lib = None


def build() -> str:
    subprocess.run(["make", "-C", _HERE, "-B", "libmep_oracle.so"], check=True,
                   stdout=subprocess.DEVNULL)
    return LIB_PATH


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            build()
        _lib = C.CDLL(LIB_PATH)
        _lib.ora_plan.restype = C.c_int
    return _lib


def _p(a):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


def plan(tpe: np.ndarray, topk_rank: np.ndarray, rank: int, S: int, K: int, tp: int, NvS: int):
    """-> (dst[N], cu_seqlens[2epn], experts_to_copy[R,epn], zero_fill[2epn,2], remote_stats[2])"""
    tpe = np.ascontiguousarray(tpe, dtype=np.int32)
    topk = np.ascontiguousarray(topk_rank, dtype=np.int32).reshape(-1)
    R, E = tpe.shape
    epn = E // R
    dst = np.empty(S * K, np.int32)
    cu = np.empty(2 * epn, np.int32)
    etc = np.empty((R, epn), np.int32)
    zf = np.empty((2 * epn, 2), np.int32)
    st = np.empty(2, np.int32)
    rc = lib().ora_plan(_p(tpe), _p(topk), rank, S, K, E, R, tp, NvS, _p(dst), _p(cu), _p(etc),
                        _p(zf), _p(st))
    if rc != 0:
        raise RuntimeError(f"ora_plan failed with {rc}")
    return dst, cu, etc, zf, st


def dispatch(hidden_u16, w, dst, zf, shards_u16, wslots, rank, K, NvS, write_dups):
    """In place on shards_u16 [R, rows, H] (uint16 bit patterns) and wslots [R, stride]."""
    S, H = hidden_u16.shape
    R, rows, _ = shards_u16.shape
    epn = zf.shape[0] // 2
    lib().ora_dispatch(_p(hidden_u16), _p(w), _p(dst), _p(zf), _p(shards_u16), C.c_int64(rows),
                       _p(wslots), C.c_int64(0 if wslots is None else wslots.shape[1]), rank, S, H,
                       K, epn, NvS, int(write_dups))


def combine(shards_u16, wslots, dst, S, K, NvS, mode):
    R, rows, H = shards_u16.shape
    out = np.empty((S, H), np.uint16)
    out_sk = None if wslots is None else np.empty((S, K), np.float32)
    acc = np.empty(2 * H, np.float32)
    lib().ora_combine(_p(shards_u16), C.c_int64(rows), _p(wslots),
                      C.c_int64(0 if wslots is None else wslots.shape[1]), _p(dst), _p(out),
                      _p(out_sk), S, H, K, NvS, mode, _p(acc))
    return out, out_sk


def prefetch(local_bytes, pool_bytes, etc, rank):
    """local [epn, nbytes] uint8, pool [R, epn, nbytes] uint8 (contiguous)."""
    epn, nb = local_bytes.shape
    R = pool_bytes.shape[0]
    lib().ora_prefetch(_p(local_bytes), _p(pool_bytes), C.c_int64(epn * nb), C.c_int64(nb),
                       _p(etc), rank, epn, R)


def grad_reduce(local, pool, etc, rank):
    """local [epn, n] fp32, pool [R, epn, n] fp32 (contiguous)."""
    epn, n = local.shape
    R = pool.shape[0]
    lib().ora_grad_reduce(_p(local), _p(pool), C.c_int64(epn * n), C.c_int64(n), _p(etc), rank,
                          epn, R)
