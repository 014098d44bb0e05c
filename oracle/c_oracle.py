"""ctypes front end of the C oracle (na_oracle.c).  TEST INFRASTRUCTURE ONLY."""

from __future__ import annotations

import ctypes
import os
import subprocess
from concurrent.futures import ThreadPoolExecutor
from typing import Optional, Sequence

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libna_oracle.so")
_lib = None


def build(force: bool = False) -> str:
    if force or not os.path.exists(_LIB_PATH):
        subprocess.check_call(["make", "-C", _HERE, "-B", "libna_oracle.so"], stdout=subprocess.DEVNULL)
    return _LIB_PATH


def lib():
    global _lib
    if _lib is None:
        build()
        _lib = ctypes.CDLL(_LIB_PATH)
        _lib.na_oracle_rows.restype = ctypes.c_int64
        _lib.na_oracle_window.restype = ctypes.c_int
    return _lib


def _pad3(x, n, fill):
    x = [int(v) for v in x]
    return [fill] * (3 - n) + x


def window(i: int, k: int, s: int, L: int, causal: bool):
    st, en = ctypes.c_int(), ctypes.c_int()
    lib().na_oracle_window(int(i), int(k), int(s), int(L), int(bool(causal)), ctypes.byref(st), ctypes.byref(en))
    return st.value, en.value


def na_rows(q, k, v, kernel_size, stride, dilation, is_causal, scale: Optional[float],
            q_batch: Sequence[int], q_token: Sequence[int], threads: int = 8):
    """Evaluate selected queries.  q/k/v heads-last float32 [B, *X, H, D]; q_token are row-major
    token indices.  Returns (out [nq, H, D] f64, lse [nq, H] f64, visited key count)."""
    q = np.ascontiguousarray(q, dtype=np.float32)
    k = np.ascontiguousarray(k, dtype=np.float32)
    v = np.ascontiguousarray(v, dtype=np.float32)
    n = q.ndim - 3
    X = _pad3(q.shape[1 : 1 + n], n, 1)
    B, H, D = q.shape[0], q.shape[-2], q.shape[-1]
    Hkv = k.shape[-2]
    ks = _pad3(kernel_size, n, 1)
    st = _pad3(stride, n, 1)
    dl = _pad3(dilation, n, 1)
    ca = _pad3([int(bool(c)) for c in is_causal], n, 0)
    scale = float(scale) if scale is not None else float(D) ** -0.5
    qb = np.ascontiguousarray(q_batch, dtype=np.int32)
    qt = np.ascontiguousarray(q_token, dtype=np.int64)
    nq = qb.shape[0]
    out = np.empty((nq, H, D), dtype=np.float64)
    lse = np.empty((nq, H), dtype=np.float64)
    I3 = ctypes.c_int * 3
    L = lib()

    def run(lo, hi):
        lo, hi = int(lo), int(hi)
        if hi <= lo:
            return 0
        return L.na_oracle_rows(
            q.ctypes.data_as(ctypes.c_void_p), k.ctypes.data_as(ctypes.c_void_p),
            v.ctypes.data_as(ctypes.c_void_p), ctypes.c_int(B), I3(*X), ctypes.c_int(H),
            ctypes.c_int(Hkv), ctypes.c_int(D), I3(*ks), I3(*st), I3(*dl), I3(*ca),
            ctypes.c_double(scale), ctypes.c_int(hi - lo),
            ctypes.c_void_p(qb.ctypes.data + 4 * lo), ctypes.c_void_p(qt.ctypes.data + 8 * lo),
            ctypes.c_void_p(out.ctypes.data + 8 * lo * H * D), ctypes.c_void_p(lse.ctypes.data + 8 * lo * H))

    threads = max(1, min(threads, nq))
    bounds = np.linspace(0, nq, threads + 1).astype(int)
    if threads == 1:
        visited = run(0, nq)
    else:
        with ThreadPoolExecutor(threads) as ex:
            visited = sum(ex.map(lambda ab: run(*ab), zip(bounds[:-1], bounds[1:])))
    return out, lse, int(visited)


def na_forward(q, k, v, kernel_size, stride, dilation, is_causal, scale=None, threads: int = 8):
    """All queries, reshaped to [B, *X, H, D] / [B, *X, H]."""
    q = np.asarray(q)
    n = q.ndim - 3
    B = q.shape[0]
    N = int(np.prod(q.shape[1 : 1 + n]))
    qb = np.repeat(np.arange(B), N)
    qt = np.tile(np.arange(N), B)
    o, l, _ = na_rows(q, k, v, kernel_size, stride, dilation, is_causal, scale, qb, qt, threads)
    return o.reshape(*q.shape[:-1], q.shape[-1]), l.reshape(q.shape[:-1])


def na_backward(q, k, v, d_out, kernel_size, stride, dilation, is_causal, scale=None, threads: int = 8):
    """Gradients (dq, dk, dv), float64, of sum(out * d_out) for neighborhood attention on heads-last
    float32 tensors [B, *X, H, D]; the work is split over (batch, KV head) pairs."""
    q = np.ascontiguousarray(q, dtype=np.float32)
    k = np.ascontiguousarray(k, dtype=np.float32)
    v = np.ascontiguousarray(v, dtype=np.float32)
    d_out = np.ascontiguousarray(d_out, dtype=np.float32)
    assert d_out.shape == q.shape and k.shape == v.shape
    n = q.ndim - 3
    X = _pad3(q.shape[1 : 1 + n], n, 1)
    B, H, D = q.shape[0], q.shape[-2], q.shape[-1]
    Hkv = k.shape[-2]
    ks = _pad3(kernel_size, n, 1)
    st = _pad3(stride, n, 1)
    dl = _pad3(dilation, n, 1)
    ca = _pad3([int(bool(c)) for c in is_causal], n, 0)
    scale = float(scale) if scale is not None else float(D) ** -0.5
    dq = np.zeros(q.shape, dtype=np.float64)
    dk = np.zeros(k.shape, dtype=np.float64)
    dv = np.zeros(v.shape, dtype=np.float64)
    I3 = ctypes.c_int * 3
    L = lib()
    L.na_oracle_backward.restype = ctypes.c_int64

    def run(job):
        b, hk = job
        return L.na_oracle_backward(
            q.ctypes.data_as(ctypes.c_void_p), k.ctypes.data_as(ctypes.c_void_p),
            v.ctypes.data_as(ctypes.c_void_p), d_out.ctypes.data_as(ctypes.c_void_p), ctypes.c_int(b), I3(*X),
            ctypes.c_int(H), ctypes.c_int(Hkv), ctypes.c_int(D), I3(*ks), I3(*st), I3(*dl), I3(*ca),
            ctypes.c_double(scale), ctypes.c_int(hk), ctypes.c_int(hk + 1),
            dq.ctypes.data_as(ctypes.c_void_p), dk.ctypes.data_as(ctypes.c_void_p),
            dv.ctypes.data_as(ctypes.c_void_p))

    jobs = [(b, hk) for b in range(B) for hk in range(Hkv)]
    with ThreadPoolExecutor(max(1, min(threads, len(jobs)))) as ex:
        visited = list(ex.map(run, jobs))
    assert all(x >= 0 for x in visited)
    return dq, dk, dv
