"""ctypes front end of the CPU oracle (oracle/dci_oracle.cpp).

TEST INFRASTRUCTURE ONLY: tests, the smoke check and the benchmark's
CPU-baseline leg import this; the shipped package never does.

All functions take and return numpy arrays.  `build()` compiles the shared
library with the Makefile beside this file when it is missing.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libdci_oracle.so")
_lib = None

_f32p = np.ctypeslib.ndpointer(np.float32, flags="C_CONTIGUOUS")
_i32p = np.ctypeslib.ndpointer(np.int32, flags="C_CONTIGUOUS")


def build(force=False):
    """Compile libdci_oracle.so (g++, OpenMP) next to the source."""
    if force or not os.path.exists(_LIB_PATH):
        subprocess.check_call(["make", "-B", "-C", _HERE, "libdci_oracle.so"],
                              stdout=subprocess.DEVNULL)
    return _LIB_PATH


def lib():
    global _lib
    if _lib is None:
        build()
        L = ctypes.CDLL(_LIB_PATH)
        L.dci_oracle_normalize.argtypes = [_f32p, ctypes.c_int, ctypes.c_int]
        L.dci_oracle_normalize.restype = None
        L.dci_oracle_matmul_nt.argtypes = [_f32p, _f32p, _f32p, ctypes.c_int64,
                                           ctypes.c_int64, ctypes.c_int]
        L.dci_oracle_matmul_nt.restype = None
        L.dci_oracle_segsort.argtypes = [_f32p, ctypes.c_int64, ctypes.c_int,
                                         ctypes.c_int, _f32p, _i32p]
        L.dci_oracle_segsort.restype = None
        L.dci_oracle_search.argtypes = [_f32p, ctypes.c_float, ctypes.c_int]
        L.dci_oracle_search.restype = ctypes.c_int
        L.dci_oracle_window_sequence.argtypes = [_f32p, ctypes.c_int, ctypes.c_int,
                                                 ctypes.c_float, _i32p, _f32p,
                                                 ctypes.c_int]
        L.dci_oracle_window_sequence.restype = ctypes.c_int
        L.dci_oracle_query.argtypes = [
            _f32p, _i32p, _f32p, _f32p, _f32p, ctypes.c_int64, ctypes.c_int,
            ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int,
            ctypes.c_int, ctypes.c_int64, ctypes.c_int64, _i32p, _f32p,
            ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int64, ctypes.c_void_p,
            ctypes.c_int]
        L.dci_oracle_query.restype = ctypes.c_int
        L.dci_oracle_query_blind.argtypes = [
            _f32p, _i32p, _f32p, ctypes.c_int64, ctypes.c_int, ctypes.c_int,
            ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int64,
            ctypes.c_int64, _i32p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int]
        L.dci_oracle_query_blind.restype = ctypes.c_int
        L.dci_oracle_max_threads.argtypes = []
        L.dci_oracle_max_threads.restype = ctypes.c_int
        _lib = L
    return _lib


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def normalize(P):
    """Rows of P scaled to unit L2 norm the way the reference does it."""
    P = _f32(P).copy()
    lib().dci_oracle_normalize(P, P.shape[0], P.shape[1])
    return P


def project(A, B):
    """out[r][c] = A[r] . B[c] in fp32; project(P, X) -> keys [I][N]."""
    A, B = _f32(A), _f32(B)
    assert A.shape[1] == B.shape[1]
    out = np.empty((A.shape[0], B.shape[0]), np.float32)
    lib().dci_oracle_matmul_nt(A, B, out, A.shape[0], B.shape[0], A.shape[1])
    return out


def segsort(keys, block_size):
    """Per (simple index, partition) sort of keys [I][N] -> (skeys, sids)."""
    keys = _f32(keys)
    I, N = keys.shape
    skeys = np.empty_like(keys)
    sids = np.empty((I, N), np.int32)
    lib().dci_oracle_segsort(keys, N, I, block_size, skeys, sids)
    return skeys, sids


def search(key, q):
    key = _f32(key)
    return lib().dci_oracle_search(key, float(np.float32(q)), key.shape[0])


def window_sequence(key, T, q):
    """(window starts, priorities) of one simple index until exhaustion."""
    key = _f32(key)
    cap = 2 * (key.shape[0] // T + 4)
    cur = np.empty(cap, np.int32)
    prio = np.empty(cap, np.float32)
    n = lib().dci_oracle_window_sequence(key, key.shape[0], T,
                                         float(np.float32(q)), cur, prio, cap)
    return cur[:n].copy(), prio[:n].copy()


def query(skeys, sids, data, queries, qproj, M, L, B, T, k, outer,
          max_cand=None, want_counters=True, cand_cap=0, num_threads=0):
    """Run the oracle query.  Returns dict(ids, dists, counters, cand_ids, cand_cnt).

    max_cand defaults to 10*k as dciknn_cuda/core.py:87 fixes it.
    """
    skeys, data, queries, qproj = _f32(skeys), _f32(data), _f32(queries), _f32(qproj)
    sids = np.ascontiguousarray(sids, dtype=np.int32)
    N, dim = data.shape
    nq = queries.shape[0]
    assert skeys.shape == (M * L, N) and sids.shape == (M * L, N)
    assert qproj.shape == (nq, M * L) and queries.shape[1] == dim
    if max_cand is None:
        max_cand = 10 * k
    ids = np.empty((nq, k), np.int32)
    dists = np.empty((nq, k), np.float32)
    counters = np.zeros((nq, 4), np.uint64) if want_counters else None
    cand_ids = np.full((nq, max(cand_cap, 1)), -1, np.int32) if cand_cap else None
    cand_cnt = np.zeros(nq, np.int64) if cand_cap else None
    rc = lib().dci_oracle_query(
        skeys, sids, data, queries, qproj, N, dim, M, L, B, T, nq, k, outer,
        max_cand, ids, dists,
        counters.ctypes.data if counters is not None else None,
        cand_ids.ctypes.data if cand_ids is not None else None, cand_cap,
        cand_cnt.ctypes.data if cand_cnt is not None else None, num_threads)
    if rc != 0:
        raise ValueError("dci_oracle_query rejected its arguments")
    return dict(ids=ids, dists=dists, counters=counters, cand_ids=cand_ids,
                cand_cnt=cand_cnt)


def query_blind(skeys, sids, qproj, M, L, B, T, k, outer, max_cand=None,
                num_threads=0):
    """Blind query: dict(ids, steps, counters), [nq][min(max_cand, outer)] each.

    ids are the promoted points ascending by (promoting step, id), -1 beyond
    them; steps the promoting steps (uint32, all ones beside -1).
    """
    skeys, qproj = _f32(skeys), _f32(qproj)
    sids = np.ascontiguousarray(sids, dtype=np.int32)
    N = skeys.shape[1]
    nq = qproj.shape[0]
    assert skeys.shape == (M * L, N) and sids.shape == (M * L, N)
    assert qproj.shape == (nq, M * L)
    if max_cand is None:
        max_cand = 10 * k
    R = min(max_cand, outer)
    ids = np.empty((nq, R), np.int32)
    steps = np.empty((nq, R), np.uint32)
    counters = np.zeros((nq, 4), np.uint64)
    rc = lib().dci_oracle_query_blind(
        skeys, sids, qproj, N, M, L, B, T, nq, k, outer, max_cand, ids,
        steps.ctypes.data, counters.ctypes.data, num_threads)
    if rc != 0:
        raise ValueError("dci_oracle_query_blind rejected its arguments")
    return dict(ids=ids, steps=steps, counters=counters)


def build_index(P, X, block_size):
    """Directions + data -> (skeys, sids), the oracle's whole add()."""
    return segsort(project(P, X), block_size)


def knn(P, X, Q, M, L, B, T, k, outer, **kw):
    """End-to-end oracle: build, project queries, query."""
    skeys, sids = build_index(P, X, B)
    qproj = project(Q, P)
    return query(skeys, sids, X, Q, qproj, M, L, B, T, k, outer, **kw)


def brute_force(X, Q, k):
    """Exact k-NN in float64 (ids, dists) for recall checks."""
    X64 = np.asarray(X, np.float64)
    Q64 = np.asarray(Q, np.float64)
    d2 = ((Q64 ** 2).sum(1)[:, None] - 2.0 * Q64 @ X64.T + (X64 ** 2).sum(1)[None, :])
    idx = np.argsort(d2, axis=1, kind="stable")[:, :k]
    dd = np.sqrt(np.maximum(np.take_along_axis(d2, idx, 1), 0.0))
    return idx.astype(np.int32), dd


def max_threads():
    return lib().dci_oracle_max_threads()
