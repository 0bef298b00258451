"""CPU oracle of the CBM multiply -- TEST INFRASTRUCTURE ONLY.

Only ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py`` may
import this module; nothing under ``cbm4gnn_amd/`` does.

It has two layers:

* ctypes bindings of ``oracle/cbm_oracle.c`` (the C restatement of the reference's builder,
  SpMM and tree walks; reference line numbers are in that file's header), and
* independent NumPy / pure-Python restatements used to pin both the C oracle and the product's
  host builder: the candidate rule by brute force on dense ``A @ A.T``
  (``cbm_extensions.cpp:75-103``), the format derived from a parent array by set differences
  (``cbm.py:69-115`` read backwards), dense fp64 closed forms of the two products, the
  reference's compression ratio (``benchmark/utility.py:45-64``).

Parity status: every function here is pinned by ``tests/test_oracle.py`` except the choice
among equal-weight arborescences (arbok's tie-breaking: "parity unpinned", the reference's own
tests do not pin it either) and MKL's fp32 summation order inside ``mkl_sparse_s_mm``
(agreement is to the 1e-4 tolerance the reference's tests use).
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "liboracle.so")

_lib = None


def build(force: bool = False) -> str:
    """Compile ``cbm_oracle.c`` with gcc (see ``oracle/Makefile`` for the same recipe)."""
    src = os.path.join(HERE, "cbm_oracle.c")
    if force or not os.path.exists(LIB_PATH) or os.path.getmtime(LIB_PATH) < os.path.getmtime(src):
        subprocess.check_call(["make", "-C", HERE, "-s", "-B", "liboracle.so"])
    return LIB_PATH


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            build()
        L = C.CDLL(LIB_PATH)
        P, I32, I64 = C.c_void_p, C.c_int32, C.c_int64
        L.oracle_build.restype = C.c_int
        L.oracle_build.argtypes = [P, P, I64, I32, I32] + [C.POINTER(P)] * 5 + [C.POINTER(I64), C.POINTER(P),
                                                                               C.POINTER(I64), C.POINTER(I64)]
        L.oracle_msa.restype = C.c_int
        L.oracle_msa.argtypes = [I32, I64, P, P, P, I32, P, C.POINTER(I64)]
        L.oracle_candidates.restype = C.c_int
        L.oracle_candidates.argtypes = [I32, P, P, I32, C.POINTER(P), C.POINTER(P), C.POINTER(P), C.POINTER(I64)]
        L.oracle_csr_spmm.restype = None
        L.oracle_csr_spmm.argtypes = [P, P, P, P, P, P, I32, I32, I32]
        L.oracle_csr_spmm_grouped.restype = None
        L.oracle_csr_spmm_grouped.argtypes = [P, P, P, P, P, P, I32, I32, I32, I32]
        L.oracle_update_plain.restype = None
        L.oracle_update_plain.argtypes = [P, P, P, I32, I32, I32]
        L.oracle_update_fused.restype = None
        L.oracle_update_fused.argtypes = [P, P, P, P, I32, I32, I32]
        L.oracle_free.restype = None
        L.oracle_free.argtypes = [P]
        L.oracle_max_threads.restype = C.c_int
        _lib = L
    return _lib


def _p(a):
    return a.ctypes.data_as(C.c_void_p) if a is not None else None


def _take(ptr, count, dtype):
    if count == 0:
        out = np.empty(0, dtype)
    else:
        out = np.ctypeslib.as_array(C.cast(ptr, C.POINTER(np.ctypeslib.as_ctypes_type(dtype))), shape=(count,)).copy()
    lib().oracle_free(ptr)
    return out


def max_threads() -> int:
    return int(lib().oracle_max_threads())


# ------------------------------------------------------------------------------------------------
# C oracle wrappers
# ------------------------------------------------------------------------------------------------
def build_format(edge_index, n: int, alpha: int) -> dict:
    """Reference builder restated (``cbm_extensions.cpp:8-326``).  Returns the reference's five
    outputs (tree CSR + delta COO with signs) plus parent[], candidate count and tree weight."""
    ei = np.ascontiguousarray(np.asarray(edge_index, np.int32))
    row, col = np.ascontiguousarray(ei[0]), np.ascontiguousarray(ei[1])
    outs = [C.c_void_p() for _ in range(5)]
    parent = C.c_void_p()
    nnz, ncand, w = C.c_int64(), C.c_int64(), C.c_int64()
    rc = lib().oracle_build(_p(row), _p(col), row.shape[0], n, alpha, *[C.byref(o) for o in outs],
                            C.byref(nnz), C.byref(parent), C.byref(ncand), C.byref(w))
    if rc != 0:
        raise RuntimeError(f"oracle_build failed with status {rc}")
    k = nnz.value
    par = _take(parent, n, np.int32)
    return {
        "mst_row": _take(outs[0], n + 2, np.int32), "mst_col": _take(outs[1], n, np.int32),
        "d_row": _take(outs[2], k, np.int32), "d_col": _take(outs[3], k, np.int32),
        "d_sign": _take(outs[4], k, np.int8), "parent": par,
        "n_candidates": ncand.value, "msa_weight": w.value, "nnz": k,
    }


def msa(n: int, eu, ev, ew, root: int):
    """Minimum spanning arborescence (Chu-Liu/Edmonds by contraction): (chosen edge per node, weight)."""
    eu = np.ascontiguousarray(eu, np.int32); ev = np.ascontiguousarray(ev, np.int32); ew = np.ascontiguousarray(ew, np.int32)
    chosen = np.empty(n, np.int64)
    w = C.c_int64()
    rc = lib().oracle_msa(n, eu.shape[0], _p(eu), _p(ev), _p(ew), root, _p(chosen), C.byref(w))
    if rc != 0:
        raise RuntimeError(f"oracle_msa failed with status {rc}")
    return chosen, w.value


def candidates(n: int, rowptr, col, alpha: int):
    """Distance-graph edges in the reference's emission order (``cbm_extensions.cpp:75-103``)."""
    rp = np.ascontiguousarray(rowptr, np.int64); ci = np.ascontiguousarray(col, np.int32)
    u, v, w = C.c_void_p(), C.c_void_p(), C.c_void_p()
    m = C.c_int64()
    rc = lib().oracle_candidates(n, _p(rp), _p(ci), alpha, C.byref(u), C.byref(v), C.byref(w), C.byref(m))
    if rc != 0:
        raise RuntimeError(f"oracle_candidates failed with status {rc}")
    return _take(u, m.value, np.int32), _take(v, m.value, np.int32), _take(w, m.value, np.int32)


def deltas_csr(fmt: dict, n: int, m=None):
    """The reference's ``deltas``: COO -> coalesce -> CSR with sorted columns
    (``cbm.py:120-141``); values +-1, or +-m[col] for the normalised builder
    (``cbm_extensions.cpp:504-585``).  Returns (crow int32 [n+1], col int32, val fp32)."""
    order = np.lexsort((fmt["d_col"], fmt["d_row"]))
    col = fmt["d_col"][order].astype(np.int32)
    val = fmt["d_sign"][order].astype(np.float32)
    if m is not None:
        val = val * np.asarray(m, np.float32)[col]
    crow = np.zeros(n + 1, np.int64)
    np.add.at(crow, fmt["d_row"].astype(np.int64) + 1, 1)
    return np.cumsum(crow).astype(np.int32), col, val.astype(np.float32)


def csr_spmm(crow, col, val, x, threads: int = 1, groups: int = 1):
    """Y = A @ X, the role of ``mkl_sparse_s_mm`` (``cbm_extensions.cpp:1149-1159``).
    ``groups`` > 1 selects the round-robin partial-sum order of a SIMD kernel (see the C file)."""
    crow = np.ascontiguousarray(crow, np.int32); col = np.ascontiguousarray(col, np.int32)
    val = None if val is None else np.ascontiguousarray(val, np.float32)
    x = np.ascontiguousarray(x, np.float32)
    n = crow.shape[0] - 1
    y = np.empty((n, x.shape[1]), np.float32)
    rb = np.ascontiguousarray(crow[:-1]); re = np.ascontiguousarray(crow[1:])
    if groups == 1:
        lib().oracle_csr_spmm(_p(rb), _p(re), _p(col), _p(val), _p(x), _p(y), n, x.shape[1], threads)
    else:
        assert groups in (2, 4, 8, 16, 32, 64)
        lib().oracle_csr_spmm_grouped(_p(rb), _p(re), _p(col), _p(val), _p(x), _p(y), n, x.shape[1], groups, threads)
    return y


def update_plain(mst_row, mst_col, y, threads: int = 1):
    """In place ``Y[v] += Y[parent(v)]`` top-down (``cbm_extensions.cpp:713-738``, ``:1166-1218``)."""
    assert y.dtype == np.float32 and y.flags.c_contiguous
    mst_row = np.ascontiguousarray(mst_row, np.int32); mst_col = np.ascontiguousarray(mst_col, np.int32)
    lib().oracle_update_plain(_p(mst_row), _p(mst_col), _p(y), y.shape[0], y.shape[1], threads)
    return y


def update_fused(mst_row, mst_col, m, y, threads: int = 1):
    """In place normalised walk (``cbm_extensions.cpp:908-995``, ``:1285-1373``)."""
    assert y.dtype == np.float32 and y.flags.c_contiguous
    mst_row = np.ascontiguousarray(mst_row, np.int32); mst_col = np.ascontiguousarray(mst_col, np.int32)
    m = np.ascontiguousarray(m, np.float32)
    lib().oracle_update_fused(_p(mst_row), _p(mst_col), _p(m), _p(y), y.shape[0], y.shape[1], threads)
    return y


def spmm_update(crow, col, val, mst_row, mst_col, x, m=None, threads: int = 1, groups: int = 1):
    """The whole reference multiply: ``*_s_spmm_update_csr_int32`` (m None) or
    ``*_s_fused_spmm_update_csr_int32`` (m given; val must already hold +-m[col])."""
    y = csr_spmm(crow, col, val, x, threads, groups)
    return update_plain(mst_row, mst_col, y, threads) if m is None else update_fused(mst_row, mst_col, m, y, threads)


def col_multiplier(edge_index, n: int):
    """m[i] = (#edges whose row is i) ** -0.5 in fp32 (``cbm.py:34-41``): one correctly rounded
    sqrt and one correctly rounded division, which is what torch's pow(-0.5) evaluates."""
    deg = np.bincount(np.asarray(edge_index[0], np.int64), minlength=n).astype(np.float32)
    with np.errstate(divide="ignore"):
        return (np.float32(1.0) / np.sqrt(deg)).astype(np.float32)


# ------------------------------------------------------------------------------------------------
# independent restatements (NumPy / pure Python) that pin the above
# ------------------------------------------------------------------------------------------------
def adjacency_lists(edge_index, n: int):
    rows = [set() for _ in range(n)]
    for r, c in zip(np.asarray(edge_index[0]).tolist(), np.asarray(edge_index[1]).tolist()):
        rows[r].add(c)
    return rows


def dense_adjacency(edge_index, n: int):
    a = np.zeros((n, n), np.float64)
    a[np.asarray(edge_index[0], np.int64), np.asarray(edge_index[1], np.int64)] = 1.0
    return a


def candidates_bruteforce(a_dense: np.ndarray, alpha: int):
    """All pairs, straight from the rule: root -> i with weight nnz_i; for i < j sharing a
    column, h = nnz_i + nnz_j - 2 (A A^T)_ij; j -> i if h < nnz_i - alpha; i -> j if
    h < nnz_j - alpha.  Returns a set of (u, v, w)."""
    n = a_dense.shape[0]
    s = (a_dense @ a_dense.T).astype(np.int64)
    nnz = a_dense.sum(axis=1).astype(np.int64)
    out = set()
    for i in range(n):
        out.add((n, i, int(nnz[i])))
        for j in range(i + 1, n):
            if s[i, j] == 0:
                continue
            h = int(nnz[i] + nnz[j] - 2 * s[i, j])
            if h < nnz[i] - alpha:
                out.add((j, i, h))
            if h < nnz[j] - alpha:
                out.add((i, j, h))
    return out


def format_from_parent(edge_index, n: int, parent):
    """Derive every integer array of the device format from parent[] alone, by set differences
    (no merge, no BFS queue): rowptr, packed idx, order, level_off, mst_row, mst_col.
    parent[v] is -1 (or n) for children of the root."""
    rows = adjacency_lists(edge_index, n)
    parent = np.asarray(parent, np.int64).copy()
    parent[parent == n] = -1
    rowptr = np.zeros(n + 1, np.int64)
    idx = []
    for v in range(n):
        u = int(parent[v])
        if u < 0:
            ent = [(c, 0) for c in rows[v]]
        else:
            ent = [(c, 0) for c in rows[v] - rows[u]] + [(c, 1) for c in rows[u] - rows[v]]
        ent.sort()
        idx.extend(c | (neg << 31) for c, neg in ent)
        rowptr[v + 1] = rowptr[v] + len(ent)
    level = np.zeros(n, np.int64)
    for v in range(n):                      # walk up; fine for test sizes
        d, u = 0, int(parent[v])
        while u >= 0:
            d += 1
            u = int(parent[u])
        level[v] = d
    order = np.array(sorted(range(n), key=lambda v: (level[v], v)), np.int32)
    n_levels = int(level.max()) + 1
    level_off = np.array([int((level < l).sum()) for l in range(n_levels + 1)], np.int32)
    kids = [[] for _ in range(n + 1)]
    for v in range(n):
        kids[n if parent[v] < 0 else int(parent[v])].append(v)
    mst_row = np.zeros(n + 2, np.int32)
    mst_col = []
    for u in range(n + 1):
        mst_col.extend(sorted(kids[u]))
        mst_row[u + 1] = len(mst_col)
    return {
        "rowptr": rowptr.astype(np.int32), "idx": np.array(idx, np.uint32), "order": order,
        "level_off": level_off, "mst_row": mst_row, "mst_col": np.array(mst_col, np.int32),
        "parent": parent.astype(np.int32),
    }


def check_format(edge_index, n: int, rowptr, idx, mst_row, mst_col) -> bool:
    """The reference's ``check_format`` (``cbm.py:69-115``) on packed arrays."""
    rows = adjacency_lists(edge_index, n)
    s = [None] * (n + 1)
    s[n] = set()
    queue = [n]
    seen = 0
    while queue:
        u = queue.pop(0)
        for v in mst_col[mst_row[u]:mst_row[u + 1]]:
            v = int(v)
            cur = set(s[u])
            for k in range(int(rowptr[v]), int(rowptr[v + 1])):
                c = int(idx[k]) & 0x7FFFFFFF
                if int(idx[k]) >> 31:
                    cur.remove(c)
                else:
                    if c in cur:
                        return False
                    cur.add(c)
            s[v] = cur
            seen += 1
            queue.append(v)
    return seen == n and all(s[v] == rows[v] for v in range(n))


def dense_product(edge_index, n: int, x, normalized: bool):
    """fp64 closed form: A @ X, or diag(m) A diag(m) @ X with m = rowdeg ** -0.5."""
    a = dense_adjacency(edge_index, n)
    x = np.asarray(x, np.float64)
    if not normalized:
        return a @ x
    m = a.sum(axis=1) ** -0.5
    return (m[:, None] * a * m[None, :]) @ x


def compression_ratio(n: int, nnz_a: int, nnz_delta: int) -> float:
    """``benchmark/utility.py:45-64`` in element counts."""
    return (n + 1 + 2 * nnz_a) / (n + 1 + 2 * nnz_delta + (n + 2) + n)


def max_rel_err(got, want) -> float:
    """max |got - want| / max |want| -- the 'max-relative error' every parity test uses."""
    got = np.asarray(got, np.float64); want = np.asarray(want, np.float64)
    denom = float(np.abs(want).max())
    return float(np.abs(got - want).max() / denom) if denom > 0 else float(np.abs(got).max())


# ------------------------------------------------------------------------------------------------
# the real MKL routines of the reference path, reached through torch's libtorch_cpu.so
# ------------------------------------------------------------------------------------------------
class _MatrixDescr(C.Structure):
    _fields_ = [("type", C.c_int), ("mode", C.c_int), ("diag", C.c_int)]


_mkl = None


def mkl():
    """ctypes handle on libtorch_cpu.so with the oneMKL sparse BLAS prototypes the reference
    calls (``cbm_extensions.cpp:1133-1159``), or None when the symbols are not exported."""
    global _mkl
    if _mkl is None:
        try:
            import torch
            path = os.path.join(os.path.dirname(torch.__file__), "lib", "libtorch_cpu.so")
            L = C.CDLL(path)
            L.mkl_sparse_s_create_csr.restype = C.c_int
            L.mkl_sparse_s_create_csr.argtypes = [C.POINTER(C.c_void_p), C.c_int, C.c_int, C.c_int,
                                                  C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p]
            L.mkl_sparse_s_mm.restype = C.c_int
            L.mkl_sparse_s_mm.argtypes = [C.c_int, C.c_float, C.c_void_p, _MatrixDescr, C.c_int, C.c_void_p,
                                          C.c_int, C.c_int, C.c_float, C.c_void_p, C.c_int]
            L.mkl_sparse_destroy.restype = C.c_int
            L.mkl_sparse_destroy.argtypes = [C.c_void_p]
            _mkl = L
        except (OSError, AttributeError, ImportError):
            _mkl = False
    return _mkl or None


def mkl_csr_spmm(rb, re, col, val, x, y):
    """``mkl_sparse_s_create_csr`` + ``mkl_sparse_s_mm`` with the reference's arguments
    (NON_TRANSPOSE=10, GENERAL=20, ROW_MAJOR=101, alpha 1, beta 0); the handle is re-created on
    every call exactly as the reference does."""
    L = mkl()
    if L is None:
        raise RuntimeError("MKL sparse BLAS symbols are not reachable through libtorch_cpu.so")
    n, d = y.shape
    h = C.c_void_p()
    # the reference passes the feature width as the column count (cbm_extensions.cpp:1136-1137);
    # MKL does not range-check it, the true column count x.shape[0] is passed here
    st = L.mkl_sparse_s_create_csr(C.byref(h), 0, n, x.shape[0], _p(rb), _p(re), _p(col), _p(val))
    if st != 0:
        raise RuntimeError(f"mkl_sparse_s_create_csr status {st}")
    st = L.mkl_sparse_s_mm(10, 1.0, h, _MatrixDescr(20, 0, 0), 101, _p(x), d, d, 0.0, _p(y), d)
    L.mkl_sparse_destroy(h)
    if st != 0:
        raise RuntimeError(f"mkl_sparse_s_mm status {st}")
    return y
