"""Drop-in for the reference's pybind11 extension ``cbm.cbm_mkl_cpp``
(``/root/reference/cbm/cbm_extensions.cpp:1757-1771``): the same 13 function names with the
same positional arguments, forwarding to the C ABI of this package.

The reference functions take the delta matrix as a 4-array CSR with fp32 values and the tree
as ``mst_row`` / ``mst_col``; the kernels here want a level ordering instead, which is derived
from the tree arrays on every call (O(N) host work).  This module exists for code that talks
to the extension directly (``gnns/message_passing/mkl_message_passing.py:13,21`` uses the two
plain CSR functions); ``cbm_matrix`` does not go through it and caches everything.

``seq_*`` and ``omp_*`` names are the same GPU code.  CPU tensors are staged through the GPU;
there is no CPU implementation.
"""
from __future__ import annotations

import ctypes as C

import numpy as np
import torch

from . import _lib
from .cbm import _check_f32_matrix, _ld, _ptr, _require_gpu, _stream, tree_levels

__all__ = [
    "from_coo_int32_t_v1_", "from_coo_int32_t_v2_",
    "seq_s_spmm_update_csr_int32", "seq_s_update_csr_int32", "seq_s_spmm_csr_int32",
    "omp_s_spmm_update_csr_int32", "omp_s_update_avx_int32", "omp_s_update_csr_int32", "omp_s_spmm_csr_int32",
    "omp_s_fused_spmm_update_csr_int32", "omp_s_fused_update_csr_int32",
    "seq_s_fused_spmm_update_csr_int32", "seq_s_fused_update_csr_int32",
    "omp_s_spmm_update_csr_int32_v2",
]


def _i32(t, name):
    if t.dtype != torch.int32:
        raise RuntimeError(f"{name} (NOT torch::kInt32)")
    return t


def _f32(t, name):
    if t.dtype != torch.float32:
        raise RuntimeError(f"{name} (NOT torch::kFloat32)")
    return t


# ---------------------------------------------------------------------------------------------
# builders (cbm_extensions.cpp:8-326, :328-644)
# ---------------------------------------------------------------------------------------------
def _build(src_row, src_col, n_rows, n_cols, alpha, col_mul):
    if int(n_rows) != int(n_cols):
        raise ValueError("CBM is defined for square matrices")
    row = _i32(src_row, "src_row").detach().cpu().contiguous()
    col = _i32(src_col, "src_col").detach().cpu().contiguous()
    n = int(n_rows)
    fmt = _lib.CbmFormat()
    rc = _lib.host_lib().cbm_build_host(_ptr(row), _ptr(col), row.numel(), n, int(alpha), 0, C.byref(fmt))
    try:
        _lib.check(rc, "cbm_build_host")
        nnz = int(fmt.nnz)
        rowptr = np.ctypeslib.as_array(fmt.rowptr, shape=(n + 1,)).astype(np.int64)
        idx = np.ctypeslib.as_array(fmt.idx, shape=(max(nnz, 1),))[:nnz].copy()
        mst_row = torch.from_numpy(np.ctypeslib.as_array(fmt.mst_row, shape=(n + 2,)).copy())
        mst_col = torch.from_numpy(np.ctypeslib.as_array(fmt.mst_col, shape=(n,)).copy())
    finally:
        _lib.host_lib().cbm_format_free(C.byref(fmt))
    d_col = (idx & 0x7FFFFFFF).astype(np.int32)
    d_val = np.where(idx >> 31, -1.0, 1.0).astype(np.float32)
    if col_mul is not None:
        d_val = d_val * _f32(col_mul, "col_mul").detach().cpu().numpy()[d_col]
    d_row = np.repeat(np.arange(n, dtype=np.int32), np.diff(rowptr))
    return [mst_row, mst_col, torch.from_numpy(d_row), torch.from_numpy(d_col), torch.from_numpy(d_val)]


def from_coo_int32_t_v1_(src_row, src_col, src_val, src_n_rows, src_n_cols, alpha):
    """-> [mst_row (N+2), mst_col (N), delta_row, delta_col, delta_val (+-1)]"""
    return _build(src_row, src_col, src_n_rows, src_n_cols, alpha, None)


def from_coo_int32_t_v2_(src_row, src_col, src_val, col_mul, src_n_rows, src_n_cols, alpha):
    """-> same as v1 with delta_val = +-col_mul[delta_col]"""
    return _build(src_row, src_col, src_n_rows, src_n_cols, alpha, col_mul)


# ---------------------------------------------------------------------------------------------
# multiplies
# ---------------------------------------------------------------------------------------------
def _device_of(*tensors):
    for t in tensors:
        if t.is_cuda:
            return t.device
    _require_gpu()
    return torch.device("cuda", torch.cuda.current_device())


def _csr_spmm(row_b, row_e, col, val, rhs, dst_dev, dev):
    _i32(row_b, "lhs_row_b"); _i32(row_e, "lhs_row_e"); _i32(col, "lhs_col"); _f32(val, "lhs_val")
    n = dst_dev.size(0)
    if row_b.numel() != n or row_e.numel() != n:
        raise ValueError("row pointer arrays must have one entry per row of dst")
    # the reference passes the two slices of one crow array (cbm.py:145-146); rebuild it
    rowptr = torch.cat([row_b.detach().cpu().reshape(-1), row_e.detach().cpu().reshape(-1)[-1:]]).contiguous()
    if n > 1 and not torch.equal(rowptr[1:-1], row_e.detach().cpu().reshape(-1)[:-1]):
        raise ValueError("row_b / row_e must be the two slices of one row-pointer array")
    # device copies stay referenced until the launch is enqueued: a temporary freed earlier could
    # be handed out again by the caching allocator and overwritten by the next upload
    x = rhs.to(dev)
    rowptr_d, col_d, val_d = rowptr.to(dev), col.to(dev).contiguous(), val.to(dev).contiguous()
    rc = _lib.hip_lib().csr_spmm_f32(_ptr(rowptr_d), _ptr(col_d), col_d.numel(), _ptr(val_d), None, _ptr(x), _ptr(dst_dev), None,
                                     0, n, x.size(1), _ld(x), _ld(dst_dev), _stream(dev))
    _lib.check(rc, "csr_spmm_f32")


def _update(edges_src, edges_dst, multiplier, dst_dev, dev):
    _i32(edges_src, "edges_src"); _i32(edges_dst, "edge_dst")
    parent, order, level_off = tree_levels(edges_src.detach().cpu().numpy(), edges_dst.detach().cpu().numpy())
    parent_d, order_d = torch.from_numpy(parent).to(dev), torch.from_numpy(order).to(dev)
    lo_h = torch.from_numpy(level_off)
    lo_d = lo_h.to(dev)
    m_d = _f32(multiplier, "multiplier").to(dev).contiguous() if multiplier is not None else None
    rc = _lib.hip_lib().cbm_propagate_f32(_ptr(parent_d), _ptr(order_d), _ptr(lo_d), _ptr(lo_h), lo_h.numel() - 1,
                                          _ptr(m_d), _ptr(dst_dev), dst_dev.size(0), dst_dev.size(1), _ld(dst_dev),
                                          _lib.CBM_PROP_SCALE_ROOTS if m_d is not None else 0, _stream(dev))
    _lib.check(rc, "cbm_propagate_f32")


def _call(dst, rhs, body):
    _check_f32_matrix(dst, "dst")
    if rhs is not None:
        _check_f32_matrix(rhs, "rhs")
        if rhs.size(1) != dst.size(1):
            raise ValueError("rhs and dst differ in width")
    dev = _device_of(dst, *([rhs] if rhs is not None else []))
    with torch.cuda.device(dev):
        dst_dev = dst if dst.is_cuda else (torch.empty(dst.shape, dtype=dst.dtype, device=dev) if rhs is not None else dst.to(dev))
        body(dst_dev, dev)
        if dst_dev is not dst:
            dst.copy_(dst_dev)


def seq_s_spmm_csr_int32(lhs_row_b, lhs_row_e, lhs_col, lhs_val, rhs, dst):
    _call(dst, rhs, lambda y, dev: _csr_spmm(lhs_row_b, lhs_row_e, lhs_col, lhs_val, rhs, y, dev))


def seq_s_spmm_update_csr_int32(lhs_row_b, lhs_row_e, lhs_col, lhs_val, rhs, edges_src, edges_dst, dst):
    def body(y, dev):
        _csr_spmm(lhs_row_b, lhs_row_e, lhs_col, lhs_val, rhs, y, dev)
        _update(edges_src, edges_dst, None, y, dev)
    _call(dst, rhs, body)


def seq_s_update_csr_int32(edges_src, edges_dst, dst):
    _call(dst, None, lambda y, dev: _update(edges_src, edges_dst, None, y, dev))


def seq_s_fused_spmm_update_csr_int32(lhs_row_b, lhs_row_e, lhs_col, lhs_val, rhs, edges_src, edges_dst, multiplier, dst):
    def body(y, dev):
        _csr_spmm(lhs_row_b, lhs_row_e, lhs_col, lhs_val, rhs, y, dev)
        _update(edges_src, edges_dst, multiplier, y, dev)
    _call(dst, rhs, body)


def seq_s_fused_update_csr_int32(edges_src, edges_dst, multiplier, dst):
    _call(dst, None, lambda y, dev: _update(edges_src, edges_dst, multiplier, y, dev))


omp_s_spmm_csr_int32 = seq_s_spmm_csr_int32
omp_s_spmm_update_csr_int32 = seq_s_spmm_update_csr_int32
omp_s_spmm_update_csr_int32_v2 = seq_s_spmm_update_csr_int32   # named by cbm.py:225, never exported by the reference
omp_s_update_csr_int32 = seq_s_update_csr_int32
omp_s_update_avx_int32 = seq_s_update_csr_int32
omp_s_fused_spmm_update_csr_int32 = seq_s_fused_spmm_update_csr_int32
omp_s_fused_update_csr_int32 = seq_s_fused_update_csr_int32
