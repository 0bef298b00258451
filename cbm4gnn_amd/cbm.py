"""``cbm_matrix`` -- the reference's Python surface (``/root/reference/cbm/cbm.py:9-275``) over
the MI355X kernels.

Same constructor, same attributes (``deltas``, ``mst_row``, ``mst_col``, ``col_multiplier``) and
the same method names with the same in-place semantics, so the reference's message-passing
layers (``gnns/message_passing/cbm_message_passing.py:16-107``) and tests run against it
unchanged.  What differs is what happens behind the methods:

* construction calls the host builder ``cbm_build_host`` (packed-sign delta CSR + level
  ordering of the arborescence) instead of ``cbm_.from_coo_int32_t_v1_/_v2_``;
* every multiply runs the two HIP kernels through the C ABI on torch's current stream.
  The reference re-slices and re-casts the CSR arrays on every call (``cbm.py:145-148``); here
  the device copies of the format are made once per device and cached;
* ``seq_*`` and ``omp_*`` twins are the same GPU path (the distinction is CPU threading);
* CPU tensors are staged through the GPU (copy in, multiply, copy out).  There is no CPU
  implementation: without a GPU or without the built library every multiply raises.

Additions that the reference lacks: ``matmul`` / ``CBMMatmul`` with a correct autograd backward
(the reference's ``*_torch_csr_matmul`` differentiates only ``deltas @ x``, ``cbm.py:255-265``),
``compression_ratio`` (``benchmark/utility.py:45-64``) and the packed arrays themselves.
"""
from __future__ import annotations

import contextlib
import ctypes as C
import os
import warnings
import zipfile
import zlib
from collections import deque

import numpy as np
import torch

from . import _lib


@contextlib.contextmanager
def _quiet_sparse_csr():
    """torch announces on first use that sparse CSR support is in beta; the reference's ``deltas``
    attribute is such a tensor, so the notice is suppressed around its construction only."""
    with warnings.catch_warnings():
        warnings.filterwarnings("ignore", message="Sparse CSR tensor support is in beta state", category=UserWarning)
        yield


__all__ = ["cbm_matrix", "CBMMatmul", "csr_spmm", "tree_levels", "schedule_rows", "relayout_slabs"]


def _ptr(t):
    return C.c_void_p(t.data_ptr()) if t is not None else None


def _stream(device):
    """The current stream of ``device`` as a raw handle (what torch's own launches use; a small graph's
    multiply is bound by the host cost of issuing it, and ``torch.cuda.current_stream`` alone is 4 us)."""
    index = device.index if device.index is not None else torch.cuda.current_device()
    return C.c_void_p(torch._C._cuda_getCurrentRawStream(index))


_gpu_seen = False


def _require_gpu():
    global _gpu_seen
    if _gpu_seen:
        return
    if not torch.cuda.is_available():
        raise RuntimeError("cbm_matrix multiplies run on the GPU only and no HIP device is available "
                           "(there is no CPU fallback)")
    _gpu_seen = True


def _check_f32_matrix(t, name, n=None):
    # dtype errors mirror the TORCH_CHECKs of cbm_extensions.cpp:659-666; shape / layout checks
    # are new (the reference has none and reads out of bounds instead)
    if not isinstance(t, torch.Tensor):
        raise TypeError(f"{name} must be a torch.Tensor")
    if t.dtype != torch.float32:
        raise RuntimeError(f"{name} tensor (NOT torch::kFloat32)")
    if t.dim() != 2:
        raise ValueError(f"{name} must be 2-D [N, d], got shape {tuple(t.shape)}")
    if n is not None and t.size(0) != n:
        raise ValueError(f"{name} has {t.size(0)} rows, the matrix has {n}")
    if t.size(1) > 1 and t.stride(1) != 1:
        raise ValueError(f"{name} must be row-major with unit column stride")
    if t.size(0) > 1 and t.stride(0) < t.size(1):
        raise ValueError(f"{name} has overlapping rows (stride {t.stride(0)} < width {t.size(1)})")


# Rows with fewer delta entries than this on average do not repay the slab-major copy of X
_MIN_ENTRIES_PER_ROW_FOR_RELAYOUT = 24
# ... and while all of X is at most this many bytes (it stays in the L2s, and the copy is one more dependent
# launch of ~10 us) rows must average this many entries: 12,000 x 128 floats, 35 entries per row: 33.1 us with
# the copy, 27.1 us gathered in place; 194 entries per row: 79.9 / 80.9 us
_SMALL_X_BYTES = 8 << 20
_MIN_ENTRIES_PER_ROW_SMALL_X = 96


def _wants_workspace(x, y, nnz):
    """Whether a multiply of ``x`` into ``y`` brings a workspace for the slab-major copy of ``x``:
    when rows average enough entries for the copy to pay off, and, whatever the row length,
    when the width would otherwise run one wavefront per row (measured on 170 000 rows of 13
    entries, d = 40: 236 us without the copy, 120 us with it; d = 128: 178 vs 203 us)."""
    n, d = x.shape
    if n == 0 or d == 0:
        return False
    need = _MIN_ENTRIES_PER_ROW_SMALL_X if 4 * n * d <= _SMALL_X_BYTES else _MIN_ENTRIES_PER_ROW_FOR_RELAYOUT
    if nnz >= need * n:
        return True
    return int(_lib.hip_lib().cbm_spmm_summation_groups(d, _ld(x), _ld(y), _ptr(x), _ptr(y), 0)) == 1


def _workspace(x, y, nnz):
    """Device scratch for the slab-major copy of ``x``, or None when the library would not use it
    for this shape or the copy would not pay off.  Allocated from torch's stream-ordered caching
    allocator, so handing it to an asynchronous launch is safe."""
    if not _wants_workspace(x, y, nnz):
        return None
    n, d = x.shape
    floats = _lib.hip_lib().cbm_spmm_workspace_floats(n, d, _ld(x), _ld(y), _ptr(x), _ptr(y))
    return torch.empty(floats, dtype=torch.float32, device=x.device) if floats > 0 else None


def _ld(t):
    return t.stride(0) if t.size(0) > 1 else max(t.size(1), 1)


# Rows of at most this many delta entries are summed a batch at a time by the slab kernel (8 rows per
# wavefront, each lane group a row of its own, entries in order): ``cbm_schedule_rows_batched``.  0 = never.
# Measured on MI355X (ms per multiply at 0 / 8 / 16 / 32 / 64): 182,400 rows of 6 delta entries, d = 256:
# 0.55 / 0.33 / 0.32 / 0.32 / 0.32; 100,000 rows of 45, d = 256: 0.395 / 0.365 / 0.359 / 0.358 / 0.373;
# 12,000 rows of 35, d = 128: 0.038 / 0.038 / 0.038 / 0.033 / 0.034; rows of 200-300 entries: no change.
DEFAULT_BATCH_ROWS = 32


def schedule_rows(rowptr, parent=None, m=None, batch=0):
    """Row schedule of the SpMM kernels (``cbm_schedule_rows``): int32 tensor [n, 4] holding
    {start, end, row, bits(left scale)} per row, longest rows first.  ``batch`` > 0: the schedule of
    ``cbm_schedule_rows_batched`` -- rows of at most ``batch`` entries last, to be summed a batch at a time --
    as an [n + 1, 4] tensor whose last descriptor is the trailer (pass it with ``CBM_SPMM_SCHED_BATCHED``)."""
    rowptr = rowptr.to("cpu", torch.int32).contiguous()
    n = rowptr.numel() - 1
    parent = None if parent is None else parent.to("cpu", torch.int32).contiguous()
    m = None if m is None else m.to("cpu", torch.float32).contiguous()
    if batch:
        out = torch.empty((n + 1, 4), dtype=torch.int32)
        rc = _lib.host_lib().cbm_schedule_rows_batched(_ptr(rowptr), _ptr(parent), _ptr(m), n, int(batch), _ptr(out))
        _lib.check(rc, "cbm_schedule_rows_batched")
        return out
    out = torch.empty((n, 4), dtype=torch.int32)
    rc = _lib.host_lib().cbm_schedule_rows(_ptr(rowptr), _ptr(parent), _ptr(m), n, _ptr(out))
    _lib.check(rc, "cbm_schedule_rows")
    return out


def tree_levels(mst_row: np.ndarray, mst_col: np.ndarray):
    """(parent, order, level_off) from the reference's tree CSR (``mst_row`` [N+2], ``mst_col``
    [N], row N = virtual root).  parent is -1 for children of the root; order is sorted by
    (level, id)."""
    mst_row = np.asarray(mst_row, np.int64)
    mst_col = np.asarray(mst_col, np.int64)
    n = mst_col.shape[0]
    if mst_row.shape[0] != n + 2:
        raise ValueError("mst_row must have N + 2 entries")
    counts = np.diff(mst_row)
    parent = np.full(n, -2, np.int64)
    parent[mst_col] = np.repeat(np.arange(n + 1), counts)
    if (parent == -2).any():
        raise ValueError("tree does not cover every row")
    parent[parent == n] = -1
    level = np.full(n, -1, np.int64)
    frontier = mst_col[mst_row[n]:mst_row[n + 1]]
    depth = 0
    seen = 0
    while frontier.size:
        level[frontier] = depth
        seen += frontier.size
        cnt = counts[frontier]
        tot = int(cnt.sum())
        if tot == 0:
            break
        starts = np.repeat(mst_row[frontier], cnt)
        offs = np.arange(tot) - np.repeat(np.cumsum(cnt) - cnt, cnt)
        frontier = mst_col[starts + offs]
        depth += 1
    if seen != n:
        raise ValueError("tree is not connected to the root")
    order = np.lexsort((np.arange(n), level))
    n_levels = int(level.max()) + 1 if n else 0
    level_off = np.searchsorted(level[order], np.arange(n_levels + 1))
    return parent.astype(np.int32), order.astype(np.int32), level_off.astype(np.int32)


_GPU_BUILDER_MIN_EDGES = 2_000_000     # builder="auto": below this the host intersections are as fast as upload + kernel + download


def _first_pair_capacity(nnz):
    """Room for admissible pairs in the first pass of the GPU row intersections (12 B each); they
    rarely outnumber the entries of the matrix, and a second, exactly sized pass runs if they do."""
    return max(1 << 16, int(nnz))


def _build_staged(ei_cpu, n, alpha, threads, fmt, gpu, max_levels):
    """Staged build (``cbm_builder_*``); with ``gpu`` the row intersections run on the current HIP
    device (``cbm_row_intersections``).  Returns (status, seconds spent on upload + kernel +
    download or None)."""
    import time
    if gpu:
        _require_gpu()
    host, hip = _lib.host_lib(), _lib.hip_lib() if gpu else None
    handle = C.c_void_p()
    rc = host.cbm_builder_create(_ptr(ei_cpu[0].contiguous()), _ptr(ei_cpu[1].contiguous()), ei_cpu.size(1), n, threads,
                                 C.byref(handle))
    if rc:
        return rc, None
    try:
        if max_levels:
            rc = host.cbm_builder_set_max_levels(handle, int(max_levels))
            if rc:
                return rc, None
        if not gpu:
            return host.cbm_builder_finish(handle, alpha, None, -1, C.byref(fmt)), None
        ptrs = [C.c_void_p() for _ in range(6)]
        nnz = C.c_int64()
        rc = host.cbm_builder_arrays(handle, *[C.byref(p) for p in ptrs], C.byref(nnz))
        if rc:
            return rc, 0.0
        t0 = time.perf_counter()
        dev = torch.device("cuda", torch.cuda.current_device())

        def up(ptr, count, ctype, dtype):
            a = np.ctypeslib.as_array(C.cast(ptr, C.POINTER(ctype)), shape=(max(count, 1),))[:count]
            return torch.from_numpy(a).to(dev)                      # borrowed host memory, copied by .to()

        rowptr = up(ptrs[0], n + 1, C.c_int64, np.int64)
        col = up(ptrs[1], nnz.value, C.c_int32, np.int32)
        colptr_t = up(ptrs[2], n + 1, C.c_int64, np.int64)
        row_t = up(ptrs[3], nnz.value, C.c_int32, np.int32)
        after = up(ptrs[4], nnz.value, C.c_int64, np.int64)
        row_nnz = up(ptrs[5], n, C.c_int32, np.int32)
        with torch.cuda.device(dev):
            groups = int(hip.cbm_row_intersections_groups())
        capacity = _first_pair_capacity(nnz.value)
        while True:
            ticket = torch.zeros(1, dtype=torch.int32, device=dev)
            count = torch.zeros(1, dtype=torch.int64, device=dev)
            pairs = torch.empty((capacity, 3), dtype=torch.int32, device=dev)
            with torch.cuda.device(dev):
                rc = hip.cbm_row_intersections(_ptr(rowptr), _ptr(col), _ptr(colptr_t), _ptr(row_t), _ptr(after),
                                               _ptr(row_nnz), n, alpha, groups, _ptr(ticket), _ptr(pairs),
                                               capacity, _ptr(count), _stream(dev))
            if rc:
                return rc, 0.0
            found = int(count.item())                               # synchronises
            if found <= capacity:
                break
            del pairs
            capacity = found                                        # exact size, second pass
        pairs_host = pairs[:found].cpu().contiguous()
        t_pairs = time.perf_counter() - t0
        rc = host.cbm_builder_finish(handle, alpha, _ptr(pairs_host) if found else None, found, C.byref(fmt))
        return rc, t_pairs
    finally:
        host.cbm_builder_free(handle)


def edge_fingerprint(edge_index, n=None) -> np.ndarray:
    """Order-independent fingerprint of an edge list (uint64[4]: the number of edges, and three sums
    modulo 2^64 over a 64-bit mix z of every edge key row * N + col: of z, of z * z and of a second
    mix of z): equal for every ordering of the same edges, different -- for all practical purposes --
    when an edge changes.  It keys the on-disk cache of the built format (no security claim: the
    sums are additive)."""
    ei = torch.as_tensor(edge_index).detach().to("cpu")
    e = int(ei.size(1))
    if n is None:
        n = int(ei.max()) + 1 if e else 0

    def s64(v):                                           # a 64-bit constant as torch's signed int64
        return v - (1 << 64) if v >= (1 << 63) else v

    def lsr(z, k):                                        # logical shift right (torch's >> is arithmetic)
        return (z >> k) & ((1 << (64 - k)) - 1)

    sums = [0, 0, 0]
    for lo in range(0, e, 1 << 24):                       # int64 arithmetic wraps modulo 2^64
        r = ei[0, lo:lo + (1 << 24)].to(torch.int64)
        c = ei[1, lo:lo + (1 << 24)].to(torch.int64)
        z = r * n + c + s64(0x9E3779B97F4A7C15)           # splitmix64 finaliser
        z = (z ^ lsr(z, 30)) * s64(0xBF58476D1CE4E5B9)
        z = (z ^ lsr(z, 27)) * s64(0x94D049BB133111EB)
        z = z ^ lsr(z, 31)
        y = (z ^ lsr(z, 33)) * s64(0xFF51AFD7ED558CCD)    # second mix (murmur3 finaliser step)
        for i, t in enumerate((z, z * z, y ^ lsr(y, 29))):
            sums[i] = (sums[i] + int(t.sum())) & ((1 << 64) - 1)
    return np.array([e] + sums, np.uint64)


class cbm_matrix:

    def __init__(self, edge_index, values, rows=None, cols=None, alpha=0, normalized=False,
                 deltas_format="csr", threads=0, builder="auto", max_levels=None, tiling="auto"):
        ei = torch.as_tensor(edge_index)
        if ei.dim() != 2 or ei.size(0) != 2:
            raise ValueError("Edge index should have shape (2, num_edges)")
        ei_cpu = ei.detach().to("cpu", torch.int32).contiguous()
        if ei_cpu.size(1) == 0:
            raise ValueError("empty edge index")
        if int(ei_cpu.min()) < 0:
            raise ValueError("Edge index should start from 0")
        n = int(max(ei_cpu[0].max(), ei_cpu[1].max())) + 1          # cbm.py:15 (square matrix)
        for given in (rows, cols):
            if given is not None and int(given) != n:
                raise ValueError(f"rows/cols ({given}) do not match edge_index.max() + 1 ({n})")
        self.num_rows = n
        self.alpha = int(alpha)
        self.normalized = bool(normalized)
        self.deltas_format = deltas_format if deltas_format in ("csr", "coo") else "csr"

        # builder: "host" = everything on the CPU; "gpu" = the row intersections (the dominant cost
        # for large graphs) on the GPU, the rest on the CPU; "auto" = "gpu" when a HIP device is
        # there and the matrix is large enough to repay the transfers.  All give the same format.
        if builder not in ("auto", "host", "gpu"):
            raise ValueError('builder must be "auto", "host" or "gpu"')
        if builder == "auto":
            builder = "gpu" if (torch.cuda.is_available() and ei_cpu.size(1) >= _GPU_BUILDER_MIN_EDGES) else "host"
        self.builder = builder
        # max_levels: no tree level beyond this one (None = no limit, as the reference).  Rows that
        # would land deeper hang off the root instead: more delta entries, fewer dependent launches.
        if max_levels is not None and int(max_levels) < 1:
            raise ValueError("max_levels must be >= 1 (1 = flat tree)")
        self.max_levels = None if max_levels is None else int(max_levels)
        fmt = _lib.CbmFormat()
        rc, t_pairs = _build_staged(ei_cpu, n, self.alpha, int(threads), fmt, builder == "gpu", self.max_levels)
        try:
            _lib.check(rc, "cbm_build_host")
            t4 = (C.c_double * 4)()
            _lib.host_lib().cbm_build_host_timings(t4)
            self.build_seconds = dict(zip(("csr", "candidates", "arborescence", "deltas"), list(t4)))
            if t_pairs is not None:
                self.build_seconds["gpu_intersections"] = t_pairs       # upload + kernel + download, before "candidates"

            def take(ptr, count, dtype):
                return torch.from_numpy(np.ctypeslib.as_array(ptr, shape=(max(count, 1),))[:count].astype(dtype, copy=True))

            self.nnz = int(fmt.nnz)
            self.nnz_a = int(fmt.nnz_a)
            self.n_candidates = int(fmt.n_candidates)
            self.n_levels = int(fmt.n_levels)
            self.is_symmetric = bool(fmt.is_symmetric)
            self.rowptr = take(fmt.rowptr, n + 1, np.int32)
            # packed column | sign << 31; kept as the int32 bit pattern (torch has no uint32 math)
            self.idx = take(fmt.idx, self.nnz, np.uint32).view(torch.int32) if self.nnz else torch.empty(0, dtype=torch.int32)
            self.parent = take(fmt.parent, n, np.int32)
            self.order = take(fmt.order, n, np.int32)
            self.level_off = take(fmt.level_off, self.n_levels + 1, np.int32)
            self.mst_row = take(fmt.mst_row, n + 2, np.int32)
            self.mst_col = take(fmt.mst_col, n, np.int32)
        finally:
            _lib.host_lib().cbm_format_free(C.byref(fmt))

        if self.normalized:
            # m[i] = (#edges with row == i) ** -0.5, cbm.py:34-41 (there a Python loop per edge)
            deg = torch.bincount(ei_cpu[0].to(torch.int64), minlength=n).to(torch.float32)
            self.col_multiplier = deg.pow(-0.5)
        else:
            self.col_multiplier = None

        self._deltas = None
        self._dev = {}
        self._stream_coefficients = True    # see the property
        self._init_tiling(tiling)
        self.relayout = True                # False: gather from the caller's row-major X, no n*d scratch per call
        self._transposed = None
        self._edge_index_cpu = ei_cpu if not self.is_symmetric else None
        self._edge_fingerprint, self._fingerprint_source = None, ei_cpu      # computed on first use (save, from_cache)

    # ------------------------------------------------------------------ on-disk cache --------
    _SAVED_ARRAYS = ("rowptr", "idx", "parent", "order", "level_off", "mst_row", "mst_col")
    # 2 adds the depth limit (max_levels); 3 the fingerprint of the edge list the format was built from
    # (what from_cache checks).  Older files load with no depth limit / no fingerprint.
    FORMAT_VERSION = 3

    @staticmethod
    def _npz_path(path):
        """``np.savez`` appends ``.npz`` to a name without it; ``save`` and ``load`` agree on that."""
        path = str(path)
        return path if path.endswith(".npz") else path + ".npz"

    def save(self, path):
        """Write the built format to ``path`` (NumPy ``.npz``, no pickled objects).  The reference
        has no serialisation: every run rebuilds (``cbm_message_passing.py:22-25``)."""
        arrays = {k: getattr(self, k).numpy() for k in self._SAVED_ARRAYS}
        if self.col_multiplier is not None:
            arrays["col_multiplier"] = self.col_multiplier.numpy()
        if self._edge_index_cpu is not None:                      # needed to build the transposed operator
            arrays["edge_index"] = self._edge_index_cpu.numpy()
        meta = np.array([self.FORMAT_VERSION, self.num_rows, self.alpha, int(self.normalized), self.nnz, self.nnz_a,
                         self.n_candidates, self.n_levels, int(self.is_symmetric), self.max_levels or 0], np.int64)
        if self.edge_fingerprint is not None:
            arrays["edge_fingerprint"] = np.asarray(self.edge_fingerprint, np.uint64)
        # written under a temporary name in the same directory and renamed into place, so that a reader
        # (another process's ``from_cache``) sees the old file or the new one, never half of one
        final = self._npz_path(path)
        tmp = f"{final}.{os.getpid()}.tmp.npz"
        try:
            np.savez(tmp, meta=meta, deltas_format=np.array(self.deltas_format), **arrays)
            os.replace(tmp, final)
        finally:
            if os.path.exists(tmp):
                os.remove(tmp)

    @classmethod
    def load(cls, path):
        """Inverse of ``save``; runs no builder.  Everything a kernel would index with is checked on the
        host first (``_validate_loaded``): a stale, truncated or edited file raises ``ValueError`` here
        instead of becoming an out-of-bounds gather on the GPU.  The reference's only guard on a format
        is ``check_format`` (``cbm.py:69-115``), which needs the edge list; these checks need only the file."""
        path = cls._npz_path(path)
        try:
            z = np.load(path, allow_pickle=False)
        except (zipfile.BadZipFile, EOFError) as e:
            raise ValueError(f"{path} is not a readable .npz file: {e}") from None
        with z:
            try:
                meta = np.asarray(z["meta"]).tolist()
                if not isinstance(meta, list) or len(meta) < 9 or meta[0] not in (1, 2, cls.FORMAT_VERSION):
                    raise ValueError(f"unsupported CBM file version {meta[0] if isinstance(meta, list) and meta else meta}")
                self = cls.__new__(cls)
                (_, self.num_rows, self.alpha, normalized, self.nnz, self.nnz_a, self.n_candidates, self.n_levels,
                 symmetric) = [int(v) for v in meta[:9]]
                self.max_levels = (int(meta[9]) or None) if (meta[0] >= 2 and len(meta) > 9) else None
                self.normalized, self.is_symmetric = bool(normalized), bool(symmetric)
                self.deltas_format = str(z["deltas_format"])
                host = {k: z[k] for k in cls._SAVED_ARRAYS}
                m = z["col_multiplier"] if "col_multiplier" in z.files else None
                edges = z["edge_index"] if "edge_index" in z.files else None
                fingerprint = z["edge_fingerprint"].copy() if "edge_fingerprint" in z.files else None
            except (zipfile.BadZipFile, EOFError, zlib.error) as e:       # a member cut short or damaged
                raise ValueError(f"{path} is damaged: {e}") from None
            except KeyError as e:
                raise ValueError(f"{path} lacks the array {e}") from None
        problem = self._validate_loaded(host, m, edges, fingerprint)
        if problem:
            raise ValueError(f"{path} does not hold a consistent CBM format: {problem}")
        for k in cls._SAVED_ARRAYS:
            setattr(self, k, torch.from_numpy(np.ascontiguousarray(host[k]).view(np.int32).copy()))
        self._col_multiplier = None
        self.col_multiplier = torch.from_numpy(m.copy()) if m is not None else None
        self._edge_index_cpu = torch.from_numpy(edges.copy()) if edges is not None else None
        self._edge_fingerprint, self._fingerprint_source = fingerprint, None
        self.build_seconds = None
        self.builder = None                                 # loaded, not built
        self._deltas, self._dev, self._transposed = None, {}, None
        self._stream_coefficients = True
        self.relayout = True
        self._init_tiling("auto")
        return self

    def _validate_loaded(self, host, m, edges, fingerprint):
        """Why the arrays read from a file are not a format the kernels may run on (a string), or None.
        O(N + nnz) vectorised NumPy.  Checked: dtypes and lengths; row offsets start at 0, never decrease
        and end at nnz; every delta column is below N and columns ascend inside a row (the tiler and the
        column-block schedule rely on it); the tree arrays ``mst_row`` / ``mst_col`` describe a tree that
        covers every row from the virtual root, and ``parent`` / ``order`` / ``level_off`` are exactly the
        arrays that tree gives (so: parents in [-1, N), ``order`` a permutation sorted by (level, id), a
        row one level below its parent, offsets monotone from 0 to N); the normalisation vector is finite
        and positive; a directed matrix carries its edge list with ids below N."""
        n, nnz, levels = self.num_rows, self.nnz, self.n_levels
        if not (0 < n < 2 ** 31 and 0 <= nnz < 2 ** 31 and 0 < levels <= n and self.nnz_a >= 0 and self.n_candidates >= 0):
            return "sizes in the header are out of range"
        if self.max_levels is not None and not (0 < self.max_levels and levels <= self.max_levels):
            return "more tree levels than the depth limit in the header"
        if self.deltas_format not in ("csr", "coo"):
            return "unknown deltas_format"
        want_len = {"rowptr": n + 1, "idx": nnz, "parent": n, "order": n, "level_off": levels + 1, "mst_row": n + 2, "mst_col": n}
        for k, length in want_len.items():
            a = host[k]
            if a.dtype not in (np.dtype(np.int32), np.dtype(np.uint32)) or a.ndim != 1:
                return f"{k} is not a vector of 32-bit integers"
            if a.shape[0] != length:
                return f"{k} has {a.shape[0]} entries, expected {length}"
        rowptr = host["rowptr"].astype(np.int64)
        if rowptr[0] != 0 or rowptr[-1] != nnz or (np.diff(rowptr) < 0).any():
            return "rowptr does not run monotonically from 0 to nnz"
        col = (host["idx"].view(np.uint32) & np.uint32(0x7FFFFFFF)).astype(np.int64)
        if nnz and int(col.max()) >= n:
            return "a delta column is not below N"
        if nnz > 1:
            inside = np.ones(nnz - 1, bool)                 # pair (k, k+1) lies inside one row
            starts = rowptr[1:-1]
            inside[starts[(starts > 0) & (starts < nnz)] - 1] = False
            if (np.diff(col)[inside] <= 0).any():
                return "delta columns do not ascend inside a row"
        mst_row, mst_col = host["mst_row"].astype(np.int64), host["mst_col"].astype(np.int64)
        if mst_row[0] != 0 or mst_row[-1] != n or (np.diff(mst_row) < 0).any():
            return "mst_row does not run monotonically from 0 to N"
        if mst_col.min() < 0 or mst_col.max() >= n or np.bincount(mst_col, minlength=n).max() != 1:
            return "mst_col is not a permutation of the rows"
        try:
            parent, order, level_off = tree_levels(mst_row, mst_col)
        except ValueError as e:
            return f"mst_row / mst_col: {e}"
        for k, derived in (("parent", parent), ("order", order), ("level_off", level_off)):
            if derived.shape[0] != host[k].shape[0] or not np.array_equal(derived, host[k].view(np.int32)):
                return f"{k} is not what the tree in mst_row / mst_col gives"
        if (m is None) == self.normalized:
            return "normalisation flag and col_multiplier disagree"
        if m is not None and not (m.dtype == np.float32 and m.shape == (n,) and np.isfinite(m).all() and (m > 0).all()):
            return "col_multiplier is not a finite positive float32 vector of N entries"
        if not self.is_symmetric and edges is None:
            return "a directed matrix without its edge list"
        if edges is not None:
            if edges.dtype != np.int32 or edges.ndim != 2 or edges.shape[0] != 2 or edges.shape[1] == 0:
                return "edge_index is not an int32 [2, E] array"
            if edges.min() < 0 or edges.max() >= n:
                return "edge_index names a row that is not below N"
        if fingerprint is not None and not (fingerprint.dtype == np.uint64 and fingerprint.shape == (4,)):
            return "edge_fingerprint is not uint64[4]"
        return None

    @property
    def edge_fingerprint(self):
        """``edge_fingerprint`` of the edge list this matrix was built from (None for a matrix loaded
        from a file written before the fingerprint existed)."""
        if self._edge_fingerprint is None and self._fingerprint_source is not None:
            self._edge_fingerprint = edge_fingerprint(self._fingerprint_source, self.num_rows)
            self._fingerprint_source = None
        return self._edge_fingerprint

    @classmethod
    def from_cache(cls, path, edge_index, values=None, alpha=0, normalized=False, max_levels=None, **kwargs):
        """The format of ``edge_index`` from the file at ``path`` when that file was built from the
        same edges (``edge_fingerprint``) with the same ``alpha``, ``normalized`` and ``max_levels``;
        otherwise build it (``cbm_matrix(edge_index, values, alpha=..., ...)``) and write the file.
        The reference rebuilds on every run and caches only inside the process
        (``cbm_message_passing.py:22-29``)."""
        file = cls._npz_path(path)
        if os.path.exists(file):
            try:
                got = cls.load(file)
            except (ValueError, KeyError, OSError, zipfile.BadZipFile):
                got = None
            ei = torch.as_tensor(edge_index)
            if (got is not None and got.edge_fingerprint is not None and got.alpha == int(alpha)
                    and got.normalized == bool(normalized) and got.max_levels == (None if max_levels is None else int(max_levels))
                    and np.array_equal(got.edge_fingerprint, edge_fingerprint(ei, got.num_rows))):
                if "tiling" in kwargs:
                    got._init_tiling(kwargs["tiling"])
                return got
        built = cls(edge_index, values, alpha=alpha, normalized=normalized, max_levels=max_levels, **kwargs)
        built.save(file)
        return built

    # ------------------------------------------------------------------ tiling --------------
    # Entries that cluster in (256-row panel, 1024-column tile) blocks -- graphs with community
    # structure whose rows are ordered by community -- can be gathered from tiles of X staged in LDS
    # (``cbm_spmm_tiled_f32``) instead of through L1/L2.  "auto": use it when the matrix is large
    # and at least ``tile_min_local_fraction`` of its delta entries fall into blocks of at least
    # ``tile_min_block_entries`` entries; "on" / "off" force the choice.
    def _init_tiling(self, policy):
        if policy not in ("auto", "on", "off"):
            raise ValueError('tiling must be "auto", "on" or "off"')
        self.tiling = policy
        self.tile_rows = 1024
        self.tile_min_block_entries = 4096
        self.tile_min_local_fraction = 0.8
        self._tiling_host = None            # None: not computed; False: computed and rejected; dict: arrays
        self.tiling_info = None
        # Rows with more delta entries than this are cut into pieces of this many entries that different
        # wavefronts gather (``cbm_schedule_rows_split``); 0 = never cut.  A hub row of a power-law graph
        # would otherwise keep one wavefront per slab busy long after all others have finished.
        self.split_chunk = 2048
        # Column blocks: every row is also cut where its columns pass from one B-th of X to the next and the
        # pieces are scheduled block by block (``cbm_schedule_rows_blocks``), so that all wavefronts gather from
        # the same part of X at about the same time.  "auto": 2 for matrices that are not tiled, have at least
        # 100,000 rows and average at least 256 delta entries per row (long rows scattered over far more of X
        # than the L2s hold: 5.9 -> 5.2 ms on the 132,534-node dense-community graph at d = 512; shorter rows
        # lose more on the extra pieces than the L2 hits gain); an integer forces it (1 = off).
        self.column_blocks = "auto"
        # Trees of 2 .. CBM_PATH_MAX_LEVELS levels are walked in ONE launch after the SpMM (every row sums down
        # its own ancestor path, ``cbm_spmm_update_paths_f32``) while the product is at most this many bytes:
        # there a launch per level costs more than the level's work.  0 = always walk level by level.
        self.path_walk_max_bytes = 64 << 20
        # Products of at most this many bytes on shallow, sparse trees run as one launch (see _single_launch);
        # 0 = never.
        self.single_launch_max_bytes = 4 << 20
        # Trees deeper than the path walk takes: "auto" walks the rows below some level by SUBTREES in one launch
        # (``cbm_propagate_subtrees_f32``) when a cost estimate from the tree's shape says that beats one launch
        # per level; "on" / "off" force it; an integer forces it with that cut level.
        self.subtree_walk = "auto"
        self._walk_plans = {}
        # Deep trees with short delta rows: the whole multiply as ONE launch that walks the subtrees and sums
        # every row's delta entries on the way (``cbm_spmm_update_subtrees_f32``: the SpMM result never goes to
        # memory and back).  "auto": when an estimate says the launch is bound by the bytes it moves, not by its
        # longest bin (see stream_plan); "on": whenever the matrix is neither tiled nor has cut rows; "off".
        self.stream_multiply = "auto"
        self._batch_rows = DEFAULT_BATCH_ROWS

    def _path_gather_ratio(self):
        """(sum over rows of the delta entries on the row's ancestor path, itself included) / nnz: the extra
        gather work of computing every row's ancestors anew (1.0 = flat tree).  Computed once."""
        if getattr(self, "_path_ratio", None) is None:
            lens = (self.rowptr[1:] - self.rowptr[:-1]).to(torch.int64)
            cost = lens.clone()
            order, lo, parent = self.order.long(), self.level_off.tolist(), self.parent.long()
            for l in range(1, self.n_levels):                       # a level's parents are final before it
                rows = order[lo[l]:lo[l + 1]]
                cost[rows] = lens[rows] + cost[parent[rows]]
            self._path_ratio = float(cost.sum()) / max(self.nnz, 1)
        return self._path_ratio

    def _single_launch(self, n, d):
        """Whether ``*_spmm_update`` runs as ONE launch (``cbm_spmm_update_single_f32``: every row gathers its
        own delta entries and those of its ancestors): small products, where a launch costs more than the
        extra gathers -- at most ``single_launch_max_bytes`` of output, a tree of 2 .. 16 levels and at
        most 1.5 x the gather work."""
        return (1 < self.n_levels <= _lib.CBM_PATH_MAX_LEVELS and 0 < 4 * n * d <= int(self.single_launch_max_bytes)
                and self._path_gather_ratio() <= 1.5)

    def _walks_paths(self, n, d):
        return (1 < self.n_levels <= _lib.CBM_PATH_MAX_LEVELS and 0 < 4 * n * d <= int(self.path_walk_max_bytes))

    def _host_tiling(self):
        """What the plan-based multiply (``cbm_spmm_tiled_f32``) needs on the host, or False when this
        matrix does not use it: the split of the delta matrix into local blocks and remote entries
        (``cbm_tile_rows``) when the tiling policy and the matrix call for it, and/or the fact that
        rows longer than ``split_chunk`` exist and are to be cut.  Computed once."""
        if self._tiling_host is not None:
            return self._tiling_host
        n = self.num_rows
        self._tiling_host = False
        if self.nnz == 0:
            return False
        cut = bool(self.split_chunk) and int((self.rowptr[1:] - self.rowptr[:-1]).max()) > int(self.split_chunk)
        if self.column_blocks == "auto":
            col_blocks = 2 if (n >= 100_000 and self.nnz >= 256 * n) else 1
        else:
            col_blocks = max(int(self.column_blocks), 1)
        tile = self.tiling != "off" and not (self.tiling == "auto" and (n < 16 * self.tile_rows or self.nnz < 32 * n))
        arrays = None
        if tile:                                            # "auto" on small matrices: tiles of 1024 rows cannot pay
            t = _lib.CbmTiling()
            rc = _lib.host_lib().cbm_tile_rows(_ptr(self.rowptr), _ptr(self.idx), n, self.tile_rows,
                                               self.tile_min_block_entries, 0, C.byref(t))
            try:
                _lib.check(rc, "cbm_tile_rows")
                info = {"n_blocks": int(t.n_blocks), "nnz_local": int(t.nnz_local), "nnz_remote": int(t.nnz_remote),
                        "local_fraction": t.nnz_local / max(self.nnz, 1), "has_negative": bool(t.has_negative)}
                self.tiling_info = info
                if t.n_blocks > 0 and not (self.tiling == "auto" and info["local_fraction"] < self.tile_min_local_fraction):

                    def take(ptr, count, dtype):
                        return torch.from_numpy(np.ctypeslib.as_array(ptr, shape=(max(count, 1),))[:count].astype(dtype, copy=True))

                    p1 = t.panel_rows + 1
                    arrays = {
                        "n_panels": int(t.n_panels), "n_blocks": int(t.n_blocks), "tile_rows": int(t.tile_rows),
                        "has_negative": int(t.has_negative), "nnz_remote": int(t.nnz_remote),
                        "panel_ptr": take(t.panel_ptr, t.n_panels + 1, np.int32), "blk_tile": take(t.blk_tile, t.n_blocks, np.int32),
                        "seg": take(t.seg, t.n_blocks * p1, np.int32),
                        "lidx": take(t.lidx, t.nnz_local_padded, np.uint16).view(torch.int16),
                        "rowptr_r": take(t.rowptr_r, n + 1, np.int32),
                        "idx_r": (take(t.idx_r, t.nnz_remote, np.uint32).view(torch.int32) if t.nnz_remote
                                  else torch.empty(0, dtype=torch.int32)),
                    }
            finally:
                _lib.host_lib().cbm_tiling_free(C.byref(t))
        if arrays is not None:
            col_blocks = 1                                  # the remote part of a tiled matrix has short rows
        if arrays is None and (cut or col_blocks > 1):      # no local blocks: the whole matrix is "remote"
            arrays = {"n_panels": (n + 255) // 256, "n_blocks": 0, "tile_rows": self.tile_rows, "has_negative": 0,
                      "nnz_remote": self.nnz, "panel_ptr": torch.zeros((n + 255) // 256 + 1, dtype=torch.int32),
                      "rowptr_r": self.rowptr, "idx_r": self.idx}
        if arrays is not None:
            arrays["col_blocks"] = col_blocks
            arrays["cut"] = col_blocks > 1 or (bool(self.split_chunk) and
                                               int((arrays["rowptr_r"][1:] - arrays["rowptr_r"][:-1]).max()) > int(self.split_chunk))
            self._tiling_host = arrays
        return self._tiling_host

    def is_tiled(self):
        """Whether multiplies of this matrix gather local blocks from LDS tiles (decides it on first call)."""
        th = self._host_tiling()
        return bool(th) and th["n_blocks"] > 0

    def has_cut_rows(self):
        """Whether the multiply cuts rows longer than ``split_chunk`` into pieces."""
        th = self._host_tiling()
        return bool(th) and th["cut"]

    def _split_schedule(self, rowptr, idx, parent, m, col_blocks=1):
        """(sched [count, 4], long_rows [n_long, 4], pieces) of ``cbm_schedule_rows_blocks``, CPU tensors."""
        n = rowptr.numel() - 1
        n_long = C.c_int32()
        chunk = int(self.split_chunk or 0)
        count = _lib.host_lib().cbm_schedule_blocks_count(_ptr(rowptr), _ptr(idx), n, chunk, int(col_blocks), C.byref(n_long))
        if count < 0:
            raise ValueError("cbm_schedule_blocks_count: bad row offsets, chunk size or block count")
        sched = torch.empty((count, 4), dtype=torch.int32)
        long_rows = torch.empty((max(n_long.value, 1), 4), dtype=torch.int32)
        rc = _lib.host_lib().cbm_schedule_rows_blocks(_ptr(rowptr), _ptr(idx), _ptr(parent), _ptr(m), n, chunk, int(col_blocks),
                                                      _ptr(sched), _ptr(long_rows))
        _lib.check(rc, "cbm_schedule_rows_blocks")
        long_rows = long_rows[:n_long.value]
        return sched, long_rows, int(long_rows[:, 2].sum()) if n_long.value else 0

    # ------------------------------------------------------------------ walk by subtrees -----
    # Rough costs of the two ways to walk a deep tree, in microseconds (measured on MI355X: a dependent launch
    # of a small kernel, one level of the register-carried chain, one row of a subtree sequence, and the rate
    # at which wide levels stream rows).  They only rank the plans of one tree against each other.
    _WALK_US_PER_LAUNCH = 4.0
    _WALK_US_PER_NARROW_LEVEL = 2.0
    _WALK_US_PER_CHAIN_LEVEL = 0.085
    _WALK_US_PER_ENTRY = 0.125
    _WALK_BYTES_PER_US = 4.0e6

    def _level_plan_cost_us(self, d, first_level=1, last_level=None):
        """Estimated time of the level-by-level launches for levels first_level .. last_level - 1."""
        lo = self.level_off.tolist()
        levels = self.n_levels if last_level is None else last_level
        width = lambda l: lo[l + 1] - lo[l]

        def chain_end(l):
            while l < levels and width(l) == 1:
                l += 1
            return l

        cost, l = 0.0, first_level
        while l < levels:
            if width(l) == 1 and chain_end(l) - l >= 4:
                e = chain_end(l)
                cost += self._WALK_US_PER_LAUNCH + (e - l) * self._WALK_US_PER_CHAIN_LEVEL
                l = e
            elif width(l) <= 64:
                e = l + 1
                while e < levels and width(e) <= 64 and chain_end(e) - e < 4:
                    e += 1
                cost += self._WALK_US_PER_LAUNCH + (e - l) * self._WALK_US_PER_NARROW_LEVEL
                l = e
            else:
                cost += max(self._WALK_US_PER_LAUNCH, width(l) * d * 12 / self._WALK_BYTES_PER_US)
                l += 1
        return cost

    def _host_walk_plan(self, cut, d):
        """``cbm_walk_plan_build`` for this tree at ``cut`` (CPU tensors + stats), cached.  The bins are sized so
        that (bins x 64-column slices) wavefronts fill the GPU a few times over."""
        target_bins = self._walk_bin_target(d)
        key = (int(cut), target_bins)
        plan = self._walk_plans.get(key)
        if plan is None:
            p = _lib.CbmWalkPlan()
            rc = _lib.host_lib().cbm_walk_plan_build(_ptr(self.parent), _ptr(self.order), _ptr(self.level_off), self.num_rows,
                                                     self.n_levels, int(cut), target_bins, C.byref(p))
            try:
                if rc == 6:                                 # more live slots than the kernel has: not for this tree
                    plan = False
                else:
                    _lib.check(rc, "cbm_walk_plan_build")
                    take = lambda ptr, count: torch.from_numpy(
                        np.ctypeslib.as_array(ptr, shape=(max(count, 1),))[:count].astype(np.int32, copy=True))
                    plan = {"cut": int(p.cut), "n_entries": int(p.n_entries), "n_bins": int(p.n_bins), "n_slots": int(p.n_slots),
                            "longest_bin": int(p.longest_bin),
                            "entries": take(p.entries, 2 * p.n_entries).view(-1, 2), "bin_off": take(p.bin_off, p.n_bins + 1)}
            finally:
                _lib.host_lib().cbm_walk_plan_free(C.byref(p))
            self._walk_plans[key] = plan
        return plan

    def _subtree_plan_cost_us(self, plan, d):
        return (self._level_plan_cost_us(d, 1, plan["cut"] + 1) + self._WALK_US_PER_LAUNCH +
                max(plan["longest_bin"] * self._WALK_US_PER_ENTRY, plan["n_entries"] * d * 8 / self._WALK_BYTES_PER_US))

    def walk_plan(self, d):
        """The subtree-walk plan a multiply of width ``d`` uses, or None when it walks level by level: by
        ``subtree_walk`` -- "off": None; an integer: that cut; "on": the cheapest cut by the estimate; "auto":
        the cheapest cut if the estimate beats the level-by-level launches by a fifth.  (A multiply that the
        one-launch path walk takes -- a shallow tree, a small product -- does not ask.)"""
        policy = self.subtree_walk
        if policy == "off" or self.n_levels < 2:
            return None
        if isinstance(policy, int) and not isinstance(policy, bool):
            return self._host_walk_plan(min(max(policy, 0), self.n_levels - 2), d) or None
        if policy not in ("auto", "on"):
            raise ValueError('subtree_walk must be "auto", "on", "off" or a cut level')
        key = ("choice", policy, (d + 63) // 64)
        if key not in self._walk_plans:
            # candidates: every cut level up to 16 (deeper cuts pay a launch per level above them anyway),
            # ranked by the estimate from the subtree sizes alone; only the winner's plan is built
            sizes, target = self._subtree_sizes(), self._walk_bin_target(d)
            lo, order = self.level_off.tolist(), self.order.numpy()
            best_cut, best_cost = None, None
            for cut in range(0, min(self.n_levels - 1, 16)):
                heads = sizes[order[lo[cut]:lo[cut + 1]]]
                heads = heads[heads > 1]
                if heads.size == 0:
                    continue
                entries = int(heads.sum())
                longest = max(int(heads.max()), -(-entries // target), 32)   # small subtrees are packed into bins
                cost = (self._level_plan_cost_us(d, 1, cut + 1) + self._WALK_US_PER_LAUNCH +
                        max(longest * self._WALK_US_PER_ENTRY, entries * d * 8 / self._WALK_BYTES_PER_US))
                if best_cut is None or cost < best_cost:
                    best_cut, best_cost = cut, cost
            best = self._host_walk_plan(best_cut, d) if best_cut is not None else None
            if best and policy == "auto" and self._subtree_plan_cost_us(best, d) > 0.8 * self._level_plan_cost_us(d):
                best = None
            self._walk_plans[key] = best or None
        return self._walk_plans[key]

    # The launch of the multiply by subtrees takes the longer of: the wavefront with the heaviest bin alone (this
    # long per stream entry, a row weighing CBM_STREAM_ROW_COST entries more for its walk step and store), and
    # the bytes of the launch (every stream entry's row of X, every row of Y once) at the second rate.  The SpMM
    # of short rows moves its bytes at the third.  Measured on staircase graphs of 11,400 .. 280,000 rows, 3 ..
    # 16 entries per delta row, d = 64 .. 512 (within 10 %).
    _STREAM_US_PER_WEIGHT = 0.041
    _STREAM_BYTES_PER_US = 7.5e6
    _SHORT_ROW_SPMM_BYTES_PER_US = 6.5e6
    _STREAM_MAX_ENTRIES_PER_ROW = 24          # "auto" asks only where the slab-major copy of X would not pay either

    @staticmethod
    def _stream_bin_target(d):
        """Bins a multiply stream aims for: (bins x 64-column slices) wavefronts fill the GPU several times over."""
        return max(64, 16384 // ((d + 63) // 64))

    def _host_stream(self, d):
        """``cbm_walk_stream_build`` for this matrix (CPU tensors + stats), cached per bin target; False when the
        tree needs more kept values than the kernel has slots (or more than 2^29 rows)."""
        target_bins = self._stream_bin_target(d)
        key = ("stream", target_bins)
        plan = self._walk_plans.get(key)
        if plan is None:
            p = _lib.CbmWalkStream()
            idx = self.idx.contiguous()
            rc = _lib.host_lib().cbm_walk_stream_build(
                _ptr(self.rowptr), _ptr(idx), _ptr(self.parent), _ptr(self.order), _ptr(self.level_off), self.num_rows,
                self.n_levels, target_bins, C.byref(p)) if self.num_rows <= _lib.CBM_STREAM_COL_MASK else 6
            try:
                if rc == 6:
                    plan = False
                else:
                    _lib.check(rc, "cbm_walk_stream_build")
                    take = lambda ptr, count: torch.from_numpy(
                        np.ctypeslib.as_array(ptr, shape=(max(count, 1),))[:count].astype(np.int32, copy=True))
                    plan = {"n_bins": int(p.n_bins), "n_slots": int(p.n_slots), "n_elems": int(p.n_elems),
                            "heaviest_bin": int(p.heaviest_bin), "gidx": take(p.gidx, p.n_elems),
                            "ginfo": take(p.ginfo, 2 * p.n_elems).view(-1, 2), "bin_goff": take(p.bin_goff, p.n_bins + 1)}
            finally:
                _lib.host_lib().cbm_walk_stream_free(C.byref(p))
            self._walk_plans[key] = plan
        return plan

    def _stream_weights(self):
        """Weight of the subtree of every row in the multiply stream (a row: its delta entries, an empty row one,
        + CBM_STREAM_ROW_COST), int64 NumPy; computed once."""
        weights = self._walk_plans.get("weights")
        if weights is None:
            weights = np.maximum(np.diff(self.rowptr.numpy().astype(np.int64)), 1) + _lib.CBM_STREAM_ROW_COST
            lo, order, parent = self.level_off.tolist(), self.order.numpy(), self.parent.numpy()
            for l in range(self.n_levels - 1, 0, -1):                       # leaves first
                rows = order[lo[l]:lo[l + 1]]
                np.add.at(weights, parent[rows], weights[rows])
            self._walk_plans["weights"] = weights
        return weights

    def _stream_cost_us(self, heaviest_bin, d):
        """Estimate for the one-launch multiply by subtrees (see the constants above)."""
        n = self.num_rows
        entries = max(self.nnz, n)                                          # about: empty rows count one
        return self._WALK_US_PER_LAUNCH + max(heaviest_bin * self._STREAM_US_PER_WEIGHT,
                                              (entries + n) * d * 4 / self._STREAM_BYTES_PER_US)

    def _two_launch_cost_us(self, d):
        """Estimate for the same product as SpMM (short rows, gathered in place) + walk."""
        n = self.num_rows
        spmm = self._WALK_US_PER_LAUNCH + (self.nnz + n) * d * 4 / self._SHORT_ROW_SPMM_BYTES_PER_US
        if self._walks_paths(n, d):
            return spmm + 2 * self._WALK_US_PER_LAUNCH                      # the one-launch path walk of a shallow tree
        plan = self.walk_plan(d)
        return spmm + (self._subtree_plan_cost_us(plan, d) if plan is not None else self._level_plan_cost_us(d))

    def stream_plan(self, d):
        """The plan of the one-launch multiply by subtrees for width ``d``, or None when the multiply runs as
        SpMM + walk: by ``stream_multiply`` -- "off": None; "on": the plan whenever the tree has two levels or
        more and the matrix is neither tiled nor has cut rows; "auto": the plan when delta rows average at most
        24 entries (the rows the SpMM gathers in place) and an estimate from the shape of the tree and the
        lengths of the rows puts the launch at 0.85 of the SpMM + walk or below -- it moves fewer bytes (no SpMM
        result written and read back) but runs one wavefront per bin of whole subtrees, so few large subtrees
        or narrow matrices keep the two launches."""
        policy = self.stream_multiply
        if policy == "off" or self.n_levels < 2 or self.num_rows == 0 or d <= 0:
            return None
        if policy not in ("auto", "on"):
            raise ValueError('stream_multiply must be "auto", "on" or "off"')
        if self._host_tiling():
            return None
        key = ("stream-choice", policy, d if policy == "auto" else (d + 63) // 64, self.subtree_walk if policy == "auto" else None)
        if key not in self._walk_plans:
            take = True
            if policy == "auto":
                take = self.nnz <= self._STREAM_MAX_ENTRIES_PER_ROW * self.num_rows
                if take:
                    weights, target = self._stream_weights(), self._stream_bin_target(d)
                    heads = weights[self.order.numpy()[:int(self.level_off[1])]]
                    heaviest = max(int(heads.max()), -(-int(heads.sum()) // target), 64)    # small subtrees are packed into bins
                    take = self._stream_cost_us(heaviest, d) <= 0.85 * self._two_launch_cost_us(d)
            self._walk_plans[key] = (self._host_stream(d) or None) if take else None
        return self._walk_plans[key]

    def _stream_struct(self, st, plan):
        """``struct cbm_walk_stream_dev`` over the device copy of ``plan`` (uploaded once per device)."""
        key = ("stream", plan["n_bins"], plan["n_elems"])
        dev = st.get(key)
        if dev is None:
            device = st["rowptr"].device
            dev = st[key] = (plan["gidx"].to(device), plan["ginfo"].contiguous().to(device), plan["bin_goff"].to(device))
        return _lib.CbmWalkStreamDev(self.num_rows, plan["n_bins"], plan["n_slots"], plan["n_elems"], dev[0].data_ptr(),
                                     dev[1].data_ptr(), dev[2].data_ptr())

    def _subtree_sizes(self):
        """Rows in the subtree of every row (itself included), int64 NumPy; computed once."""
        sizes = self._walk_plans.get("sizes")
        if sizes is None:
            sizes = np.ones(self.num_rows, np.int64)
            lo, order, parent = self.level_off.tolist(), self.order.numpy(), self.parent.numpy()
            for l in range(self.n_levels - 1, 0, -1):                       # leaves first
                rows = order[lo[l]:lo[l + 1]]
                np.add.at(sizes, parent[rows], sizes[rows])
            self._walk_plans["sizes"] = sizes
        return sizes

    @staticmethod
    def _walk_bin_target(d):
        """Bins a plan aims for: (bins x 64-column slices) wavefronts fill the GPU a few times over."""
        return max(64, 8192 // ((d + 63) // 64))

    def _walk_struct(self, st, plan):
        """``struct cbm_walk_dev`` over the device copy of ``plan`` (uploaded once per device and cut)."""
        key = ("walk", plan["cut"], plan["n_bins"])
        dev = st.get(key)
        if dev is None:
            device = st["rowptr"].device
            dev = st[key] = (plan["entries"].contiguous().to(device), plan["bin_off"].to(device))
        return _lib.CbmWalkDev(plan["cut"], plan["n_entries"], plan["n_bins"], plan["n_slots"], dev[0].data_ptr(), dev[1].data_ptr())

    # Settings the cached device arrays depend on: changing one drops the cache, so that a later
    # multiply never runs on coefficients or schedules derived from the old value.
    @property
    def stream_coefficients(self):
        """True (default): the SpMM streams ``+-m[col]`` per delta entry, expanded once per device;
        False: it gathers ``m[col]`` in the kernel, 4 B per entry less device memory."""
        return self._stream_coefficients

    @stream_coefficients.setter
    def stream_coefficients(self, value):
        if bool(value) != self._stream_coefficients:
            self._dev = {}
        self._stream_coefficients = bool(value)

    @property
    def batch_rows(self):
        """Rows of at most this many delta entries are summed a batch at a time by the slab kernel, each lane
        group a row of its own, entries strictly in order (``cbm_schedule_rows_batched``); 0 = every row is
        summed by a whole wavefront."""
        return self._batch_rows

    @batch_rows.setter
    def batch_rows(self, value):
        if not 0 <= int(value) <= 64:
            raise ValueError("batch_rows must be 0 .. 64")
        if int(value) != self._batch_rows:
            self._dev = {}
        self._batch_rows = int(value)

    @property
    def col_multiplier(self):
        return self._col_multiplier

    @col_multiplier.setter
    def col_multiplier(self, value):
        self._col_multiplier = value
        self._dev, self._deltas = {}, None

    # ------------------------------------------------------------------ format views --------
    def columns(self):
        """Delta column indices (int64) and signs (+1/-1, fp32), unpacked from ``idx``."""
        col = (self.idx & 0x7FFFFFFF).to(torch.int64)
        sign = torch.where(self.idx < 0, -1.0, 1.0).to(torch.float32)
        return col, sign

    @property
    def deltas(self):
        """Delta matrix as a torch sparse tensor with values +-1 (or +-m[col] when normalised),
        what the reference keeps in ``self.deltas`` (``cbm.py:56-66``).  Built on first use."""
        if self._deltas is None:
            col, val = self.columns()
            if self.col_multiplier is not None:
                val = val * self.col_multiplier[col]
            n = self.num_rows
            with _quiet_sparse_csr():
                csr = torch.sparse_csr_tensor(self.rowptr.to(torch.int64), col, val, size=(n, n))
            self._deltas = csr if self.deltas_format == "csr" else csr.to_sparse_coo().coalesce()
        return self._deltas

    def to_sparse_coo_tensor(self, row, col, val, data_type=torch.float32):
        """COO triplets -> coalesced torch COO tensor (``cbm.py:120-129``)."""
        size = int(max(row.max(), col.max())) + 1
        index = torch.stack((row.to(torch.int64), col.to(torch.int64)))
        return torch.sparse_coo_tensor(index, val, size=(size, size)).to(data_type).coalesce()

    def to_sparse_csr_tensor(self, row, col, val, data_type=torch.float32):
        """COO triplets -> torch CSR tensor (``cbm.py:132-141``)."""
        with _quiet_sparse_csr():
            return self.to_sparse_coo_tensor(row, col, val, data_type).to_sparse_csr()

    def compression_ratio(self):
        """Element-count ratio CSR(A) / CBM, ``benchmark/utility.py:45-64``."""
        n = self.num_rows
        return (n + 1 + 2 * self.nnz_a) / (n + 1 + 2 * self.nnz + (n + 2) + n)

    def check_format(self, edge_index):
        """Rebuild every row from the tree and the signed deltas and compare with the adjacency
        lists (``cbm.py:69-115``).  Raises ``ValueError`` on any mismatch."""
        ei = torch.as_tensor(edge_index).to("cpu", torch.int64)
        n_rows = int(ei[0].max()) + 1
        rowptr = self.rowptr.tolist()
        col, sign = self.columns()
        col = col.tolist(); sign = sign.tolist()
        mst_row = self.mst_row.tolist(); mst_col = self.mst_col.tolist()
        s = [set() for _ in range(n_rows + 1)]
        queue = deque([n_rows])
        visited = 0
        while queue:
            u = queue.popleft()
            for v in mst_col[mst_row[u]:mst_row[u + 1]]:
                queue.append(v)
                visited += 1
                sv = set(s[u])
                for k in range(rowptr[v], rowptr[v + 1]):
                    if sign[k] > 0:
                        sv.add(col[k])
                    else:
                        sv.remove(col[k])
                s[v] = sv
        if visited != n_rows:
            raise ValueError("Format is incorrect!")
        a = [set() for _ in range(n_rows)]
        for r, c in zip(ei[0].tolist(), ei[1].tolist()):
            a[r].add(c)
        for v in range(n_rows):
            if s[v] != a[v]:
                raise ValueError("Format is incorrect!")
        return True

    # ------------------------------------------------------------------ device state --------
    def _device_arrays(self, device):
        device = torch.device(device)
        key = (device.type, device.index if device.index is not None else torch.cuda.current_device())
        st = self._dev.get(key)
        if st is None:
            st = {
                "rowptr": self.rowptr.to(device), "idx": self.idx.to(device), "parent": self.parent.to(device),
                "order": self.order.to(device), "level_off": self.level_off.to(device),
                "m": self.col_multiplier.to(device) if self.col_multiplier is not None else None,
                "coef": None,
                # row schedules (longest rows first): without and with the left scale of root children
                "sched": schedule_rows(self.rowptr, None, None, self.batch_rows).to(device),
                "sched_scaled": (schedule_rows(self.rowptr, self.parent, self.col_multiplier, self.batch_rows).to(device)
                                 if self.col_multiplier is not None else None),
            }
            th = self._host_tiling()
            st["tiled"] = None
            if th:
                tiled = th["n_blocks"] > 0
                if tiled:
                    tensors = {k: th[k].to(device) for k in ("panel_ptr", "blk_tile", "seg", "lidx", "rowptr_r", "idx_r")}
                else:                                        # the remote part is the matrix itself
                    tensors = {"panel_ptr": th["panel_ptr"].to(device), "rowptr_r": st["rowptr"], "idx_r": st["idx"]}
                # schedules of the remote part.  With local blocks the left scale is applied by their kernel
                # (row_scale); without, by the schedule, which then exists with and without the scales.
                scaled = (None, None) if (tiled or self.col_multiplier is None) else (self.parent, self.col_multiplier)
                for name, (par, mm) in (("plain", (None, None)), ("scaled", scaled)):
                    if name == "scaled" and par is None:
                        continue
                    if th["cut"]:
                        sched, long_rows, pieces = self._split_schedule(th["rowptr_r"], th["idx_r"], par, mm, th["col_blocks"])
                        tensors["sched_" + name] = sched.to(device)
                        tensors["long_" + name] = long_rows.to(device)
                        tensors["n_long"], tensors["n_pieces"], tensors["n_sched"] = long_rows.size(0), pieces, sched.size(0)
                    else:
                        tensors["sched_" + name] = schedule_rows(th["rowptr_r"], par, mm).to(device)
                        tensors["n_long"], tensors["n_pieces"], tensors["n_sched"] = 0, 0, 0
                if tiled and self.col_multiplier is not None:    # left scale: m[r] for children of the root
                    scale = torch.where(self.parent < 0, self.col_multiplier, torch.ones_like(self.col_multiplier))
                    tensors["row_scale"] = scale.to(device)
                st["tiled"] = tensors
            self._dev[key] = st
        return st

    def _tiled_struct(self, st, with_scale):
        """``struct cbm_tiling_dev`` over the device tensors of ``st`` (host-side struct, per call)."""
        th, tt = self._tiling_host, st["tiled"]
        tiled = th["n_blocks"] > 0
        flavour = "scaled" if (with_scale and not tiled and "sched_scaled" in tt) else "plain"
        ptr = lambda name: tt[name].data_ptr() if (name in tt and tt[name].numel()) else None
        return _lib.CbmTilingDev(th["n_panels"], th["n_blocks"], th["tile_rows"], th["has_negative"], th["nnz_remote"],
                                 ptr("panel_ptr"), ptr("blk_tile"), ptr("seg"), ptr("lidx"), ptr("rowptr_r"), ptr("idx_r"),
                                 ptr("sched_" + flavour), ptr("row_scale") if (with_scale and tiled) else None,
                                 tt["n_sched"], tt["n_long"], tt["n_pieces"], 0, ptr("long_" + flavour))

    def workspace_floats(self, n, d, device):
        """Floats of workspace a multiply of an [n, d] matrix on ``device`` uses at most: the slab-major
        copy of X, plus the piece sums of cut rows."""
        floats = int(_lib.hip_lib().cbm_relayout_floats(n, d))
        st = self._device_arrays(device)
        if st["tiled"] is not None:
            floats = max(floats, int(_lib.hip_lib().cbm_spmm_tiled_workspace_floats(C.byref(self._tiled_struct(st, False)), n, d)))
        return max(floats, 1)

    def _tiled_workspace(self, xd, workspace=None):
        need = self.workspace_floats(xd.size(0), xd.size(1), xd.device)
        if workspace is None:
            return torch.empty(need, dtype=torch.float32, device=xd.device)
        if workspace.numel() < need:
            raise ValueError(f"workspace holds {workspace.numel()} floats, this multiply needs {need} "
                             "(cbm_matrix.workspace_floats)")
        return workspace

    def _coef(self, st, device):
        """``+-m[col]`` per delta entry on ``device`` (what the reference keeps as the fp32 values of
        its delta matrix), expanded on first need: only a normalised multiply that gathers from
        the caller's row-major X streams it -- one that copies X slab-major scales the copy by
        ``m`` instead and needs no coefficient per entry.  None when ``stream_coefficients`` is off."""
        if st["m"] is None or not self.nnz or not self.stream_coefficients:
            return None
        if st["coef"] is None:
            st["coef"] = torch.empty(self.nnz, dtype=torch.float32, device=device)
            with torch.cuda.device(device):
                rc = _lib.hip_lib().cbm_expand_coef_f32(_ptr(st["idx"]), _ptr(st["m"]), _ptr(st["coef"]),
                                                        self.nnz, _stream(device))
            _lib.check(rc, "cbm_expand_coef_f32")
        return st["coef"]

    def to(self, device):
        """Upload the format to ``device`` now (it is otherwise uploaded at the first multiply)."""
        _require_gpu()
        self._device_arrays(device)
        return self

    def _stage(self, t):
        """(device tensor, needs_copy_back).  CPU tensors are staged through the current GPU."""
        if t.is_cuda:
            return t, False
        _require_gpu()
        return t.to("cuda"), True

    def summation_groups(self, x, y=None):
        """Interleaved partial sums per output element that the next multiply of ``x`` into ``y``
        keeps (1 = entries accumulate strictly in order); lets a checker reproduce the fp32 order."""
        y = x if y is None else y
        use_ws = self.relayout and _wants_workspace(x, y, self.nnz)
        return int(_lib.hip_lib().cbm_spmm_summation_groups(x.size(1), _ld(x), _ld(y), _ptr(x), _ptr(y), int(use_ws)))

    # ------------------------------------------------------------------ kernels -------------
    def _run_spmm(self, x, y, use_m, scale_roots, workspace=None, workspace_ready=False, workspace_prescaled=False):
        n = self.num_rows
        _check_f32_matrix(x, "rhs", n)
        _check_f32_matrix(y, "dst", n)
        if x.size(1) != y.size(1):
            raise ValueError(f"rhs has {x.size(1)} columns, dst has {y.size(1)}")
        if use_m and self.col_multiplier is None:
            raise RuntimeError("this cbm_matrix was built with normalized=False")
        _require_gpu()
        xd, _ = self._stage(x)
        yd = y if y.is_cuda else torch.empty(y.shape, dtype=y.dtype, device=xd.device)
        if yd.device != xd.device:
            raise ValueError("rhs and dst are on different devices")
        st = self._device_arrays(xd.device)
        if st["tiled"] is not None and self.relayout and not (workspace_ready and use_m and not workspace_prescaled):
            ws = self._tiled_workspace(xd, workspace)
            flags = (_lib.CBM_SPMM_WORKSPACE_READY if workspace_ready else 0) | \
                    (_lib.CBM_SPMM_WORKSPACE_PRESCALED if (workspace_prescaled and use_m) else 0)
            ts = self._tiled_struct(st, with_scale=use_m and scale_roots)
            with torch.cuda.device(xd.device):
                rc = _lib.hip_lib().cbm_spmm_tiled_f32(C.byref(ts), _ptr(st["m"]) if use_m else None, _ptr(xd), _ptr(yd),
                                                       _ptr(ws), flags, n, x.size(1), _ld(xd), _ld(yd), _stream(xd.device))
            _lib.check(rc, "cbm_spmm_tiled_f32")
            if yd is not y:
                y.copy_(yd)
            return
        ws = workspace if workspace is not None else (_workspace(xd, yd, self.nnz) if self.relayout else None)
        # per-entry coefficients are only read when the multiply does not scale its own copy of X
        coef = self._coef(st, xd.device) if (use_m and (ws is None or (workspace_ready and not workspace_prescaled))) else None
        flags = (_lib.CBM_SPMM_WORKSPACE_READY if workspace_ready else 0) | \
                (_lib.CBM_SPMM_WORKSPACE_PRESCALED if workspace_prescaled else 0) | \
                (_lib.CBM_SPMM_SCHED_BATCHED if self.batch_rows else 0)
        with torch.cuda.device(xd.device):
            rc = _lib.hip_lib().cbm_spmm_f32(
                _ptr(st["rowptr"]), _ptr(st["idx"]), self.nnz, _ptr(st["m"]) if use_m else None,
                _ptr(coef),
                _ptr(st["parent"]) if scale_roots else None,
                _ptr(st["sched_scaled"] if (scale_roots and use_m) else st["sched"]), _ptr(xd), _ptr(yd),
                _ptr(ws), flags, n, x.size(1), _ld(xd), _ld(yd),
                _stream(xd.device))
        _lib.check(rc, "cbm_spmm_f32")
        if yd is not y:
            y.copy_(yd)

    def _run_propagate(self, y, use_m, flags=0, scale_roots=True):
        n = self.num_rows
        _check_f32_matrix(y, "dst", n)
        if use_m and self.col_multiplier is None:
            raise RuntimeError("this cbm_matrix was built with normalized=False")
        _require_gpu()
        yd, back = self._stage(y)
        st = self._device_arrays(yd.device)
        if use_m and scale_roots:
            flags |= _lib.CBM_PROP_SCALE_ROOTS
        plan = self.walk_plan(y.size(1)) if n and y.size(1) else None
        with torch.cuda.device(yd.device):
            if plan is not None:
                rc = _lib.hip_lib().cbm_propagate_subtrees_f32(
                    C.byref(self._walk_struct(st, plan)), _ptr(st["parent"]), _ptr(st["order"]), _ptr(st["level_off"]),
                    _ptr(self.level_off), self.n_levels, _ptr(st["m"]) if use_m else None, _ptr(yd), n, y.size(1), _ld(yd),
                    flags, _stream(yd.device))
            else:
                rc = _lib.hip_lib().cbm_propagate_f32(
                    _ptr(st["parent"]), _ptr(st["order"]), _ptr(st["level_off"]), _ptr(self.level_off),
                    self.n_levels, _ptr(st["m"]) if use_m else None, _ptr(yd), n, y.size(1), _ld(yd),
                    flags & _lib.CBM_PROP_SCALE_ROOTS, _stream(yd.device))
        _lib.check(rc, "cbm_propagate_subtrees_f32" if plan is not None else "cbm_propagate_f32")
        if back:
            y.copy_(yd)

    def _run_spmm_update(self, x, y, use_m, flags=0, workspace=None, workspace_ready=False, relu=False,
                         workspace_prescaled=False):
        """``y = A_hat x`` (``cbm_spmm_update_f32``).  ``workspace``: device scratch for the slab-major
        copy of ``x`` (default: one from torch's caching allocator when the shape repays the copy);
        ``workspace_ready``: it already holds that copy (``relayout_slabs``), ``x`` is not read;
        ``workspace_prescaled``: that copy was made with ``scale=m``; ``relu``: ``y = max(A_hat x, 0)``."""
        n = self.num_rows
        _check_f32_matrix(x, "rhs", n)
        _check_f32_matrix(y, "dst", n)
        if x.size(1) != y.size(1):
            raise ValueError(f"rhs has {x.size(1)} columns, dst has {y.size(1)}")
        if use_m and self.col_multiplier is None:
            raise RuntimeError("this cbm_matrix was built with normalized=False")
        _require_gpu()
        xd, _ = self._stage(x)
        yd = y if y.is_cuda else torch.empty(y.shape, dtype=y.dtype, device=xd.device)
        if yd.device != xd.device:
            raise ValueError("rhs and dst are on different devices")
        if yd.data_ptr() == xd.data_ptr():
            raise ValueError("dst must not alias rhs")
        st = self._device_arrays(xd.device)
        tiled = st["tiled"] is not None and self.relayout and not (workspace_ready and use_m and not workspace_prescaled)
        if not tiled and workspace is None and not workspace_ready and self._single_launch(n, x.size(1)):
            with torch.cuda.device(xd.device):
                rc = _lib.hip_lib().cbm_spmm_update_single_f32(
                    _ptr(st["rowptr"]), _ptr(st["idx"]), _ptr(st["m"]) if use_m else None, None, _ptr(st["parent"]),
                    self.n_levels, _ptr(xd), _ptr(yd), n, x.size(1), _ld(xd), _ld(yd),
                    _lib.CBM_UPDATE_RELU if relu else 0, _stream(xd.device))
            _lib.check(rc, "cbm_spmm_update_single_f32")
            if yd is not y:
                y.copy_(yd)
            return
        if st["tiled"] is None and workspace is None and not workspace_ready:
            sp = self.stream_plan(x.size(1))
            if sp is not None:                                  # a deep tree, short delta rows: one launch does it all
                with torch.cuda.device(xd.device):
                    rc = _lib.hip_lib().cbm_spmm_update_subtrees_f32(
                        C.byref(self._stream_struct(st, sp)), _ptr(st["m"]) if use_m else None, _ptr(xd), _ptr(yd), n,
                        x.size(1), _ld(xd), _ld(yd), _lib.CBM_UPDATE_RELU if relu else 0, _stream(xd.device))
                _lib.check(rc, "cbm_spmm_update_subtrees_f32")
                if yd is not y:
                    y.copy_(yd)
                return
        if (tiled or not self._walks_paths(n, x.size(1))) and self.walk_plan(x.size(1)) is not None:
            # a deep tree: the SpMM (root children scaled in its epilogue), then the walk by subtrees
            self._run_spmm(xd, yd, use_m, scale_roots=use_m, workspace=workspace, workspace_ready=workspace_ready,
                           workspace_prescaled=workspace_prescaled)
            self._run_propagate(yd, use_m, flags=_lib.CBM_UPDATE_RELU if relu else 0, scale_roots=False)
            if yd is not y:
                y.copy_(yd)
            return
        if tiled:
            ws = self._tiled_workspace(xd, workspace)
        else:
            ws = workspace if workspace is not None else (_workspace(xd, yd, self.nnz) if self.relayout else None)
        if workspace_ready:
            flags |= _lib.CBM_UPDATE_WORKSPACE_READY
        if workspace_prescaled:
            flags |= _lib.CBM_UPDATE_WORKSPACE_PRESCALED
        if relu:
            flags |= _lib.CBM_UPDATE_RELU
        if tiled:
            if not use_m:
                flags &= ~_lib.CBM_UPDATE_WORKSPACE_PRESCALED
            ts = self._tiled_struct(st, with_scale=use_m)
            with torch.cuda.device(xd.device):
                rc = _lib.hip_lib().cbm_spmm_update_tiled_f32(
                    C.byref(ts), _ptr(st["m"]) if use_m else None, _ptr(st["parent"]), _ptr(st["order"]),
                    _ptr(st["level_off"]), _ptr(self.level_off), self.n_levels, _ptr(xd), _ptr(yd), _ptr(ws), n, x.size(1),
                    _ld(xd), _ld(yd), flags, _stream(xd.device))
            _lib.check(rc, "cbm_spmm_update_tiled_f32")
            if yd is not y:
                y.copy_(yd)
            return
        coef = self._coef(st, xd.device) if (use_m and (ws is None or (workspace_ready and not workspace_prescaled))) else None
        if self.batch_rows:
            flags |= _lib.CBM_UPDATE_SCHED_BATCHED
        if self._walks_paths(n, x.size(1)):
            zs = torch.empty(_lib.hip_lib().cbm_spmm_update_paths_scratch_floats(n, x.size(1), self.n_levels),
                             dtype=torch.float32, device=xd.device)
            with torch.cuda.device(xd.device):
                rc = _lib.hip_lib().cbm_spmm_update_paths_f32(
                    _ptr(st["rowptr"]), _ptr(st["idx"]), self.nnz, _ptr(st["m"]) if use_m else None,
                    _ptr(coef), _ptr(st["parent"]),
                    _ptr(st["sched_scaled"] if use_m else st["sched"]), _ptr(st["order"]), _ptr(st["level_off"]),
                    _ptr(self.level_off), self.n_levels, _ptr(xd), _ptr(yd), _ptr(ws), _ptr(zs), n, x.size(1), _ld(xd),
                    _ld(yd), flags, _stream(xd.device))
            _lib.check(rc, "cbm_spmm_update_paths_f32")
            if yd is not y:
                y.copy_(yd)
            return
        with torch.cuda.device(xd.device):
            rc = _lib.hip_lib().cbm_spmm_update_f32(
                _ptr(st["rowptr"]), _ptr(st["idx"]), self.nnz, _ptr(st["m"]) if use_m else None,
                _ptr(coef), _ptr(st["parent"]),
                _ptr(st["sched_scaled"] if use_m else st["sched"]), _ptr(st["order"]), _ptr(st["level_off"]), _ptr(self.level_off), self.n_levels,
                _ptr(xd), _ptr(yd), _ptr(ws), n, x.size(1), _ld(xd), _ld(yd), flags, _stream(xd.device))
        _lib.check(rc, "cbm_spmm_update_f32")
        if yd is not y:
            y.copy_(yd)

    def _plain_spmm_update(self, x, y):
        """The reference's un-fused ``*_spmm_update``: delta SpMM, then the plain walk.  On a
        matrix built with ``normalized=True`` the reference's delta values are ``+-m[col]``
        (``cbm.py:56-66`` with the v2 builder, ``cbm_extensions.cpp:504-585``), so that call
        returns ``A diag(m) X`` -- the right scaling only; the same here."""
        if self.col_multiplier is None:
            self._run_spmm_update(x, y, use_m=False)
            return
        self._run_spmm(x, y, use_m=True, scale_roots=False)
        self._run_propagate(y, use_m=False)

    # ------------------------------------------------------------------ reference methods ---
    # "Sequential" methods (cbm.py:144-188)
    def seq_mkl_csr_spmm_update(self, x, y):
        self._plain_spmm_update(x, y)

    def seq_mkl_csr_spmm(self, x, y):
        self._run_spmm(x, y, use_m=self.col_multiplier is not None, scale_roots=False)

    def seq_mkl_csr_update(self, y):
        self._run_propagate(y, use_m=False)

    def seq_mkl_csr_fused_spmm_update(self, x, y):
        self._run_spmm_update(x, y, use_m=True)

    def seq_mkl_csr_fused_update(self, y):
        self._run_propagate(y, use_m=True)

    # "Parallel" methods (cbm.py:191-249)
    def omp_mkl_csr_spmm_update(self, x, y):
        self._plain_spmm_update(x, y)

    def omp_mkl_csr_spmm(self, x, y):
        self._run_spmm(x, y, use_m=self.col_multiplier is not None, scale_roots=False)

    def omp_mkl_csr_update(self, y):
        self._run_propagate(y, use_m=False)

    def omp_avx_csr_update(self, y):
        self._run_propagate(y, use_m=False)

    def omp_mkl_csr_spmm_update_v2(self, x, y):
        # the reference wrapper (cbm.py:219-228) names a native function that its extension
        # never exports; here it is the plain spmm + update
        self._plain_spmm_update(x, y)

    def omp_mkl_csr_fused_spmm_update(self, x, y):
        self._run_spmm_update(x, y, use_m=True)

    def omp_mkl_csr_fused_update(self, y):
        self._run_propagate(y, use_m=True)

    # "mixed" methods (cbm.py:255-275): deltas @ x, then the update; here both on the GPU and
    # differentiable with the full operator (not only the delta part)
    def seq_torch_csr_matmul(self, x):
        return CBMMatmul.apply(x, self, False)

    def omp_torch_csr_matmul(self, x):
        return CBMMatmul.apply(x, self, False)

    def seq_torch_csr_fused_matmul(self, x):
        return CBMMatmul.apply(x, self, True)

    def omp_torch_csr_fused_matmul(self, x):
        return CBMMatmul.apply(x, self, True)

    # ------------------------------------------------------------------ additions -----------
    def matmul(self, x):
        """``A_hat @ x`` (normalised if the matrix was built so), differentiable in ``x``."""
        return CBMMatmul.apply(x, self, self.col_multiplier is not None)

    def transposed(self):
        """CBM of the transposed matrix (the operator of the backward pass).  For a symmetric
        edge list -- every undirected graph -- this is the object itself."""
        if self.is_symmetric:
            return self
        if self._transposed is None:
            ei = self._edge_index_cpu
            t = cbm_matrix(torch.stack([ei[1], ei[0]]), None, alpha=self.alpha, normalized=False, max_levels=self.max_levels,
                           tiling=self.tiling)
            t.col_multiplier = self.col_multiplier      # diag(m) A^T diag(m): same vector both sides
            t.normalized = self.normalized
            t._transposed = self
            self._transposed = t
        return self._transposed


class CBMMatmul(torch.autograd.Function):
    """y = A_hat x with backward g -> A_hat^T g, both through the HIP kernels.

    ``fused=True``: ``diag(m) A diag(m) x`` (the fused normalised path).  ``fused=False``: the
    reference's un-fused path, ``A x`` on a plain matrix and ``A diag(m) x`` on a normalised one
    (its delta values carry the right scaling, ``cbm.py:255-265``); backward is then
    ``diag(m) A^T g``."""

    @staticmethod
    def forward(ctx, x, mat, fused):
        ctx.mat = mat
        ctx.fused = fused
        xd = x.detach()
        if xd.dtype != torch.float32:
            raise RuntimeError("rhs tensor (NOT torch::kFloat32)")
        xd = xd.contiguous()
        y = torch.empty_like(xd)
        if fused:
            mat._run_spmm_update(xd, y, use_m=True)
        else:
            mat._plain_spmm_update(xd, y)
        return y

    @staticmethod
    def backward(ctx, g):
        g = g.contiguous()
        gx = torch.empty_like(g)
        mat = ctx.mat
        mat.transposed()._run_spmm_update(g, gx, use_m=ctx.fused)
        if not ctx.fused and mat.col_multiplier is not None:
            gx.mul_(mat.col_multiplier.to(gx.device).unsqueeze(1))
        return gx, None, None


def relayout_slabs(x, mask=None, out=None, scale=None):
    """Slab-major copy of ``x`` for ``cbm_spmm_f32(..., CBM_SPMM_WORKSPACE_READY)`` (None for an
    empty matrix).  With ``mask`` (same shape) the copy holds ``x`` where ``mask > 0`` and zero
    elsewhere (``cbm_relayout_slabs_masked_f32``: a ReLU gradient folded into the copy).  With
    ``scale`` (fp32 [n], e.g. the matrix's ``col_multiplier`` on the device) row r of the copy is
    multiplied by ``scale[r]``: announce such a copy with ``workspace_prescaled=True``.  ``out``: a
    float32 device tensor of at least ``cbm_relayout_floats(n, d)`` elements to reuse."""
    n, d = x.shape
    floats = _lib.hip_lib().cbm_relayout_floats(n, d)
    if floats <= 0:
        return None
    if out is not None and (out.numel() < floats or out.device != x.device or out.dtype != torch.float32):
        raise ValueError("out is too small, on another device or not float32")
    ws = out if out is not None else torch.empty(floats, dtype=torch.float32, device=x.device)
    if scale is not None and (scale.dtype != torch.float32 or scale.numel() != n or scale.device != x.device
                              or not scale.is_contiguous()):
        raise ValueError("scale must be a contiguous float32 vector of n elements on x's device")
    with torch.cuda.device(x.device):
        if mask is None and scale is None:
            rc = _lib.hip_lib().cbm_relayout_slabs_f32(_ptr(x), _ptr(ws), n, d, _ld(x), _stream(x.device))
        elif mask is None:
            rc = _lib.hip_lib().cbm_relayout_slabs_scaled_f32(_ptr(x), _ptr(scale), _ptr(ws), n, d, _ld(x), _stream(x.device))
        else:
            _check_f32_matrix(mask, "mask", n)
            if mask.size(1) != d or mask.device != x.device:
                raise ValueError("mask must have the shape and device of x")
            rc = _lib.hip_lib().cbm_relayout_slabs_masked_f32(_ptr(x), _ptr(mask), _ptr(scale), _ptr(ws), n, d, _ld(x),
                                                              _ld(mask), _stream(x.device))
    _lib.check(rc, "cbm_relayout_slabs_f32")
    return ws


def csr_spmm(rowptr, col, val, x, y, sched=None):
    """Plain CSR SpMM ``y = A @ x`` on the GPU: the hand-written baseline the CBM multiply is
    measured against (role of ``omp_s_spmm_csr_int32``, ``cbm_extensions.cpp:1707-1755``).
    ``rowptr`` [N+1] / ``col`` int32 device tensors, ``val`` fp32 or None (all ones); ``sched``:
    optional device copy of ``schedule_rows(rowptr)`` or ``schedule_rows(rowptr, batch=...)`` (same
    scheduling as the CBM kernels, short rows in batches included)."""
    n = rowptr.numel() - 1
    _check_f32_matrix(x, "rhs")
    _check_f32_matrix(y, "dst", n)
    if rowptr.dtype != torch.int32 or col.dtype != torch.int32:
        raise RuntimeError("lhs_col (NOT torch::kInt32)")
    if val is not None and val.dtype != torch.float32:
        raise RuntimeError("lhs_val (NOT torch::kFloat32)")
    if not (x.is_cuda and y.is_cuda and rowptr.is_cuda and col.is_cuda):
        raise ValueError("csr_spmm expects device tensors")
    ws = _workspace(x, y, col.numel())
    flags = 0
    if sched is not None:
        if tuple(sched.shape) == (n + 1, 4):
            flags = _lib.CBM_SPMM_SCHED_BATCHED
        elif tuple(sched.shape) != (n, 4):
            raise ValueError("sched must be schedule_rows(rowptr) ([n, 4]) or its batched form ([n + 1, 4])")
    with torch.cuda.device(x.device):
        rc = _lib.hip_lib().csr_spmm_f32(_ptr(rowptr), _ptr(col), col.numel(), _ptr(val), _ptr(sched), _ptr(x), _ptr(y), _ptr(ws),
                                         flags, n, x.size(1), _ld(x), _ld(y), _stream(x.device))
    _lib.check(rc, "csr_spmm_f32")
