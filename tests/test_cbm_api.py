"""Host-side surface of cbm_matrix (no GPU): constructor, attributes, the reference's method
names, error behaviour, and the loud failure when no HIP device exists."""
import os

import numpy as np
import pytest
import torch

from cbm4gnn_amd import graphs
from cbm.cbm import cbm_matrix                    # the reference's import path

REFERENCE_METHODS = [                             # cbm/cbm.py:144-275
    "seq_mkl_csr_spmm_update", "seq_mkl_csr_spmm", "seq_mkl_csr_update", "seq_mkl_csr_fused_spmm_update",
    "seq_mkl_csr_fused_update", "omp_mkl_csr_spmm_update", "omp_mkl_csr_spmm", "omp_mkl_csr_update",
    "omp_avx_csr_update", "omp_mkl_csr_spmm_update_v2", "omp_mkl_csr_fused_spmm_update", "omp_mkl_csr_fused_update",
    "seq_torch_csr_matmul", "omp_torch_csr_matmul", "seq_torch_csr_fused_matmul", "omp_torch_csr_fused_matmul",
    "check_format", "to_sparse_coo_tensor", "to_sparse_csr_tensor",
]


@pytest.fixture(scope="module")
def er25():
    ei = graphs.erdos_renyi(25, 0.5, 0)
    return torch.from_numpy(ei), torch.ones(ei.shape[1], dtype=torch.float32)


@pytest.mark.parametrize("alpha", [1, 2, 3, 4])
def test_creation_like_the_reference_test(er25, alpha):
    # tests/test_cbm_creation.py:33-48: construction succeeds for alpha in 1..4
    ei, vals = er25
    assert cbm_matrix(ei, vals, alpha=alpha) is not None
    assert cbm_matrix(ei, vals, alpha=alpha, normalized=True) is not None


def test_attributes_and_methods(er25):
    ei, vals = er25
    c = cbm_matrix(ei, vals, alpha=3)
    for name in REFERENCE_METHODS:
        assert callable(getattr(c, name)), name
    assert c.mst_row.dtype == torch.int32 and c.mst_row.numel() == 25 + 2
    assert c.mst_col.dtype == torch.int32 and c.mst_col.numel() == 25
    assert c.col_multiplier is None
    assert c.deltas.layout == torch.sparse_csr and tuple(c.deltas.shape) == (25, 25)
    assert cbm_matrix(ei, vals, alpha=3, deltas_format="coo").deltas.layout == torch.sparse_coo
    cn = cbm_matrix(ei, vals, alpha=3, normalized=True)
    deg = torch.bincount(ei[0].long(), minlength=25).float()
    assert torch.equal(cn.col_multiplier, deg.pow(-0.5))
    # the reference's compression-ratio helper reads exactly these attributes (benchmark/utility.py:54-60)
    total = (c.deltas.col_indices().numel() + c.deltas.crow_indices().numel() + c.deltas.values().numel()
             + c.mst_row.numel() + c.mst_col.numel())
    assert c.compression_ratio() == pytest.approx((26 + 2 * ei.size(1)) / total)


def test_check_format_detects_corruption(er25):
    ei, vals = er25
    c = cbm_matrix(ei, vals, alpha=0)
    assert c.check_format(ei)
    bad = c.idx.clone()
    k = int(torch.nonzero(bad >= 0)[0])
    c.idx = bad
    c.idx[k] = (int(bad[k]) + 1) % 25
    with pytest.raises((ValueError, KeyError)):
        c.check_format(ei)


def test_deltas_times_x_plus_walk_equals_product_on_cpu_tensors_math(er25):
    # pure host arithmetic on the format (dense fp64): Delta @ X, then the top-down walk, is A @ X
    ei, vals = er25
    c = cbm_matrix(ei, vals, alpha=2)
    x = np.random.default_rng(0).integers(0, 10, (25, 10)).astype(np.float64)
    y = c.deltas.to_dense().double().numpy() @ x
    parent = c.parent.numpy()
    for v in c.order.numpy():
        if parent[v] >= 0:
            y[v] += y[parent[v]]
    a = np.zeros((25, 25)); a[ei[0].numpy(), ei[1].numpy()] = 1
    assert np.array_equal(y, a @ x)


@pytest.mark.skipif(torch.cuda.is_available(), reason="checks the no-GPU failure mode")
def test_multiply_without_gpu_raises_instead_of_falling_back(er25):
    ei, vals = er25
    c = cbm_matrix(ei, vals, alpha=3)
    x = torch.ones(25, 10)
    y = torch.empty(25, 10)
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        c.omp_mkl_csr_spmm_update(x, y)
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        c.seq_torch_csr_matmul(x)
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        c.omp_mkl_csr_update(y)


def test_argument_checks_come_before_any_device_work(er25):
    ei, vals = er25
    c = cbm_matrix(ei, vals, alpha=3)
    y = torch.empty(25, 10)
    with pytest.raises(RuntimeError, match="kFloat32"):             # the reference's TORCH_CHECK text
        c.omp_mkl_csr_spmm_update(torch.ones(25, 10, dtype=torch.float64), y)
    with pytest.raises(ValueError):
        c.omp_mkl_csr_spmm_update(torch.ones(24, 10), y)
    with pytest.raises(ValueError):
        c.omp_mkl_csr_spmm_update(torch.ones(25, 9), y)
    with pytest.raises(ValueError):
        c.omp_mkl_csr_spmm_update(torch.ones(10, 25).t(), y)        # column-major view
    with pytest.raises(RuntimeError, match="normalized=False"):
        c.omp_mkl_csr_fused_spmm_update(torch.ones(25, 10), y)


def test_symmetry_flag_and_transpose():
    ei = torch.tensor([[0, 1, 2, 2], [1, 2, 0, 1]], dtype=torch.int32)
    c = cbm_matrix(ei, None)
    assert not c.is_symmetric
    t = c.transposed()
    assert t is not c and t.transposed() is c
    # the transposed object is the CBM of A^T: its rows rebuild to the transposed adjacency
    assert t.check_format(torch.stack([ei[1], ei[0]]))
    with pytest.raises(ValueError):
        t.check_format(ei)                                  # and not to A itself (A is not symmetric)
    assert t.nnz_a == c.nnz_a == 4 and t.num_rows == c.num_rows
    # a larger directed graph, where the deltas really compress: same checks
    rng = np.random.default_rng(4)
    base = rng.integers(0, 40, (2, 300)).astype(np.int32)
    big = torch.from_numpy(np.unique(np.concatenate([base, np.stack([np.arange(40), np.arange(40)]).astype(np.int32)], 1), axis=1))
    cb = cbm_matrix(big, None, alpha=0)
    tb = cb.transposed()
    assert not cb.is_symmetric and tb.check_format(torch.stack([big[1], big[0]]))
    und = cbm_matrix(torch.from_numpy(graphs.erdos_renyi(10, 0.5, 1)), None)
    assert und.is_symmetric and und.transposed() is und


def test_save_and_load_round_trip(tmp_path):
    ei = torch.from_numpy(graphs.add_self_loops(graphs.erdos_renyi(60, 0.2, 5), 60))
    directed = torch.tensor([[0, 1, 2, 2], [1, 2, 0, 1]], dtype=torch.int32)
    for edge_index, normalized in ((ei, True), (ei, False), (directed, True)):
        a = cbm_matrix(edge_index, None, alpha=2, normalized=normalized)
        path = str(tmp_path / "m.npz")
        a.save(path)
        b = cbm_matrix.load(path)
        for name in ("rowptr", "idx", "parent", "order", "level_off", "mst_row", "mst_col"):
            assert torch.equal(getattr(a, name), getattr(b, name)), name
        assert (a.col_multiplier is None) == (b.col_multiplier is None)
        if normalized:
            assert torch.equal(a.col_multiplier, b.col_multiplier)
        for name in ("num_rows", "alpha", "normalized", "nnz", "nnz_a", "n_candidates", "n_levels", "is_symmetric"):
            assert getattr(a, name) == getattr(b, name), name
        assert torch.equal(a.deltas.to_dense(), b.deltas.to_dense())
        assert b.check_format(edge_index)
        if not b.is_symmetric:
            assert torch.equal(b.transposed().rowptr, a.transposed().rowptr)
    # a path without the extension names the same file in save and load; the depth limit survives
    deep = cbm_matrix(ei, None, alpha=0, max_levels=2)
    bare = str(tmp_path / "no_extension")
    deep.save(bare)
    again = cbm_matrix.load(bare)
    assert again.max_levels == 2 and again.n_levels <= 2 and torch.equal(again.idx, deep.idx)
    assert cbm_matrix.load(bare + ".npz").max_levels == 2
    assert cbm_matrix.load(path).max_levels is None
    bad = dict(np.load(path))
    bad["order"] = bad["order"][:-1]
    np.savez(str(tmp_path / "bad.npz"), **bad)
    with pytest.raises(ValueError):
        cbm_matrix.load(str(tmp_path / "bad.npz"))


def test_edge_fingerprint_and_cache_file(tmp_path):
    """The cache file is keyed by an order-independent fingerprint of the edge list plus alpha, the
    normalisation and the depth limit: same graph in another edge order -> loaded, anything else -> rebuilt."""
    from cbm4gnn_amd.cbm import edge_fingerprint
    ei = graphs.add_self_loops(graphs.sbm(300, 6, 0.5, 0.01, seed=2), 300)
    perm = np.random.default_rng(0).permutation(ei.shape[1])
    shuffled = np.ascontiguousarray(ei[:, perm])
    assert np.array_equal(edge_fingerprint(ei), edge_fingerprint(shuffled))
    assert edge_fingerprint(ei).dtype == np.uint64 and int(edge_fingerprint(ei)[0]) == ei.shape[1]
    moved = ei.copy(); moved[1, 7] = (moved[1, 7] + 1) % 300               # one edge points elsewhere
    assert not np.array_equal(edge_fingerprint(ei), edge_fingerprint(moved))
    assert not np.array_equal(edge_fingerprint(ei), edge_fingerprint(ei[:, :-1]))
    assert not np.array_equal(edge_fingerprint(ei, 300), edge_fingerprint(ei, 301))     # the key depends on N
    swapped = np.ascontiguousarray(ei[::-1])                                # symmetric graph: the transpose is the same edge set
    assert np.array_equal(edge_fingerprint(ei), edge_fingerprint(swapped))
    directed = np.array([[0, 1, 2, 2], [1, 2, 0, 1]], np.int32)
    assert not np.array_equal(edge_fingerprint(directed), edge_fingerprint(directed[::-1].copy()))

    path = str(tmp_path / "cache")
    first = cbm_matrix.from_cache(path, torch.from_numpy(ei), alpha=1, normalized=True)
    assert first.builder is not None and first.build_seconds is not None           # built, file written
    assert (tmp_path / "cache.npz").exists()
    second = cbm_matrix.from_cache(path, torch.from_numpy(shuffled), alpha=1, normalized=True)
    assert second.builder is None and second.build_seconds is None                  # loaded
    for name in ("rowptr", "idx", "parent", "order", "level_off", "mst_row", "mst_col", "col_multiplier"):
        assert torch.equal(getattr(first, name), getattr(second, name)), name
    assert np.array_equal(second.edge_fingerprint, first.edge_fingerprint)
    assert second.check_format(torch.from_numpy(ei))
    # anything that changes the format rebuilds and overwrites the file
    for kw in (dict(alpha=2, normalized=True), dict(alpha=1, normalized=False), dict(alpha=1, normalized=True, max_levels=2)):
        again = cbm_matrix.from_cache(path, torch.from_numpy(ei), **kw)
        assert again.builder is not None, kw
        assert cbm_matrix.from_cache(path, torch.from_numpy(ei), **kw).builder is None, kw
    other = cbm_matrix.from_cache(path, torch.from_numpy(moved), alpha=1, normalized=True, max_levels=2)
    assert other.builder is not None and other.check_format(torch.from_numpy(moved))
    # a file of an older version (no fingerprint) still loads, but never satisfies the cache
    old = dict(np.load(str(tmp_path / "cache.npz")))
    old.pop("edge_fingerprint"); old["meta"] = old["meta"].copy(); old["meta"][0] = 2
    np.savez(str(tmp_path / "old.npz"), **old)
    assert cbm_matrix.load(str(tmp_path / "old.npz")).edge_fingerprint is None
    assert cbm_matrix.from_cache(str(tmp_path / "old"), torch.from_numpy(moved), alpha=1, normalized=True, max_levels=2).builder is not None
    # a damaged file is rebuilt, not trusted
    (tmp_path / "junk.npz").write_bytes(b"not a zip file")
    assert cbm_matrix.from_cache(str(tmp_path / "junk"), torch.from_numpy(ei), alpha=0).builder is not None
    assert cbm_matrix.from_cache(str(tmp_path / "junk"), torch.from_numpy(ei), alpha=0).builder is None


def _corruptions(z, n):
    """(name, changed arrays) pairs: one damaged copy of a saved file per array a kernel indexes with."""
    def with_(**kw):
        out = {k: v.copy() for k, v in z.items()}
        out.update(kw)
        return out

    idx, rowptr, parent, order = z["idx"], z["rowptr"], z["parent"], z["order"]
    level_off, mst_row, mst_col = z["level_off"], z["mst_row"], z["mst_col"]
    k = int(np.argmax(np.diff(rowptr) >= 2))                 # a row with at least two entries
    lo = int(rowptr[k])
    swapped = idx.copy(); swapped[[lo, lo + 1]] = swapped[[lo + 1, lo]]
    big = idx.copy(); big[3] = 10 ** 6
    neg_big = idx.copy(); neg_big[3] = np.int32(-(2 ** 31) + n)          # sign bit set, column N
    far = parent.copy(); far[5] = 4000
    root = int(np.argmax(parent >= 0))                       # a row that has a parent: claim it hangs off the root
    orphan = parent.copy(); orphan[root] = -1
    other = parent.copy(); other[root] = (other[root] + 1) % n
    dup = order.copy(); dup[1] = dup[0]
    rev = order.copy(); rev[:2] = rev[:2][::-1]
    hump = rowptr.copy(); hump[k + 1] = hump[k] - 1 if hump[k] > 0 else hump[k + 2] + 1
    short_end = rowptr.copy(); short_end[-1] -= 1
    lv = level_off.copy(); lv[1] = lv[1] - 1 if lv.shape[0] > 2 else lv[1]
    mr = mst_row.copy(); mr[1:-1] = mr[1:-1][::-1] if not np.array_equal(mr[1:-1], mr[1:-1][::-1]) else mr[1:-1] + 1
    mc = mst_col.copy(); mc[0] = mc[1]
    mc_swap = mst_col.copy(); mc_swap[[0, n - 1]] = mc_swap[[n - 1, 0]]
    meta = z["meta"].copy(); meta[1] += 1
    meta_nnz = z["meta"].copy(); meta_nnz[4] += 1
    cases = [("idx out of range", with_(idx=big)), ("idx out of range under the sign bit", with_(idx=neg_big)),
             ("idx unsorted", with_(idx=swapped)), ("idx truncated", with_(idx=idx[:-1])),
             ("idx dtype", with_(idx=idx.astype(np.int64))),
             ("parent out of range", with_(parent=far)), ("parent says root", with_(parent=orphan)),
             ("parent names another row", with_(parent=other)),
             ("order not a permutation", with_(order=dup)), ("order not sorted", with_(order=rev)),
             ("rowptr not monotone", with_(rowptr=hump)), ("rowptr end", with_(rowptr=short_end)),
             ("level_off", with_(level_off=lv)), ("level_off truncated", with_(level_off=level_off[:-1])),
             ("mst_row", with_(mst_row=mr)), ("mst_col not a permutation", with_(mst_col=mc)),
             ("mst_col another tree", with_(mst_col=mc_swap)),
             ("N in the header", with_(meta=meta)), ("nnz in the header", with_(meta=meta_nnz))]
    if "col_multiplier" in z:
        nan = z["col_multiplier"].copy(); nan[2] = np.nan
        cases += [("m not finite", with_(col_multiplier=nan)), ("m truncated", with_(col_multiplier=z["col_multiplier"][:-1])),
                  ("m missing", {k_: v for k_, v in z.items() if k_ != "col_multiplier"})]
    if "edge_index" in z:
        e = z["edge_index"].copy(); e[0, 0] = n + 7
        cases += [("edge_index out of range", with_(edge_index=e)),
                  ("edge_index missing", {k_: v for k_, v in z.items() if k_ != "edge_index"})]
    return cases


@pytest.mark.parametrize("kind", ["undirected", "directed"])
def test_load_rejects_every_damaged_array(tmp_path, kind):
    """A file whose arrays would send a kernel out of bounds (or to a wrong product) never loads: every
    check of ``load`` is exercised on the host with one damaged copy of a good file per array.  None of
    these files goes anywhere near a GPU."""
    n = 50
    if kind == "undirected":
        ei = torch.from_numpy(graphs.add_self_loops(graphs.sbm(n, 5, 0.7, 0.05, seed=4), n))
    else:
        rng = np.random.default_rng(3)
        dense = rng.random((n, n)) < 0.25
        dense[np.arange(n), (np.arange(n) + 1) % n] = True              # every row and column used
        dense[10:20] = dense[10]                                         # rows that share everything: a tree
        dense[10:20, 30:40] ^= np.eye(10, dtype=bool)
        ei = torch.from_numpy(np.stack(np.nonzero(dense)).astype(np.int32))
    a = cbm_matrix(ei, None, alpha=0, normalized=True)
    assert a.n_levels >= 2 and (kind == "undirected") == a.is_symmetric
    good = str(tmp_path / "good.npz")
    a.save(good)
    assert not [f for f in os.listdir(tmp_path) if ".tmp" in f]          # written under a temporary name, renamed
    z = dict(np.load(good))
    assert cbm_matrix.load(good).check_format(ei)
    seen = set()
    for name, arrays in _corruptions(z, n):
        path = str(tmp_path / "damaged.npz")
        np.savez(path, **arrays)
        with pytest.raises(ValueError) as err:
            cbm_matrix.load(path)
        seen.add(str(err.value).split(": ", 1)[-1])
        # ... and the cache rebuilds instead of trusting it
        rebuilt = cbm_matrix.from_cache(path, ei, alpha=0, normalized=True)
        assert rebuilt.builder is not None and torch.equal(rebuilt.idx, a.idx), name
        assert cbm_matrix.from_cache(path, ei, alpha=0, normalized=True).builder is None, name
    assert len(seen) >= 12                                               # the cases trip different checks
    # a file cut short (a writer that died, a partial copy)
    blob = open(good, "rb").read()
    for cut in (len(blob) // 2, len(blob) - 7, 10):
        (tmp_path / "cut.npz").write_bytes(blob[:cut])
        with pytest.raises(ValueError):
            cbm_matrix.load(str(tmp_path / "cut.npz"))
        assert cbm_matrix.from_cache(str(tmp_path / "cut"), ei, alpha=0, normalized=True).builder is not None
