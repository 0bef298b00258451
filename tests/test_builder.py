"""The product's host builder (libcbm_host.so) against the oracle and against invariants.
"Bit-exact format arrays": every integer array the builder emits equals the independent
derivation from its own parent[] (oracle.format_from_parent, set differences)."""
import ctypes as C

import numpy as np
import pytest
import torch

from cbm4gnn_amd import _lib, graphs
from cbm4gnn_amd.cbm import cbm_matrix, tree_levels


def _u32(t):
    return t.numpy().view(np.uint32)


def _assert_format_equals_derivation(orc, ei, n, mat):
    f = orc.format_from_parent(ei, n, mat.parent.numpy())
    assert np.array_equal(f["rowptr"], mat.rowptr.numpy())
    assert np.array_equal(f["idx"], _u32(mat.idx))
    assert np.array_equal(f["order"], mat.order.numpy())
    assert np.array_equal(f["level_off"], mat.level_off.numpy())
    assert np.array_equal(f["mst_row"], mat.mst_row.numpy())
    assert np.array_equal(f["mst_col"], mat.mst_col.numpy())


@pytest.mark.parametrize("seed", range(10))
@pytest.mark.parametrize("alpha", [0, 1, 3, 8])
def test_builder_matches_oracle_small(orc, seed, alpha):
    n = 25 + 6 * seed
    ei = graphs.erdos_renyi(n, [0.15, 0.5, 0.75][seed % 3], seed)
    if seed % 2:
        ei = graphs.add_self_loops(ei, n)
    mat = cbm_matrix(torch.from_numpy(ei), torch.ones(ei.shape[1]), alpha=alpha)
    o = orc.build_format(ei, n, alpha)
    assert mat.n_candidates == o["n_candidates"]
    assert mat.nnz == o["msa_weight"] == o["nnz"]          # two different MSA algorithms, same optimum
    assert mat.nnz_a == ei.shape[1]
    _assert_format_equals_derivation(orc, ei, n, mat)
    assert orc.check_format(ei, n, mat.rowptr.numpy(), _u32(mat.idx), mat.mst_row.numpy(), mat.mst_col.numpy())
    assert mat.check_format(torch.from_numpy(ei))


def _small_chain_workload():
    # the alpha-sweep workload's construction (clique blocks + staircase chain) at a size the
    # oracle's O(V E) arborescence finishes in seconds
    ei = graphs.sbm_with_chain(n=1500, blocks=24, p_in=1.0, mean_deg=80.0, chain=64, base=48, seed=0)
    return graphs.Workload("c5-small", ei, 1500, 32, False, (0, 4), "normal")


@pytest.mark.parametrize("name,scale", [("c1", 1.0), ("c2", 0.25), ("c3", 0.02), ("c5-small", 1.0)])
def test_builder_matches_oracle_workloads(orc, name, scale):
    w = _small_chain_workload() if name == "c5-small" else graphs.workload(name, scale=scale)
    for alpha in w.alphas[:2]:
        mat = cbm_matrix(torch.from_numpy(w.edge_index), None, alpha=alpha, normalized=w.normalized)
        o = orc.build_format(w.edge_index, w.n, alpha)
        assert mat.n_candidates == o["n_candidates"]
        assert mat.nnz == o["msa_weight"]
        assert orc.check_format(w.edge_index, w.n, mat.rowptr.numpy(), _u32(mat.idx), mat.mst_row.numpy(), mat.mst_col.numpy())
        assert mat.compression_ratio() == pytest.approx(orc.compression_ratio(w.n, w.edge_index.shape[1], o["nnz"]))


def test_level_ordering_invariants():
    w = graphs.workload("c2", scale=0.25)
    mat = cbm_matrix(torch.from_numpy(w.edge_index), None, alpha=0)
    n = w.n
    parent, order, lo = mat.parent.numpy(), mat.order.numpy(), mat.level_off.numpy()
    assert sorted(order.tolist()) == list(range(n))
    assert lo[0] == 0 and lo[-1] == n and (np.diff(lo) > 0).all()
    level = np.empty(n, np.int64)
    for l in range(len(lo) - 1):
        seg = order[lo[l]:lo[l + 1]]
        assert (np.diff(seg) > 0).all()                     # ids ascending inside a level
        level[seg] = l
    roots = parent < 0
    assert (level[roots] == 0).all()
    assert (level[~roots] == level[parent[~roots]] + 1).all()
    assert mat.n_levels > 3                                 # the workload really has a deep-ish tree
    # the tree CSR and the level arrays describe the same tree
    p2, o2, lo2 = tree_levels(mat.mst_row.numpy(), mat.mst_col.numpy())
    assert np.array_equal(p2, parent) and np.array_equal(o2, order) and np.array_equal(lo2, lo)


def test_packed_sign_round_trip_and_deltas_tensor(orc):
    n = 60
    ei = graphs.add_self_loops(graphs.erdos_renyi(n, 0.4, 4), n)
    for normalized in (False, True):
        mat = cbm_matrix(torch.from_numpy(ei), None, alpha=1, normalized=normalized)
        d = mat.deltas
        assert d.layout == torch.sparse_csr
        assert d.crow_indices().dtype == torch.int64 and d.values().dtype == torch.float32
        idx = _u32(mat.idx)
        assert np.array_equal(d.col_indices().numpy(), (idx & 0x7FFFFFFF).astype(np.int64))
        assert np.array_equal(d.values().numpy() < 0, (idx >> 31).astype(bool))
        assert (idx >> 31).any()                            # the case has negative entries at all
        # values are +-1, or +-m[col] exactly as the reference's v2 builder stores them
        o = orc.build_format(ei, n, 1)
        m = orc.col_multiplier(ei, n) if normalized else None
        if np.array_equal(o["parent"] % n, mat.parent.numpy() % n):
            crow, col, val = orc.deltas_csr(o, n, m)
            assert np.array_equal(d.crow_indices().numpy(), crow)
            assert np.array_equal(d.col_indices().numpy(), col)
            assert np.array_equal(d.values().numpy(), val)
        if normalized:
            assert np.array_equal(mat.col_multiplier.numpy(), m)
        # columns ascending within each row
        crow = d.crow_indices().numpy()
        for r in range(n):
            assert (np.diff(d.col_indices().numpy()[crow[r]:crow[r + 1]]) > 0).all()


def test_special_cases():
    n = 40
    ei = graphs.erdos_renyi(n, 0.5, 3)
    flat = cbm_matrix(torch.from_numpy(ei), None, alpha=10_000)
    assert flat.n_levels == 1 and (flat.parent == -1).all() and flat.nnz == ei.shape[1]
    assert np.array_equal((_u32(flat.idx)).astype(np.int64), ei[1][np.lexsort((ei[1], ei[0]))])
    clique = np.array([(i, j) for i in range(9) for j in range(9)], np.int32).T
    star = cbm_matrix(torch.from_numpy(clique), None, alpha=0)
    assert star.nnz == 9 and int((star.parent == -1).sum()) == 1 and star.n_levels == 2
    assert star.compression_ratio() > 1.5


def test_deep_chain_is_found():
    # the staircase of the alpha-sweep workload forces a path of chain+1 rows
    w = _small_chain_workload()
    for alpha in (0, 8, 32):
        mat = cbm_matrix(torch.from_numpy(w.edge_index), None, alpha=alpha)
        assert mat.n_levels >= 65                            # root -> c_0 -> ... -> c_64


def test_builder_is_thread_count_invariant_and_merges_duplicates():
    w = graphs.workload("c1")
    ei = torch.from_numpy(w.edge_index)
    a = cbm_matrix(ei, None, alpha=0, threads=1)
    b = cbm_matrix(ei, None, alpha=0, threads=4)
    perm = torch.randperm(ei.size(1), generator=torch.Generator().manual_seed(0))
    c = cbm_matrix(torch.cat([ei[:, perm], ei[:, :100]], dim=1), None, alpha=0)     # shuffled + duplicates
    for x in (b, c):
        for name in ("rowptr", "idx", "parent", "order", "level_off", "mst_row", "mst_col"):
            assert torch.equal(getattr(a, name), getattr(x, name)), name
        assert x.nnz_a == a.nnz_a


def test_builder_error_codes():
    fmt = _lib.CbmFormat()
    lib = _lib.host_lib()
    row = np.array([0, 1, 5], np.int32); col = np.array([1, 0, 0], np.int32)
    p = lambda a: a.ctypes.data_as(C.c_void_p)
    assert lib.cbm_build_host(p(row), p(col), 3, 3, 0, 0, C.byref(fmt)) == 3         # index out of range
    assert lib.cbm_build_host(p(row), p(col), 3, 0, 0, 0, C.byref(fmt)) == 3         # n <= 0
    assert lib.cbm_build_host(None, None, 3, 3, 0, 0, C.byref(fmt)) == 1             # NULL
    assert lib.cbm_build_host(p(row), p(col), 3, 6, 0, 0, None) == 1
    assert lib.cbm_build_host(p(row), p(col), 3, 6, 0, 0, C.byref(fmt)) == 0         # rows 2,3,4 empty: fine
    assert fmt.n == 6 and fmt.nnz == 2                                         # rows 1 and 5 are identical
    lib.cbm_format_free(C.byref(fmt))
    assert not fmt.rowptr
    with pytest.raises(ValueError):
        cbm_matrix(torch.zeros((3, 4), dtype=torch.int32), None)
    with pytest.raises(ValueError):
        cbm_matrix(torch.tensor([[0, 1], [1, 0]], dtype=torch.int32), None, rows=7)


def test_graph_generators_are_pinned():
    import json, os
    with open(os.path.join(os.path.dirname(__file__), "golden", "graph_hashes.json")) as f:
        want = json.load(f)
    for name in ("c1", "c2", "c2b", "c3", "c6", "c7"):
        w = graphs.workload(name)
        assert w.edge_index.shape[1] == want[name]["edges"] and w.n == want[name]["n"]
        assert graphs.edge_hash(w.edge_index) == want[name]["sha256"], name
        if name == "c1":
            from cbm4gnn_amd.utility import check_edge_index
            check_edge_index(torch.from_numpy(w.edge_index).long())
        if name == "c2b":                       # the size the configuration names: about 240k undirected edges
            assert abs((w.edge_index.shape[1] - w.n) // 2 - 240_000) < 5_000


def test_row_schedule_properties():
    from cbm4gnn_amd.cbm import schedule_rows
    rng = np.random.default_rng(0)
    n = 500
    lens = np.concatenate([rng.integers(0, 70, n - 5), [0, 64, 65, 700, 129]])
    rowptr = torch.tensor(np.concatenate([[0], np.cumsum(lens)]), dtype=torch.int32)
    parent = torch.tensor(rng.integers(-1, n, n), dtype=torch.int32)
    m = torch.tensor(rng.random(n) + 0.5, dtype=torch.float32)
    plain = schedule_rows(rowptr).numpy()
    scaled = schedule_rows(rowptr, parent, m).numpy()
    for s in (plain, scaled):
        rows = s[:, 2]
        assert sorted(rows.tolist()) == list(range(n))                      # a permutation
        assert np.array_equal(s[:, 0], rowptr.numpy()[:-1][rows]) and np.array_equal(s[:, 1], rowptr.numpy()[1:][rows])
        rounds = (lens[rows] + 63) // 64
        assert (np.diff(rounds) <= 0).all()                                 # longest first
        for r in np.unique(rounds):
            assert (np.diff(rows[rounds == r]) > 0).all()                   # stable inside a bucket
    assert (plain[:, 3].view(np.float32) == 1.0).all()
    want = np.where(parent.numpy()[scaled[:, 2]] < 0, m.numpy()[scaled[:, 2]], np.float32(1.0))
    assert np.array_equal(scaled[:, 3].view(np.float32), want.astype(np.float32))
    assert _lib.host_lib().cbm_schedule_rows(None, None, None, 3, None) == 1


def test_graphs_with_empty_rows_single_node_and_self_loop_only(orc):
    # node 3 has no edge at all (its row is empty), node 0 only a self loop
    ei = torch.tensor([[0, 1, 2, 4, 2], [0, 2, 1, 2, 4]], dtype=torch.int32)
    mat = cbm_matrix(ei, None, alpha=0)
    assert mat.num_rows == 5 and mat.nnz_a == 5
    assert np.diff(mat.rowptr.numpy())[3] == 0
    assert orc.check_format(ei.numpy(), 5, mat.rowptr.numpy(), _u32(mat.idx), mat.mst_row.numpy(), mat.mst_col.numpy())
    one = cbm_matrix(torch.tensor([[0], [0]], dtype=torch.int32), None, alpha=0, normalized=True)
    assert one.num_rows == 1 and one.nnz == 1 and one.n_levels == 1 and float(one.col_multiplier[0]) == 1.0


def _staged_build(ei, n, alpha, pairs):
    """cbm_builder_create -> (arrays) -> cbm_builder_finish; returns (status, format arrays, host arrays)."""
    host = _lib.host_lib()
    row = np.ascontiguousarray(ei[0], np.int32); col = np.ascontiguousarray(ei[1], np.int32)
    handle = C.c_void_p()
    assert host.cbm_builder_create(row.ctypes.data_as(C.c_void_p), col.ctypes.data_as(C.c_void_p), ei.shape[1], n, 2,
                                   C.byref(handle)) == 0
    try:
        ptrs = [C.c_void_p() for _ in range(6)]
        nnz = C.c_int64()
        assert host.cbm_builder_arrays(handle, *[C.byref(p) for p in ptrs], C.byref(nnz)) == 0
        take = lambda p, count, ct: np.ctypeslib.as_array(C.cast(p, C.POINTER(ct)), shape=(max(count, 1),))[:count].copy()
        arrays = dict(rowptr=take(ptrs[0], n + 1, C.c_int64), col=take(ptrs[1], nnz.value, C.c_int32),
                      colptr_t=take(ptrs[2], n + 1, C.c_int64), row_t=take(ptrs[3], nnz.value, C.c_int32),
                      after=take(ptrs[4], nnz.value, C.c_int64), row_nnz=take(ptrs[5], n, C.c_int32))
        fmt = _lib.CbmFormat()
        if pairs is None:
            rc = host.cbm_builder_finish(handle, alpha, None, -1, C.byref(fmt))
        else:
            p = np.ascontiguousarray(pairs, np.int32).reshape(-1, 3)
            rc = host.cbm_builder_finish(handle, alpha, p.ctypes.data_as(C.c_void_p) if len(p) else None, len(p), C.byref(fmt))
        out = None
        if rc == 0:
            g = lambda ptr, count: np.ctypeslib.as_array(ptr, shape=(max(count, 1),))[:count].copy()
            out = dict(nnz=int(fmt.nnz), n_candidates=int(fmt.n_candidates), rowptr=g(fmt.rowptr, n + 1),
                       idx=g(fmt.idx, int(fmt.nnz)), parent=g(fmt.parent, n), order=g(fmt.order, n),
                       level_off=g(fmt.level_off, fmt.n_levels + 1))
        host.cbm_format_free(C.byref(fmt))
        return rc, out, arrays
    finally:
        host.cbm_builder_free(handle)


def _all_pairs(ei, n):
    """(i, j > i, |row_i ^ row_j|) for every pair of rows that share a column, by dense arithmetic."""
    a = np.zeros((n, n), np.int64)
    a[ei[0], ei[1]] = 1
    s = a @ a.T
    i, j = np.nonzero(np.triu(s, 1))
    return np.stack([i, j, s[i, j]], 1).astype(np.int32)


@pytest.mark.parametrize("alpha", [0, 2, 5])
def test_staged_build_from_pairs_equals_one_call_build(alpha):
    n = 90
    ei = graphs.add_self_loops(graphs.sbm(n, 6, 0.6, 0.05, seed=alpha), n)
    ref = cbm_matrix(torch.from_numpy(ei), None, alpha=alpha)
    pairs = _all_pairs(ei, n)
    rng = np.random.default_rng(alpha)
    for given in (None, pairs, pairs[rng.permutation(len(pairs))]):      # host intersections / any order of pairs
        rc, out, arrays = _staged_build(ei, n, alpha, given)
        assert rc == 0
        assert out["nnz"] == ref.nnz and out["n_candidates"] == ref.n_candidates
        assert np.array_equal(out["rowptr"], ref.rowptr.numpy()) and np.array_equal(out["idx"], _u32(ref.idx))
        assert np.array_equal(out["parent"], ref.parent.numpy()) and np.array_equal(out["order"], ref.order.numpy())
        assert np.array_equal(out["level_off"], ref.level_off.numpy())
    # only the admissible pairs are needed
    nz = arrays["row_nnz"]
    adm = pairs[2 * pairs[:, 2] > np.minimum(nz[pairs[:, 0]], nz[pairs[:, 1]]) + alpha]
    rc, out, _ = _staged_build(ei, n, alpha, adm)
    assert rc == 0 and np.array_equal(out["idx"], _u32(ref.idx)) and np.array_equal(out["parent"], ref.parent.numpy())
    # the arrays handed to the GPU kernel: after[k] = first position in row_t of a row id > r within column col[k]
    rp, col, tp, rt, after = (arrays[k] for k in ("rowptr", "col", "colptr_t", "row_t", "after"))
    for r in range(n):
        for k in range(rp[r], rp[r + 1]):
            seg = rt[tp[col[k]]:tp[col[k] + 1]]
            assert after[k] == tp[col[k]] + np.searchsorted(seg, r, side="right") and seg[after[k] - tp[col[k]] - 1] == r


def test_staged_build_rejects_bad_pairs():
    n = 40
    ei = graphs.add_self_loops(graphs.erdos_renyi(n, 0.4, 1), n)
    pairs = _all_pairs(ei, n)
    assert _staged_build(ei, n, 0, pairs)[0] == 0
    for bad in ([5, 5, 1], [7, 3, 1], [0, n, 1], [-1, 2, 1], [0, 1, 0], [0, 1, 10_000]):
        assert _staged_build(ei, n, 0, np.vstack([pairs, [bad]]))[0] == 3, bad
    assert _staged_build(ei, n, 0, np.vstack([pairs, pairs[:1]]))[0] in (0, 3)     # a duplicate: refused if admissible
    nz = np.bincount(ei[0], minlength=n)
    adm = pairs[2 * pairs[:, 2] > np.minimum(nz[pairs[:, 0]], nz[pairs[:, 1]])]
    if len(adm):
        assert _staged_build(ei, n, 0, np.vstack([pairs, adm[:1]]))[0] == 3
    host = _lib.host_lib()
    assert host.cbm_builder_finish(None, 0, None, -1, C.byref(_lib.CbmFormat())) == 1
    assert host.cbm_builder_create(None, None, 5, 4, 1, C.byref(C.c_void_p())) == 1


@pytest.mark.parametrize("max_levels", [1, 2, 3, 6])
def test_depth_limit_gives_a_valid_shallower_format(orc, max_levels):
    w = _small_chain_workload()                               # 64-level chain below clique blocks
    ei, n = w.edge_index, w.n
    free = cbm_matrix(torch.from_numpy(ei), None, alpha=0)
    mat = cbm_matrix(torch.from_numpy(ei), None, alpha=0, max_levels=max_levels)
    assert free.n_levels > 6 and mat.n_levels == min(max_levels, free.n_levels)
    assert mat.nnz >= free.nnz and mat.n_candidates == free.n_candidates
    if max_levels == 1:
        assert mat.nnz == mat.nnz_a and (mat.parent == -1).all()           # flat tree: delta = A
    _assert_format_equals_derivation(orc, ei, n, mat)
    assert orc.check_format(ei, n, mat.rowptr.numpy(), _u32(mat.idx), mat.mst_row.numpy(), mat.mst_col.numpy())
    assert mat.check_format(torch.from_numpy(ei))
    # rows above the limit keep the parent the arborescence gave them
    keep = mat.parent.numpy() >= 0
    assert np.array_equal(mat.parent.numpy()[keep], free.parent.numpy()[keep])
    with pytest.raises(ValueError):
        cbm_matrix(torch.from_numpy(ei), None, alpha=0, max_levels=0)
