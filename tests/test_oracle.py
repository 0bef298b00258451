"""Pins the CPU oracle (oracle/cbm_oracle.c + oracle/cbm_oracle.py) WITHOUT the product:
brute force, closed forms, networkx, special cases and the committed golden vectors.  A dropped
term, a wrong sign or a transposed operand in the oracle fails at least one test here."""
import itertools

import numpy as np
import pytest
import torch

from cbm4gnn_amd import graphs


def _csr(ei, n):
    order = np.lexsort((ei[1], ei[0]))
    rp = np.zeros(n + 1, np.int64)
    np.add.at(rp, ei[0].astype(np.int64) + 1, 1)
    return np.cumsum(rp), ei[1][order].astype(np.int32)


@pytest.mark.parametrize("seed", range(6))
@pytest.mark.parametrize("alpha", [0, 1, 3, 7])
def test_candidate_rule_matches_bruteforce(orc, seed, alpha):
    # cbm_extensions.cpp:75-103 restated two ways: sparse accumulator in C, dense A A^T here
    n = 20 + 5 * seed
    ei = graphs.erdos_renyi(n, [0.1, 0.3, 0.5, 0.75][seed % 4], seed)
    if seed % 2:
        ei = graphs.add_self_loops(ei, n)
    rp, ci = _csr(ei, n)
    u, v, w = orc.candidates(n, rp, ci, alpha)
    got = set(zip(u.tolist(), v.tolist(), w.tolist()))
    assert len(got) == len(u)                       # no duplicates
    assert got == orc.candidates_bruteforce(orc.dense_adjacency(ei, n), alpha)
    # emission order of the reference: root edge of row i first, then pairs (i, j>i), j ascending
    roots = np.flatnonzero(u == n)
    assert np.array_equal(v[roots], np.arange(n))


def _brute_msa_weight(n, edges, root):
    best = None
    inc = [[(u, w) for (u, v, w) in edges if v == x] for x in range(n)]
    nodes = [x for x in range(n) if x != root]
    for choice in itertools.product(*[inc[x] for x in nodes]):
        par = {x: c[0] for x, c in zip(nodes, choice)}
        ok = True
        for x in nodes:                              # every node must reach the root
            seen, y = set(), x
            while y != root:
                if y in seen:
                    ok = False
                    break
                seen.add(y)
                y = par[y]
            if not ok:
                break
        if ok:
            wsum = sum(c[1] for c in choice)
            best = wsum if best is None else min(best, wsum)
    return best


@pytest.mark.parametrize("seed", range(25))
def test_msa_weight_bruteforce_tiny(orc, seed):
    rng = np.random.default_rng(seed)
    n = int(rng.integers(3, 7))
    root = n - 1
    edges = [(root, v, int(rng.integers(1, 12))) for v in range(n - 1)]
    for u in range(n - 1):
        for v in range(n - 1):
            if u != v and rng.random() < 0.6:
                edges.append((u, v, int(rng.integers(0, 9))))
    eu, ev, ew = map(np.array, zip(*edges))
    chosen, w = orc.msa(n, eu, ev, ew, root)
    assert w == _brute_msa_weight(n, edges, root)
    # the chosen edges form an arborescence of that weight
    assert sum(ew[chosen[v]] for v in range(n) if v != root) == w
    for v in range(n):
        if v == root:
            continue
        assert ev[chosen[v]] == v
        y, steps = v, 0
        while y != root:
            y = int(eu[chosen[y]]); steps += 1
            assert steps <= n


@pytest.mark.parametrize("seed", range(8))
def test_msa_weight_matches_networkx(orc, seed):
    nx = pytest.importorskip("networkx")
    rng = np.random.default_rng(100 + seed)
    n = int(rng.integers(8, 40))
    root = n - 1
    edges = {}
    for v in range(n - 1):
        edges[(root, v)] = int(rng.integers(5, 30))
    for _ in range(n * 4):
        u, v = int(rng.integers(0, n - 1)), int(rng.integers(0, n - 1))
        if u != v:
            edges[(u, v)] = int(rng.integers(0, 20))
    g = nx.DiGraph()
    for (u, v), w in edges.items():
        g.add_edge(u, v, weight=w)
    ref = nx.minimum_spanning_arborescence(g, attr="weight")
    ref_w = sum(d["weight"] for _, _, d in ref.edges(data=True))
    eu = np.array([k[0] for k in edges]); ev = np.array([k[1] for k in edges]); ew = np.array(list(edges.values()))
    _, w = orc.msa(n, eu, ev, ew, root)
    assert w == ref_w


@pytest.mark.parametrize("seed", range(6))
@pytest.mark.parametrize("alpha", [0, 2, 5])
def test_build_reconstructs_every_row(orc, seed, alpha):
    # the reference's check_format (cbm.py:69-115): tree + signed deltas rebuild A exactly
    n = 30 + 7 * seed
    ei = graphs.erdos_renyi(n, 0.4, seed)
    fmt = orc.build_format(ei, n, alpha)
    crow, col, val = orc.deltas_csr(fmt, n)
    idx = col.astype(np.uint32) | ((val < 0).astype(np.uint32) << 31)
    assert orc.check_format(ei, n, crow, idx, fmt["mst_row"], fmt["mst_col"])
    assert fmt["nnz"] == fmt["msa_weight"]
    assert fmt["nnz"] <= ei.shape[1]
    # deltas derived from the parent array by set differences agree with the merge
    f2 = orc.format_from_parent(ei, n, fmt["parent"])
    assert np.array_equal(f2["rowptr"], crow) and np.array_equal(f2["idx"], idx)
    assert np.array_equal(f2["mst_row"], fmt["mst_row"]) and np.array_equal(f2["mst_col"], fmt["mst_col"])
    # alpha admission: a non-root parent saves more than alpha entries
    deg = np.bincount(ei[0], minlength=n)
    nd = np.diff(crow)
    for v in range(n):
        if fmt["parent"][v] != n:
            assert nd[v] < deg[v] - alpha


def test_special_case_flat_tree_when_alpha_is_large(orc):
    n = 40
    ei = graphs.erdos_renyi(n, 0.5, 3)
    fmt = orc.build_format(ei, n, alpha=10_000)
    assert (fmt["parent"] == n).all()
    crow, col, val = orc.deltas_csr(fmt, n)
    rp, ci = _csr(ei, n)
    assert np.array_equal(crow, rp) and np.array_equal(col, ci) and (val == 1).all()
    assert fmt["n_candidates"] == n
    assert np.array_equal(fmt["mst_col"], np.arange(n)) and fmt["mst_row"][n] == 0 and fmt["mst_row"][n + 1] == n


def test_special_case_identical_rows_give_empty_delta(orc):
    # rows 0 and 1 both equal {2,3,4}; one of them becomes a child of the other with no delta
    edges = [(0, 2), (0, 3), (0, 4), (1, 2), (1, 3), (1, 4), (2, 0), (2, 1), (3, 0), (3, 1), (4, 0), (4, 1)]
    ei = np.array(edges, np.int32).T
    fmt = orc.build_format(ei, 5, alpha=0)
    crow, _, _ = orc.deltas_csr(fmt, 5)
    nd = np.diff(crow)
    assert (nd[0] == 0) != (nd[1] == 0)
    child = 0 if nd[0] == 0 else 1
    assert fmt["parent"][child] == 1 - child


def test_special_case_clique_with_self_loops_is_a_star_of_empty_deltas(orc):
    n = 9
    ei = np.array([(i, j) for i in range(n) for j in range(n)], np.int32).T
    fmt = orc.build_format(ei, n, alpha=0)
    assert fmt["nnz"] == n                     # one full row, eight empty deltas
    assert (fmt["parent"] == n).sum() == 1


@pytest.mark.parametrize("case", range(5))
def test_golden_products_plain_bit_exact(orc, golden, case):
    # integer features: every partial sum is an exact fp32 integer, so any summation order gives
    # exactly the dense fp64 product (tests/test_matmul_correctness.py:22 uses randint(0, 10))
    ei, x = golden[f"case{case}_edge_index"], golden[f"case{case}_x"]
    n = x.shape[0]
    for alpha in (0, 2, 3):
        fmt = orc.build_format(ei, n, alpha)
        crow, col, val = orc.deltas_csr(fmt, n)
        y = orc.spmm_update(crow, col, val, fmt["mst_row"], fmt["mst_col"], x)
        assert np.array_equal(y.astype(np.float64), golden[f"case{case}_ax"])
        # multi-threaded walk (cbm_extensions.cpp:1166-1218) is the same function of the tree
        y8 = orc.spmm_update(crow, col, val, fmt["mst_row"], fmt["mst_col"], x, threads=4)
        assert np.array_equal(y, y8)


@pytest.mark.parametrize("case", range(5))
def test_golden_products_normalised(orc, golden, case):
    ei, x = golden[f"case{case}_edge_index"], golden[f"case{case}_x"]
    n = x.shape[0]
    m = orc.col_multiplier(ei, n)
    assert np.allclose(m, golden[f"case{case}_row_degree"].astype(np.float64) ** -0.5, rtol=1e-7)
    for alpha in (0, 3):
        fmt = orc.build_format(ei, n, alpha)
        crow, col, val = orc.deltas_csr(fmt, n, m)
        y = orc.spmm_update(crow, col, val, fmt["mst_row"], fmt["mst_col"], x, m)
        assert orc.max_rel_err(y, golden[f"case{case}_ax_normalized"]) <= 1e-4   # north-star tolerance
        np.testing.assert_allclose(y, golden[f"case{case}_ax_normalized"], rtol=1e-4, atol=1e-4)


@pytest.mark.parametrize("case", range(5))
def test_dense_product_closed_form_against_golden(orc, golden, case):
    """``dense_product`` is the fp64 closed form the GPU tests lean on; the golden products were written by
    a script that imports neither kernels nor oracle (tests/golden/make_fixtures.py)."""
    ei, x = golden[f"case{case}_edge_index"], golden[f"case{case}_x"]
    n = x.shape[0]
    assert np.array_equal(orc.dense_product(ei, n, x, False), golden[f"case{case}_ax"])         # integers: exact
    np.testing.assert_allclose(orc.dense_product(ei, n, x, True), golden[f"case{case}_ax_normalized"], rtol=1e-13, atol=0)
    # a directed list must not be symmetrised, and the row (not the column) degree normalises
    tri = np.array([[0, 0, 1], [1, 2, 2]], np.int32)
    got = orc.dense_product(np.concatenate([tri, np.array([[2], [2]], np.int32)], axis=1), 3, np.eye(3, dtype=np.float32), False)
    assert np.array_equal(got, np.array([[0, 1, 1], [0, 0, 1], [0, 0, 1]], np.float64))
    loops = np.array([[0, 0, 1, 2], [0, 1, 1, 2]], np.int32)                                   # row degrees 2, 1, 1
    got = orc.dense_product(loops, 3, np.eye(3, dtype=np.float32), True)
    assert np.allclose(got, np.array([[0.5, 2 ** -0.5, 0], [0, 1, 0], [0, 0, 1]]), rtol=1e-15)


def test_fused_walk_formula_by_hand(orc):
    # chain root -> 0 -> 1 -> 2, d = 10: columns 0..7 take the FMA form, 8..9 the division
    # form (cbm_extensions.cpp:966-990); recompute both in NumPy fp32 step by step
    n, d = 3, 10
    mst_row = np.array([0, 1, 2, 2, 3], np.int32)       # children: 0->[1], 1->[2], 2->[], root->[0]
    mst_col = np.array([1, 2, 0], np.int32)
    m = np.array([0.5, 0.37, 0.81], np.float32)
    rng = np.random.default_rng(5)
    z = rng.standard_normal((n, d)).astype(np.float32)
    y = orc.update_fused(mst_row, mst_col, m, z.copy())
    e = z.copy()
    e[0] = e[0] * m[0]
    for u, v in ((0, 1), (1, 2)):
        inv = np.float32(1.0) / m[u]
        head = (e[u, :8].astype(np.float64) * np.float64(inv) + e[v, :8].astype(np.float64)).astype(np.float32) * m[v]
        tail = (e[v, 8:] + e[u, 8:] / m[u]).astype(np.float32) * m[v]
        e[v] = np.concatenate([head, tail])
    assert np.array_equal(y, e)
    # and mathematically: y[v] = m[v] * sum of z over the path
    want = np.cumsum(z.astype(np.float64), axis=0) * m[:, None].astype(np.float64)
    assert orc.max_rel_err(y, want) < 1e-6


def test_plain_walk_is_a_path_prefix_sum(orc):
    n, d = 6, 5
    parent = [-1, 0, 1, 1, -1, 4]
    kids = [[] for _ in range(n + 1)]
    for v, p in enumerate(parent):
        kids[n if p < 0 else p].append(v)
    mst_col = np.array(sum(kids, []), np.int32)
    mst_row = np.concatenate([[0], np.cumsum([len(k) for k in kids])]).astype(np.int32)
    z = np.arange(n * d, dtype=np.float32).reshape(n, d)
    y = orc.update_plain(mst_row, mst_col, z.copy())
    want = z.copy()
    for v in (1, 2, 3, 5):
        want[v] = z[v] + want[parent[v]]
    assert np.array_equal(y, want)


def test_col_multiplier_equals_torch_pow(orc):
    # the reference evaluates val ** (-1/2) on a torch fp32 tensor (cbm.py:40-41)
    ei = graphs.workload("c1").edge_index
    m = orc.col_multiplier(ei, 4096)
    deg = torch.bincount(torch.from_numpy(ei[0]).long(), minlength=4096).float()
    assert np.array_equal(m, deg.pow(-0.5).numpy())
    assert np.array_equal(m, np.array([float(v ** (-1 / 2)) for v in deg[:64]], np.float32).tolist() + m[64:].tolist())


def test_csr_spmm_against_mkl_and_dense(orc):
    rng = np.random.default_rng(0)
    n, d = 300, 37
    ei = graphs.erdos_renyi(n, 0.05, 11)
    rp, ci = _csr(ei, n)
    val = rng.standard_normal(ci.shape[0]).astype(np.float32)
    x = rng.standard_normal((n, d)).astype(np.float32)
    y = orc.csr_spmm(rp, ci, val, x, threads=2)
    a = np.zeros((n, n)); a[ei[0][np.lexsort((ei[1], ei[0]))], ci] = val
    assert orc.max_rel_err(y, a @ x.astype(np.float64)) < 1e-6
    if orc.mkl() is not None:                      # the reference's own SpMM routine, via torch's MKL
        rp32 = rp.astype(np.int32)
        ym = np.empty_like(y)
        orc.mkl_csr_spmm(np.ascontiguousarray(rp32[:-1]), np.ascontiguousarray(rp32[1:]), ci, val, x, ym)
        assert orc.max_rel_err(y, ym) < 1e-6


def test_compression_ratio_formula(orc):
    # benchmark/utility.py:45-64 in element counts
    assert orc.compression_ratio(10, 40, 40) == pytest.approx((11 + 80) / (11 + 80 + 12 + 10))
    assert orc.compression_ratio(10, 40, 10) > 1.0


def test_grouped_csr_spmm_order_is_pinned(orc):
    """``csr_spmm(groups=g)``: entry k of a row goes to partial sum k mod g (each an in-order FMA
    chain) and the g sums are added pairwise as a balanced tree.  Pinned by integer features
    (exact for every order), by real features against the in-order sum, and by a row whose fp32
    result differs between the orders in a way worked out by hand."""
    rng = np.random.default_rng(3)
    n, d = 257, 19
    ei = graphs.add_self_loops(graphs.erdos_renyi(n, 0.3, 17), n)
    rp, ci = _csr(ei, n)
    a = np.zeros((n, n))
    a[ei[0], ei[1]] = 1.0
    xi = rng.integers(0, 10, (n, d)).astype(np.float32)
    xr = rng.standard_normal((n, d)).astype(np.float32)
    val = rng.standard_normal(ci.shape[0]).astype(np.float32)
    av = np.zeros((n, n)); av[ei[0][np.lexsort((ei[1], ei[0]))], ci] = val
    in_order = orc.csr_spmm(rp, ci, val, xr)
    for g in (2, 4, 8, 16, 32, 64):
        assert np.array_equal(orc.csr_spmm(rp, ci, None, xi, groups=g).astype(np.float64), a @ xi.astype(np.float64))
        got = orc.csr_spmm(rp, ci, val, xr, threads=2, groups=g)
        assert orc.max_rel_err(got, in_order) <= 1e-6
        assert orc.max_rel_err(got, av @ xr.astype(np.float64)) <= 1e-6
        assert not np.array_equal(got, in_order)            # it IS another order
    assert np.array_equal(orc.csr_spmm(rp, ci, val, xr, groups=1), in_order)
    # one row (1e8, 1, -1e8, 1) times a column of ones, fp32:
    #   in order          ((1e8 + 1) - 1e8) + 1 = (1e8 - 1e8) + 1           = 1
    #   2 partial sums    (1e8 - 1e8) + (1 + 1)                             = 2
    #   4 partial sums    (1e8 + 1) + (-1e8 + 1) = 1e8 + -1e8               = 0
    #   8 partial sums    ((1e8 + 1) + (-1e8 + 1)) + ((0 + 0) + (0 + 0))    = 0
    rp1 = np.array([0, 4], np.int32); c1 = np.array([0, 1, 2, 3], np.int32)
    v1 = np.array([1e8, 1.0, -1e8, 1.0], np.float32)
    ones = np.ones((4, 1), np.float32)
    # the matrix is 1 x 4: the oracle takes the row count from crow
    assert [float(orc.csr_spmm(rp1, c1, v1, ones, groups=g)[0, 0]) for g in (1, 2, 4, 8)] == [1.0, 2.0, 0.0, 0.0]
    # six entries in 4 partial sums: sums 0 and 1 get two entries each, in order
    #   p0 = 1e8 + 3 (= 1e8, 3 is below half an ulp of 8), p1 = 1 + 5 = 6, p2 = -1e8, p3 = 1
    #   tree: (p0 + p1) + (p2 + p3) = (1e8 + 6 -> 1e8 + 8) + (-1e8 + 1 -> -1e8) = 8
    rp2 = np.array([0, 6], np.int32); c2 = np.arange(6, dtype=np.int32)
    v2 = np.array([1e8, 1.0, -1e8, 1.0, 3.0, 5.0], np.float32)
    assert float(orc.csr_spmm(rp2, c2, v2, np.ones((6, 1), np.float32), groups=4)[0, 0]) == 8.0
