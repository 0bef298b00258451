"""Full-size checks at the benchmark workloads, where the CPU oracle is too slow to run per test:
size-independent properties (linearity, determinism, exactness on integer features, agreement
with the plain CSR product) plus one CPU CSR product as the anchor."""
import sys

import numpy as np
import pytest
import torch

from cbm4gnn_amd import _lib, graphs
from cbm4gnn_amd.cbm import cbm_matrix, csr_spmm

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def c3():
    if not torch.cuda.is_available():
        pytest.skip("no HIP device")
    w = graphs.workload("c3")
    ei = torch.from_numpy(w.edge_index)
    mats = {a: cbm_matrix(ei, None, alpha=a, normalized=True) for a in (0, 16)}
    return w, mats


def _mul(mat, xd):
    yd = torch.empty_like(xd)
    mat.omp_mkl_csr_fused_spmm_update(xd, yd)
    return yd


def test_full_size_against_cpu_csr_and_gpu_csr(c3, orc):
    w, mats = c3
    x = w.features(0)
    ei = w.edge_index
    m = orc.col_multiplier(ei, w.n)
    order = np.lexsort((ei[1], ei[0]))
    rp = np.concatenate([[0], np.cumsum(np.bincount(ei[0], minlength=w.n))]).astype(np.int32)
    vals = (m[ei[0][order]] * m[ei[1][order]]).astype(np.float32)
    cpu = orc.csr_spmm(rp, ei[1][order], vals, x.numpy(), threads=orc.max_threads())
    xd = x.cuda()
    for alpha, mat in mats.items():
        print("[gpu-case] c3 full size alpha", alpha, flush=True); sys.stdout.flush()
        got = _mul(mat, xd).cpu().numpy()
        assert orc.max_rel_err(got, cpu) <= 1e-3            # vs plain CSR A_hat X
        np.testing.assert_allclose(got, cpu, rtol=1e-3, atol=1e-4)
    yd = torch.empty_like(xd)
    csr_spmm(torch.from_numpy(rp).cuda(), torch.from_numpy(ei[1][order].astype(np.int32)).cuda(),
             torch.from_numpy(vals).cuda(), xd, yd)
    assert orc.max_rel_err(yd.cpu().numpy(), cpu) <= 1e-5
    # alpha = 16 prunes every candidate on this graph: flat tree, Delta == A
    assert mats[16].n_levels == 1 and mats[16].nnz == ei.shape[1]
    assert mats[0].n_levels > 1 and mats[0].nnz < ei.shape[1]


def test_full_size_linearity_and_determinism(c3):
    w, mats = c3
    g = torch.Generator().manual_seed(5)
    a = torch.randn((w.n, 256), generator=g).cuda(); b = torch.randn((w.n, 256), generator=g).cuda()
    for alpha, mat in mats.items():
        print("[gpu-case] c3 linearity alpha", alpha, flush=True); sys.stdout.flush()
        ya, yb, yab = _mul(mat, a), _mul(mat, b), _mul(mat, a + 2.0 * b)
        err = (yab - (ya + 2.0 * yb)).abs().max() / yab.abs().max()
        assert float(err) <= 1e-5
        assert torch.equal(ya, _mul(mat, a))                # no atomics: run-to-run identical
        assert float(_mul(mat, torch.zeros_like(a)).abs().max()) == 0.0


def test_full_size_plain_integer_features_exact(c3):
    # un-normalised operator on integer features: every tree, every order gives the exact sums
    w, _ = c3
    ei = torch.from_numpy(w.edge_index)
    x = torch.randint(0, 4, (w.n, 256), generator=torch.Generator().manual_seed(0)).float().cuda()
    order = np.lexsort((w.edge_index[1], w.edge_index[0]))
    rp = torch.from_numpy(np.concatenate([[0], np.cumsum(np.bincount(w.edge_index[0], minlength=w.n))]).astype(np.int32)).cuda()
    col = torch.from_numpy(w.edge_index[1][order].astype(np.int32)).cuda()
    want = torch.empty_like(x)
    csr_spmm(rp, col, None, x, want)
    for alpha in (0, 4):
        print("[gpu-case] c3 integer alpha", alpha, flush=True); sys.stdout.flush()
        mat = cbm_matrix(ei, None, alpha=alpha)
        got = torch.empty_like(x)
        mat.omp_mkl_csr_spmm_update(x, got)
        assert torch.equal(got, want)


def test_alpha_sweep_graph_full_size_deep_chain_exact():
    """132,534 nodes, 82.5 M non-zeros, a 2000-level chain, d = 512, plain operator, integer
    features: every partial sum is an exact integer, so the CBM product (delta SpMM, 9 wide levels,
    narrow levels, the 1986-level chain kernel) must equal the CSR product bit for bit."""
    if not torch.cuda.is_available():
        pytest.skip("no HIP device")
    w = graphs.workload("c5")
    print("[gpu-case] c5 full size, building", flush=True); sys.stdout.flush()
    ei = torch.from_numpy(w.edge_index)
    mat = cbm_matrix(ei, None, alpha=0)
    assert mat.n_levels >= 2001 and mat.compression_ratio() > 2.0
    x = torch.randint(0, 3, (w.n, 512), generator=torch.Generator().manual_seed(1)).float().cuda()
    order = np.lexsort((w.edge_index[1], w.edge_index[0]))
    rp = torch.from_numpy(np.concatenate([[0], np.cumsum(np.bincount(w.edge_index[0], minlength=w.n))]).astype(np.int32)).cuda()
    col = torch.from_numpy(w.edge_index[1][order].astype(np.int32)).cuda()
    want = torch.empty_like(x)
    csr_spmm(rp, col, None, x, want)
    print("[gpu-case] c5 full size, multiply", flush=True); sys.stdout.flush()
    got = torch.empty_like(x)
    mat.omp_mkl_csr_spmm_update(x, got)
    assert torch.equal(got, want)
    # the deepest chain row really is the sum of ~2050 columns
    deep = int(mat.order[-1])
    assert float(got[deep].max()) > 1000.0
    # and on real-valued features: within the plain-CSR tolerance, linear, deterministic
    a = torch.randn((w.n, 512), generator=torch.Generator().manual_seed(2)).cuda()
    ya = torch.empty_like(a); mat.omp_mkl_csr_spmm_update(a, ya)
    csr_spmm(rp, col, None, a, want)
    assert float((ya - want).abs().max() / want.abs().max()) <= 1e-3
    yb = torch.empty_like(a); mat.omp_mkl_csr_spmm_update(a, yb)
    assert torch.equal(ya, yb)


def _csr(ei, n):
    order = np.lexsort((ei[1], ei[0]))
    rp = np.concatenate([[0], np.cumsum(np.bincount(ei[0], minlength=n))]).astype(np.int64)
    return rp, np.ascontiguousarray(ei[1][order].astype(np.int32))


def _rows_fp64(rp, col, m, x, rows, transposed_scale=None):
    """Rows ``rows`` of diag(m) A diag(m) X (m None: A X) in fp64 with SciPy, straight from the CSR
    arrays of the edge list: an anchor that shares no code with the kernels or the oracle."""
    import scipy.sparse as sp
    cnt = rp[rows + 1] - rp[rows]
    take = np.repeat(rp[rows], cnt) + (np.arange(int(cnt.sum())) - np.repeat(np.cumsum(cnt) - cnt, cnt))
    c = col[take]
    v = np.ones(take.shape[0]) if m is None else (np.repeat(m[rows].astype(np.float64), cnt) * m[c].astype(np.float64))
    sub = sp.csr_matrix((v, c, np.concatenate([[0], np.cumsum(cnt)])), shape=(rows.shape[0], x.shape[0]))
    return sub @ x.astype(np.float64)


def _assert_rows_close(got, want):
    """fp32 product rows against fp64 rows: the global max-relative error at 1e-4, and element by element
    at rtol 1e-4 with an absolute floor of 1e-5 of the largest element (so that small elements are held
    to their own size, not to the largest one's)."""
    assert _max_rel(got, want) <= 1e-4
    np.testing.assert_allclose(got, want, rtol=1e-4, atol=1e-5 * float(np.abs(want).max()))


def _max_rel(got, want):
    return float(np.abs(got - want).max() / np.abs(want).max())


@pytest.fixture(scope="module")
def c4():
    if not torch.cuda.is_available():
        pytest.skip("no HIP device")
    w = graphs.workload("c4")
    print("[gpu-case] c4 full size, building", flush=True); sys.stdout.flush()
    mat = cbm_matrix(torch.from_numpy(w.edge_index), None, alpha=2, normalized=True)
    rp, col = _csr(w.edge_index, w.n)
    return w, mat, rp, col


def test_gcn_graph_full_size_against_cpu_rows_and_gpu_csr(c4):
    """232,965 nodes, 114 M non-zeros (the GCN epoch workload), normalised, d = 128 and d = 41:
    2,048 random rows of the product against an fp64 SciPy product built from the edge list, and
    the whole product against the GPU CSR baseline."""
    w, mat, rp, col = c4
    m = mat.col_multiplier.numpy()
    val = torch.from_numpy((np.repeat(m, np.diff(rp)) * m[col]).astype(np.float32)).cuda()
    rp_d, col_d = torch.from_numpy(rp.astype(np.int32)).cuda(), torch.from_numpy(col).cuda()
    rows = np.sort(np.random.default_rng(4).choice(w.n, size=2048, replace=False))
    rows_d = torch.from_numpy(rows).cuda()
    for d in (128, 41):
        print("[gpu-case] c4 full size, d", d, flush=True); sys.stdout.flush()
        x = torch.randn((w.n, d), generator=torch.Generator().manual_seed(d))
        xd = x.cuda()
        got = _mul(mat, xd)
        want_rows = _rows_fp64(rp, col, m, x.numpy(), rows)
        _assert_rows_close(got[rows_d].cpu().numpy().astype(np.float64), want_rows)
        base = torch.empty_like(xd)
        csr_spmm(rp_d, col_d, val, xd, base)
        _assert_rows_close(base[rows_d].cpu().numpy().astype(np.float64), want_rows)
        assert float((got - base).abs().max() / base.abs().max()) <= 1e-3
        ones = _mul(mat, torch.ones_like(xd))
        assert float(ones.min()) > 0.0 and torch.isfinite(ones).all()
        # the two-launch plan (slab kernel on the remote entries first) sums the same entries in another order
        assert mat.is_tiled() and not mat.has_cut_rows()
        try:
            assert _lib.hip_lib().cbm_set_tiled_fused(0) == 0
            two = _mul(mat, xd)
        finally:
            assert _lib.hip_lib().cbm_set_tiled_fused(1) == 0
        assert float((two - got).abs().max() / got.abs().max()) <= 1e-5 and not torch.equal(two, got)


def test_gcn_epoch_full_size_anchored_rows(c4):
    """One full-size forward + backward of the 2-layer GCN (602-128-41) with the fused CBM layers:
    loss and weight gradients against the CSR-layer model, and every aggregation of the epoch --
    both forward multiplies and both backward multiplies, on the inputs they really had -- against
    2,048 fp64 rows computed with SciPy from the edge list."""
    from cbm4gnn_amd.gcn import CBMGCNLayer, CSRGCNLayer, TwoLayerGCN, csr_operator
    w, mat, rp, col = c4
    n, hidden, classes = w.n, 128, 41
    dev = torch.device("cuda")
    m = mat.col_multiplier.numpy()
    g = torch.Generator().manual_seed(0)
    x = torch.randn((n, w.d), generator=g).to(dev)
    labels = torch.randint(0, classes, (n,), generator=g).to(dev)
    torch.manual_seed(0)
    model = TwoLayerGCN(CBMGCNLayer(w.d, hidden, mat, relu=True), CBMGCNLayer(hidden, classes, mat), relu_between=False).to(dev)
    print("[gpu-case] c4 full size gcn epoch, fused layers", flush=True); sys.stdout.flush()
    logits = model(x)
    loss = torch.nn.functional.cross_entropy(logits, labels)
    loss.backward()
    torch.cuda.synchronize()
    rows = np.sort(np.random.default_rng(6).choice(n, size=2048, replace=False))
    rows_d = torch.from_numpy(rows).to(dev)
    b1, b2 = model.first_layer._cache, model.last_layer._cache
    cpu = lambda t: t.detach().cpu().numpy()
    # forward, layer 1: y1 = relu(A_hat h1)
    want = np.maximum(_rows_fp64(rp, col, m, cpu(b1["h"]), rows), 0.0)
    _assert_rows_close(cpu(b1["y"][rows_d]).astype(np.float64), want)
    # forward, layer 2: logits = A_hat h2
    want = _rows_fp64(rp, col, m, cpu(b2["h"]), rows)
    _assert_rows_close(cpu(logits[rows_d]).astype(np.float64), want)
    # backward, layer 2: gh2 = A_hat^T g_logits (the graph is symmetric), g_logits = (softmax - onehot) / n
    g_logits = torch.softmax(logits.detach(), dim=1)
    g_logits[torch.arange(n, device=dev), labels] -= 1.0
    g_logits /= n
    want = _rows_fp64(rp, col, m, cpu(g_logits), rows)
    _assert_rows_close(cpu(b2["gh"][rows_d]).astype(np.float64), want)
    # backward, layer 1: gh1 = A_hat^T (relu'(y1) * (gh2 W2))
    g_y1 = (b2["gh"] @ model.last_layer.lin.weight.detach()) * (b1["y"] > 0)
    want = _rows_fp64(rp, col, m, cpu(g_y1), rows)
    _assert_rows_close(cpu(b1["gh"][rows_d]).astype(np.float64), want)
    # the CSR-layer model: same loss, same weight gradients
    print("[gpu-case] c4 full size gcn epoch, csr layers", flush=True); sys.stdout.flush()
    ei = torch.from_numpy(w.edge_index)
    mt = mat.col_multiplier
    fwd = csr_operator(torch.stack([ei[1], ei[0]]), n, mt[ei[0].long()] * mt[ei[1].long()], dev)
    torch.manual_seed(0)
    base = TwoLayerGCN(CSRGCNLayer(w.d, hidden, fwd, fwd), CSRGCNLayer(hidden, classes, fwd, fwd)).to(dev)
    base_loss = torch.nn.functional.cross_entropy(base(x), labels)
    base_loss.backward()
    assert abs(float(loss.detach()) - float(base_loss.detach())) <= 1e-5 * abs(float(base_loss.detach()))
    for p, q in zip(model.parameters(), base.parameters()):
        assert float((p.grad - q.grad).abs().max() / q.grad.abs().max()) <= 1e-3


def test_duplication_graph_full_size():
    """12,000-node duplication graph at full size (3.64 M non-zeros, A + I normalised, d = 128),
    alpha 0 and 8: 1,024 rows against fp64 SciPy rows, everything against the GPU CSR baseline."""
    if not torch.cuda.is_available():
        pytest.skip("no HIP device")
    w = graphs.workload("c2")
    rp, col = _csr(w.edge_index, w.n)
    x = w.features(0)
    xd = x.cuda()
    rows = np.sort(np.random.default_rng(2).choice(w.n, size=1024, replace=False))
    rows_d = torch.from_numpy(rows).cuda()
    for alpha in (0, 8):
        print("[gpu-case] c2 full size alpha", alpha, flush=True); sys.stdout.flush()
        mat = cbm_matrix(torch.from_numpy(w.edge_index), None, alpha=alpha, normalized=True)
        assert mat.n_levels > 4 and mat.compression_ratio() > 1.4
        m = mat.col_multiplier.numpy()
        got = _mul(mat, xd)
        want_rows = _rows_fp64(rp, col, m, x.numpy(), rows)
        _assert_rows_close(got[rows_d].cpu().numpy().astype(np.float64), want_rows)
        val = torch.from_numpy((np.repeat(m, np.diff(rp)) * m[col]).astype(np.float32)).cuda()
        base = torch.empty_like(xd)
        csr_spmm(torch.from_numpy(rp.astype(np.int32)).cuda(), torch.from_numpy(col).cuda(), val, xd, base)
        assert float((got - base).abs().max() / base.abs().max()) <= 1e-3
        # the multiply walked the 11-level tree in one launch (every row down its own ancestor path): bit for
        # bit what the level-by-level walk returns
        assert mat._walks_paths(w.n, xd.size(1))
        mat.path_walk_max_bytes = 0
        assert torch.equal(_mul(mat, xd), got)


def test_duplication_graph_at_the_configured_size():
    """c2b: the duplication process held to the ~240k undirected edges the configuration names (489,520
    non-zeros with A + I), normalised, d = 128, alpha 0 and 8: 1,024 rows against fp64 SciPy rows, everything
    against the GPU CSR baseline, and the one-launch path walk against the level-by-level walk."""
    if not torch.cuda.is_available():
        pytest.skip("no HIP device")
    w = graphs.workload("c2b")
    assert abs((w.edge_index.shape[1] - w.n) // 2 - 240_000) < 5_000
    rp, col = _csr(w.edge_index, w.n)
    x = w.features(0)
    xd = x.cuda()
    rows = np.sort(np.random.default_rng(3).choice(w.n, size=1024, replace=False))
    rows_d = torch.from_numpy(rows).cuda()
    for alpha in (0, 8):
        print("[gpu-case] c2b full size alpha", alpha, flush=True); sys.stdout.flush()
        mat = cbm_matrix(torch.from_numpy(w.edge_index), None, alpha=alpha, normalized=True)
        assert mat.n_levels >= 3 and 1.0 < mat.compression_ratio() < 1.3
        m = mat.col_multiplier.numpy()
        got = _mul(mat, xd)
        _assert_rows_close(got[rows_d].cpu().numpy().astype(np.float64), _rows_fp64(rp, col, m, x.numpy(), rows))
        val = torch.from_numpy((np.repeat(m, np.diff(rp)) * m[col]).astype(np.float32)).cuda()
        base = torch.empty_like(xd)
        csr_spmm(torch.from_numpy(rp.astype(np.int32)).cuda(), torch.from_numpy(col).cuda(), val, xd, base)
        assert float((got - base).abs().max() / base.abs().max()) <= 1e-3
        assert mat._walks_paths(w.n, xd.size(1))
        mat.path_walk_max_bytes = 0                          # the walk by subtrees / level by level instead
        assert torch.equal(_mul(mat, xd), got)
        mat.subtree_walk = "off"
        assert torch.equal(_mul(mat, xd), got)


def test_deep_and_wide_tree_full_size():
    """c6: 182,400 rows in 800 staircases + noise, compression 9.4, 65 tree levels of ~3,000 rows: the one-launch
    multiply by subtrees against the SpMM + walk, the walk by subtrees against the level-by-level walk bit for bit, 1,024 rows against fp64 SciPy rows, the
    whole product against the GPU CSR baseline; short delta rows in batches against one row per wavefront."""
    if not torch.cuda.is_available():
        pytest.skip("no HIP device")
    w = graphs.workload("c6")
    print("[gpu-case] c6 full size, building", flush=True); sys.stdout.flush()
    mat = cbm_matrix(torch.from_numpy(w.edge_index), None, alpha=0, normalized=True)
    assert mat.compression_ratio() > 8 and mat.n_levels > 50
    widths = np.diff(mat.level_off.numpy())
    assert int((widths > 64).sum()) >= 50
    plan = mat.walk_plan(w.d)
    assert plan is not None and plan["cut"] == 0 and plan["n_bins"] > 1000      # "auto" takes the subtree walk
    assert mat.stream_plan(w.d) is not None                  # and, before it, the one-launch multiply by subtrees
    rp, col = _csr(w.edge_index, w.n)
    m = mat.col_multiplier.numpy()
    x = w.features(0)
    xd = x.cuda()
    print("[gpu-case] c6 full size, multiply", flush=True); sys.stdout.flush()
    got = _mul(mat, xd)
    rows = np.sort(np.random.default_rng(5).choice(w.n, size=1024, replace=False))
    rows_d = torch.from_numpy(rows).cuda()
    _assert_rows_close(got[rows_d].cpu().numpy().astype(np.float64), _rows_fp64(rp, col, m, x.numpy(), rows))
    val = torch.from_numpy((np.repeat(m, np.diff(rp)) * m[col]).astype(np.float32)).cuda()
    base = torch.empty_like(xd)
    csr_spmm(torch.from_numpy(rp.astype(np.int32)).cuda(), torch.from_numpy(col).cuda(), val, xd, base)
    assert float((got - base).abs().max() / base.abs().max()) <= 1e-3
    print("[gpu-case] c6 full size, SpMM + walk by subtrees", flush=True); sys.stdout.flush()
    mat.stream_multiply = "off"                              # the SpMM and the walk apart: another summation order
    one_launch, got = got, _mul(mat, xd)
    assert float((one_launch - got).abs().max() / got.abs().max()) <= 1e-5
    _assert_rows_close(got[rows_d].cpu().numpy().astype(np.float64), _rows_fp64(rp, col, m, x.numpy(), rows))
    mat.subtree_walk = "off"
    print("[gpu-case] c6 full size, level-by-level walk", flush=True); sys.stdout.flush()
    assert torch.equal(_mul(mat, xd), got)
    mat.batch_rows = 0                                       # another summation order for the short rows
    unbatched = _mul(mat, xd)
    assert float((unbatched - got).abs().max() / got.abs().max()) <= 1e-5


def test_union_of_cliques_full_size():
    """c7: 150,000 rows in 12,000 overlapping cliques (the co-authorship shape), compression ~5.8, 43 tree levels:
    1,024 rows against fp64 SciPy rows and the whole product against the GPU CSR baseline at d = 128 (SpMM + walk
    by the automatic choice) and d = 256 (the one-launch multiply by the automatic choice); the two paths against
    each other, and a depth limit of 8 levels against the same anchors."""
    if not torch.cuda.is_available():
        pytest.skip("no HIP device")
    w = graphs.workload("c7")
    print("[gpu-case] c7 full size, building", flush=True); sys.stdout.flush()
    mat = cbm_matrix(torch.from_numpy(w.edge_index), None, alpha=0, normalized=True)
    assert mat.compression_ratio() > 5 and mat.n_levels > 30
    rp, col = _csr(w.edge_index, w.n)
    m = mat.col_multiplier.numpy()
    val = torch.from_numpy((np.repeat(m, np.diff(rp)) * m[col]).astype(np.float32)).cuda()
    rp_d, col_d = torch.from_numpy(rp.astype(np.int32)).cuda(), torch.from_numpy(col).cuda()
    rows = np.sort(np.random.default_rng(7).choice(w.n, size=1024, replace=False))
    rows_d = torch.from_numpy(rows).cuda()
    shallow = cbm_matrix(torch.from_numpy(w.edge_index), None, alpha=0, normalized=True, max_levels=8)
    assert shallow.n_levels == 8 and 2 < shallow.compression_ratio() < mat.compression_ratio()
    for d, one_launch in ((128, False), (256, True)):
        print("[gpu-case] c7 full size, d", d, flush=True); sys.stdout.flush()
        x = w.features(0, d)
        xd = x.cuda()
        assert (mat.stream_plan(d) is not None) == one_launch
        got = _mul(mat, xd)
        want_rows = _rows_fp64(rp, col, m, x.numpy(), rows)
        _assert_rows_close(got[rows_d].cpu().numpy().astype(np.float64), want_rows)
        base = torch.empty_like(xd)
        csr_spmm(rp_d, col_d, val, xd, base)
        assert float((got - base).abs().max() / base.abs().max()) <= 1e-3
        mat.stream_multiply = "off" if one_launch else "on"          # the other path: another summation order
        other = _mul(mat, xd)
        mat.stream_multiply = "auto"
        assert float((other - got).abs().max() / got.abs().max()) <= 1e-5
        lim = _mul(shallow, xd)
        _assert_rows_close(lim[rows_d].cpu().numpy().astype(np.float64), want_rows)
        assert float((lim - base).abs().max() / base.abs().max()) <= 1e-3


def test_alpha_sweep_graph_same_format_for_every_alpha():
    """On the dense-community graph alpha <= 32 prunes nothing (every admissible pair clears the
    threshold by far more): the builder must return the arrays of alpha = 0 for the whole sweep."""
    if not torch.cuda.is_available():
        pytest.skip("no HIP device")
    w = graphs.workload("c5")
    ei = torch.from_numpy(w.edge_index)
    print("[gpu-case] c5 alpha 0", flush=True); sys.stdout.flush()
    ref = cbm_matrix(ei, None, alpha=0)
    for alpha in (2, 4, 8, 16, 32):
        print("[gpu-case] c5 alpha", alpha, flush=True); sys.stdout.flush()
        mat = cbm_matrix(ei, None, alpha=alpha)
        assert mat.nnz == ref.nnz and mat.n_levels == ref.n_levels
        for name in ("rowptr", "idx", "parent", "order", "level_off"):
            assert torch.equal(getattr(mat, name), getattr(ref, name)), (alpha, name)
