"""Full-size checks at the benchmark workloads, where the CPU oracle is too slow to run per test:
size-independent properties (linearity, determinism, exactness on integer features, agreement
with the plain CSR product) plus one CPU CSR product as the anchor."""
import sys

import numpy as np
import pytest
import torch

from cbm4gnn_amd import graphs
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


def test_gcn_graph_full_size_against_gpu_csr():
    """232,965 nodes, 114 M non-zeros (the GCN epoch workload), normalised, d = 128 and d = 41."""
    if not torch.cuda.is_available():
        pytest.skip("no HIP device")
    w = graphs.workload("c4")
    print("[gpu-case] c4 full size, building", flush=True); sys.stdout.flush()
    ei = torch.from_numpy(w.edge_index)
    mat = cbm_matrix(ei, None, alpha=2, normalized=True)
    m = mat.col_multiplier
    order = np.lexsort((w.edge_index[1], w.edge_index[0]))
    rp = torch.from_numpy(np.concatenate([[0], np.cumsum(np.bincount(w.edge_index[0], minlength=w.n))]).astype(np.int32)).cuda()
    col = torch.from_numpy(w.edge_index[1][order].astype(np.int32)).cuda()
    val = (m[torch.from_numpy(w.edge_index[0][order].astype(np.int64))] * m[torch.from_numpy(w.edge_index[1][order].astype(np.int64))]).cuda()
    for d in (128, 41):
        print("[gpu-case] c4 full size, d", d, flush=True); sys.stdout.flush()
        x = torch.randn((w.n, d), generator=torch.Generator().manual_seed(d)).cuda()
        want = torch.empty_like(x)
        csr_spmm(rp, col, val, x, want)
        got = _mul(mat, x)
        assert float((got - want).abs().max() / want.abs().max()) <= 1e-3
        ones = _mul(mat, torch.ones_like(x))
        # rows of D^-1/2 (A+I) D^-1/2 applied to the all-ones vector: sum_j m_i m_j over neighbours, < sqrt(deg_i) * max m
        assert float(ones.min()) > 0.0 and torch.isfinite(ones).all()
