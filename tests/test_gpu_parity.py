"""Parity of the HIP path (through the C ABI) with the CPU oracle on identical seeded inputs.

Tolerances (stated by the task this library serves): fp32 max-relative error <= 1e-4 against the
reference-style CPU CBM path, <= 1e-3 against a plain CSR / dense product; integer format arrays
and integer-feature products bit-exact."""
import ctypes as C
import sys

import numpy as np
import pytest
import torch

from cbm4gnn_amd import _lib, graphs
from cbm4gnn_amd.cbm import cbm_matrix, csr_spmm

pytestmark = pytest.mark.gpu

TOL_CBM = 1e-4
TOL_CSR = 1e-3


def say(*a):
    print("[gpu-case]", *a, flush=True)
    sys.stdout.flush()


@pytest.fixture(scope="module", autouse=True)
def _need_gpu():
    if not torch.cuda.is_available():
        pytest.skip("no HIP device")
    _lib.hip_lib()


@pytest.fixture(autouse=True)
def _copy_rule_of_large_matrices(monkeypatch):
    """The matrices of these tests are small (X of a few MB), where the Python layer asks for 96 entries per row
    before it copies X slab-major; the tests are about the kernels behind that choice, so they run under the rule
    for large matrices (24 entries per row).  ``test_small_x_is_gathered_in_place`` covers the small-X rule."""
    from cbm4gnn_amd import cbm as cbm_mod
    monkeypatch.setattr(cbm_mod, "_SMALL_X_BYTES", 0)


def groups_for(d, ld=None, workspace=False):
    """Partial sums per output element the SpMM keeps for 16-byte aligned [*, d] matrices of row
    stride ld (1 = strictly in order), with or without a workspace for the slab-major copy of X;
    the oracle reproduces that order bit for bit."""
    ld = d if ld is None else ld
    return int(_lib.hip_lib().cbm_spmm_summation_groups(d, ld, ld, C.c_void_p(256), C.c_void_p(256), int(workspace)))


def tail_for(d, ld=None, workspace=False):
    """Trailing columns that the SpMM sums in 16 partial sums (the 64-byte half slab of the copy)."""
    ld = d if ld is None else ld
    return int(_lib.hip_lib().cbm_spmm_tail_columns(d, ld, ld, C.c_void_p(256), C.c_void_p(256), int(workspace)))


def grouped_spmm(orc, rp, col, val, xs, groups, tail=0, threads=1, seq_upto=0):
    """``orc.csr_spmm`` in ``groups`` interleaved partial sums, the last ``tail`` columns in 16; rows of at
    most ``seq_upto`` entries strictly in order where the others are not (the slab kernel sums such rows a
    batch at a time, every lane group a row of its own: ``cbm_schedule_rows_batched``)."""
    y = orc.csr_spmm(rp, col, val, xs, threads=threads, groups=groups)
    if tail and groups != 16:
        y[:, xs.shape[1] - tail:] = orc.csr_spmm(rp, col, val, xs, threads=threads, groups=16)[:, xs.shape[1] - tail:]
    if seq_upto and groups > 1:
        short = np.diff(np.asarray(rp, np.int64)) <= seq_upto
        y[short] = orc.csr_spmm(rp, col, val, xs, threads=threads, groups=1)[short]
    return y


def brings_workspace(relayout, nnz, n, d, ld=None):
    """The Python layer's rule: a workspace when rows average >= 24 entries (>= 96 while all of X is at most
    ``_SMALL_X_BYTES``), or when the width would otherwise run one wavefront per row."""
    from cbm4gnn_amd import cbm as cbm_mod
    need = cbm_mod._MIN_ENTRIES_PER_ROW_SMALL_X if 4 * n * d <= cbm_mod._SMALL_X_BYTES else cbm_mod._MIN_ENTRIES_PER_ROW_FOR_RELAYOUT
    return bool(relayout) and n > 0 and (nnz >= need * n or groups_for(d, ld) == 1)


def takes_stream(mat, d):
    """Whether ``*_spmm_update`` of width ``d`` runs as the one-launch multiply by subtrees (the Python layer's
    rule: after the single launch of small products, for matrices that are neither tiled nor have cut rows)."""
    if mat.is_tiled() or mat.has_cut_rows() or mat._single_launch(mat.num_rows, d):
        return False
    return mat.stream_plan(d) is not None


def mat_groups(mat, d, ld=None, update=False):
    """The same for a multiply through ``cbm_matrix``, which brings a workspace when rows are long enough.
    ``update``: the whole product (``*_spmm_update``), which for small products on shallow, sparse trees is
    one launch that sums every row strictly in order."""
    n = mat.num_rows
    if update and not mat.is_tiled() and not mat.has_cut_rows() and mat._single_launch(n, d):
        return 1
    if update and takes_stream(mat, d):                     # every row strictly in entry order
        return 1
    return groups_for(d, ld, workspace=brings_workspace(mat.relayout, mat.nnz, n, d, ld))


def mat_tail(mat, d, ld=None, update=False):
    if update and not mat.is_tiled() and not mat.has_cut_rows() and mat._single_launch(mat.num_rows, d):
        return 0
    if update and takes_stream(mat, d):
        return 0
    return tail_for(d, ld, workspace=brings_workspace(mat.relayout, mat.nnz, mat.num_rows, d, ld))


def oracle_product(orc, mat, ei, n, x, normalized, threads=4, groups=None, prescaled=None):
    """Reference-style CPU multiply on the PRODUCT's tree (so both sides sum in the same order).
    ``prescaled``: the arithmetic of a normalised multiply that copies X slab-major -- row c of
    the copy is fl(m[c] * x[c]) and the delta entries are +-1 -- instead of the reference's
    fma(+-m[c], x[c], acc); by default whichever the multiply through ``cbm_matrix`` uses."""
    col, sign = mat.columns()
    m = orc.col_multiplier(ei, n) if normalized else None
    if groups is None and prescaled is None and mat.relayout and (mat.is_tiled() or mat.has_cut_rows()):
        z = oracle_delta_spmm(orc, mat, ei, n, x, normalized)
        return (orc.update_fused(mat.mst_row.numpy(), mat.mst_col.numpy(), m, z, threads) if normalized
                else orc.update_plain(mat.mst_row.numpy(), mat.mst_col.numpy(), z, threads))
    g = mat_groups(mat, x.shape[1], update=True) if groups is None else groups
    tail = mat_tail(mat, x.shape[1], update=True) if groups is None else 0
    if prescaled is None:                                  # the copy is only made for the slab kernel (g > 1)
        prescaled = (normalized and brings_workspace(mat.relayout, mat.nnz, n, x.shape[1])
                     and mat_groups(mat, x.shape[1], update=True) > 1)
    if prescaled:
        xs = (m[:, None] * x).astype(np.float32)
        z = grouped_spmm(orc, mat.rowptr.numpy(), col.numpy().astype(np.int32), sign.numpy().astype(np.float32), xs, g, tail,
                         threads, seq_upto=mat.batch_rows)
        return orc.update_fused(mat.mst_row.numpy(), mat.mst_col.numpy(), m, z, threads)
    val = sign.numpy() * (m[col.numpy()] if normalized else np.float32(1))
    z = grouped_spmm(orc, mat.rowptr.numpy(), col.numpy().astype(np.int32), val.astype(np.float32), x, g, tail, threads,
                     seq_upto=mat.batch_rows)
    return (orc.update_plain(mat.mst_row.numpy(), mat.mst_col.numpy(), z, threads) if m is None
            else orc.update_fused(mat.mst_row.numpy(), mat.mst_col.numpy(), m, z, threads))


def tiled_split(mat):
    """Per delta entry: does it lie in a (256-row panel, 1024-column tile) block that holds at least
    ``tile_min_block_entries`` entries -- the definition of the local part of the tiled multiply."""
    n = mat.num_rows
    rp = mat.rowptr.numpy().astype(np.int64)
    row = np.repeat(np.arange(n), np.diff(rp))
    col = (mat.idx.numpy().view(np.uint32) & 0x7FFFFFFF).astype(np.int64)
    n_tiles = (n + mat.tile_rows - 1) // mat.tile_rows
    key = (row // 256) * n_tiles + col // mat.tile_rows
    return np.bincount(key)[key] >= mat.tile_min_block_entries, row


def grouped_with_cuts(orc, rp, col, sgn, xs, chunk, groups=8, tail=0, col_blocks=1):
    """CSR product in ``groups`` interleaved partial sums per row, where a row is cut into pieces --
    where its columns pass from one block of ceil(n / col_blocks) columns to the next (col_blocks >= 2)
    and, within such a run, every ``chunk`` entries (chunk = 0: never): each piece of a row with at
    least two of them is summed like a row of its own and the piece sums are then added one after the
    other, starting from zero -- the order of ``cbm_schedule_rows_blocks`` + ``combine_pieces``."""
    rp = np.asarray(rp, np.int64)
    n = rp.shape[0] - 1
    block_cols = (n + col_blocks - 1) // col_blocks if col_blocks >= 2 else 0
    lens = np.diff(rp)
    candidates = np.arange(n) if block_cols else (np.nonzero(lens > chunk)[0] if chunk else np.empty(0, np.int64))
    starts, ends, owner, long_rows = [], [], [], []
    for r in candidates:
        pieces, k, e = [], int(rp[r]), int(rp[r + 1])
        while k < e:
            run_end = e
            if block_cols:
                run_end = k + int(np.searchsorted(col[k:e], (col[k] // block_cols + 1) * block_cols, side="left"))
            step = chunk if chunk else run_end - k
            pieces += [(q, min(q + step, run_end)) for q in range(k, run_end, step)]
            k = run_end
        if len(pieces) >= 2:
            long_rows.append(r)
            for a, b in pieces:
                starts.append(a); ends.append(b); owner.append(r)
    if not long_rows:
        return grouped_spmm(orc, rp.astype(np.int32), col, sgn, xs, groups, tail)
    long_rows = np.array(long_rows)
    is_long = np.zeros(n, bool); is_long[long_rows] = True
    # auxiliary matrix: the original rows (cut rows emptied) followed by one row per piece
    keep = ~np.repeat(is_long, lens)
    piece_idx = np.concatenate([np.arange(a, b) for a, b in zip(starts, ends)])
    aux_col = np.concatenate([col[keep], col[piece_idx]])
    aux_sgn = np.concatenate([sgn[keep], sgn[piece_idx]])
    aux_len = np.concatenate([np.where(is_long, 0, lens), np.array(ends) - np.array(starts)])
    aux_rp = np.concatenate([[0], np.cumsum(aux_len)]).astype(np.int32)
    y = grouped_spmm(orc, aux_rp, aux_col.astype(np.int32), aux_sgn.astype(np.float32), xs, groups, tail)
    z = y[:n].copy()
    owner = np.array(owner)
    first = np.concatenate([[0], np.flatnonzero(owner[1:] != owner[:-1]) + 1, [owner.shape[0]]])
    for a, b in zip(first[:-1], first[1:]):                # pieces of a row are consecutive, in column order
        acc = np.zeros(xs.shape[1], np.float32)
        for p in range(a, b):
            acc = (acc + y[n + p]).astype(np.float32)
        z[owner[a]] = acc
    return z


def oracle_delta_spmm(orc, mat, ei, n, x, normalized):
    """The delta SpMM alone, Z = Delta diag(m) X, in the arithmetic and order of the multiply
    through ``cbm_matrix`` (see ``oracle_product``)."""
    col, sign = mat.columns()
    d = x.shape[1]
    g = mat_groups(mat, d)
    tail = mat_tail(mat, d)
    plan_tail = tail_for(d, workspace=True)               # the plan-based multiply always copies
    plan_groups = groups_for(d, workspace=True)
    if mat.relayout and not mat.is_tiled() and mat.has_cut_rows():
        # long rows cut into pieces; the plan-based multiply always gathers from the (scaled) copy
        xs = (orc.col_multiplier(ei, n)[:, None] * x).astype(np.float32) if normalized else x
        return grouped_with_cuts(orc, mat.rowptr.numpy(), col.numpy().astype(np.int32), sign.numpy().astype(np.float32), xs,
                                 int(mat.split_chunk or 0), plan_groups, plan_tail, mat._host_tiling()["col_blocks"])
    if mat.relayout and mat.is_tiled():
        # tiled multiply: (remote entries) + (local entries in storage order, one after the other), on the
        # copy of X scaled by m.  Remote entries: when no row is cut, the kernel of the local part gathers
        # them itself, one after the other in column order; otherwise (or with that fusion switched off)
        # the slab kernel sums them in 8 interleaved partial sums (16 in the half slab), pieces in order.
        local, row = tiled_split(mat)
        xs = (orc.col_multiplier(ei, n)[:, None] * x).astype(np.float32) if normalized else x
        c, sg = col.numpy(), sign.numpy().astype(np.float32)
        rp = np.concatenate([[0], np.cumsum(np.bincount(row[~local], minlength=n))]).astype(np.int32)
        if TILED_FUSED and not mat.has_cut_rows():
            remote = orc.csr_spmm(rp, c[~local].astype(np.int32), sg[~local], xs, groups=1)
        else:
            remote = grouped_with_cuts(orc, rp, c[~local].astype(np.int32), sg[~local], xs,
                                       mat.split_chunk if mat.has_cut_rows() else 0, plan_groups, plan_tail)
        # local entries in storage order: by tile, then by class (column - row) mod 4 in the order 0, 2, 1, 3
        lr, lc, ls = row[local], c[local], sg[local]
        phase = np.array([0, 2, 1, 3])[(lc - lr) % 4]
        order = np.lexsort((lc, phase, lc // mat.tile_rows, lr))
        rp = np.concatenate([[0], np.cumsum(np.bincount(lr, minlength=n))]).astype(np.int32)
        return remote + orc.csr_spmm(rp, lc[order].astype(np.int32), ls[order], xs, groups=1)
    if not normalized:
        return grouped_spmm(orc, mat.rowptr.numpy(), col.numpy().astype(np.int32), sign.numpy().astype(np.float32), x, g, tail,
                            seq_upto=mat.batch_rows)
    m = orc.col_multiplier(ei, n)
    if brings_workspace(mat.relayout, mat.nnz, n, d) and g > 1:      # the copy of X is scaled by m
        return grouped_spmm(orc, mat.rowptr.numpy(), col.numpy().astype(np.int32), sign.numpy().astype(np.float32),
                            (m[:, None] * x).astype(np.float32), g, tail, seq_upto=mat.batch_rows)
    val = (sign.numpy() * m[col.numpy()]).astype(np.float32)
    return grouped_spmm(orc, mat.rowptr.numpy(), col.numpy().astype(np.int32), val, x, g, tail, seq_upto=mat.batch_rows)


TILED_FUSED = True            # state of cbm_set_tiled_fused (the library's default), for the oracle's order


@pytest.fixture(params=[True, False], ids=["fused", "two-launch"])
def tiled_fused(request):
    """Run a test of the tiled multiply once with the remote entries gathered by the kernel of the local
    part (default) and once with the slab kernel gathering them first."""
    global TILED_FUSED
    lib = _lib.hip_lib()
    assert lib.cbm_set_tiled_fused(int(request.param)) == 0
    TILED_FUSED = request.param
    yield request.param
    assert lib.cbm_set_tiled_fused(1) == 0
    TILED_FUSED = True


@pytest.fixture(params=["auto", "wave-per-row"])
def spmm_kernel(request):
    """Run a test once per SpMM kernel: automatic choice (slabs where the shape allows) and the
    wave-per-row kernel forced."""
    lib = _lib.hip_lib()
    assert lib.cbm_set_spmm_kernel(1 if request.param == "wave-per-row" else 0) == 0
    yield request.param
    assert lib.cbm_set_spmm_kernel(0) == 0


def gpu_product(mat, x, normalized):
    xd = torch.from_numpy(x).cuda()
    yd = torch.full_like(xd, float("nan"))                 # beta = 0: stale contents must not leak
    (mat.omp_mkl_csr_fused_spmm_update if normalized else mat.omp_mkl_csr_spmm_update)(xd, yd)
    torch.cuda.synchronize()
    return yd.cpu().numpy()


# ---------------------------------------------------------------- golden fixtures ---------
@pytest.mark.parametrize("case", range(5))
@pytest.mark.parametrize("alpha", [0, 2, 3])
def test_golden_integer_products_bit_exact(golden, case, alpha):
    ei, x = golden[f"case{case}_edge_index"], golden[f"case{case}_x"]
    say("golden", case, alpha)
    mat = cbm_matrix(torch.from_numpy(ei), None, alpha=alpha)
    got = gpu_product(mat, x, False)
    assert np.array_equal(got.astype(np.float64), golden[f"case{case}_ax"])
    matn = cbm_matrix(torch.from_numpy(ei), None, alpha=alpha, normalized=True)
    gotn = gpu_product(matn, x, True)
    np.testing.assert_allclose(gotn, golden[f"case{case}_ax_normalized"], rtol=TOL_CBM, atol=TOL_CBM)


# ---------------------------------------------------------------- oracle parity -----------
@pytest.mark.parametrize("d", [1, 3, 10, 41, 64, 100, 128, 256, 258, 512, 602, 1000, 1028, 2052])
@pytest.mark.parametrize("normalized", [False, True])
def test_widths_against_oracle(orc, d, normalized, spmm_kernel):
    n = 700
    ei = graphs.add_self_loops(graphs.sbm(n, 10, 0.3, 0.01, seed=d), n)
    mat = cbm_matrix(torch.from_numpy(ei), None, alpha=1, normalized=normalized)
    say("widths", d, normalized, spmm_kernel, "groups", mat_groups(mat, d))
    assert mat.n_levels >= 2 and (mat.idx < 0).any()
    if spmm_kernel == "auto":
        assert mat_groups(mat, d) > 1                      # every width takes the slab kernel (rows are long enough)
        # 128-byte slabs from the slab-major copy; the last d % 32 <= 16 columns as a 64-byte half slab
        # where the full slabs split evenly over the XCDs (widths up to 16: the half slab alone)
        assert groups_for(d, workspace=True) == (16 if d <= 16 else 8)
        assert tail_for(d, workspace=True) == {1: 1, 3: 3, 10: 10, 41: 9, 258: 2, 1028: 4, 2052: 4}.get(d, 0)
        # without a workspace only multiples of 32 run on slabs; 256-byte slabs (4 groups) where 8 of them fit
        assert groups_for(d) == (1 if d % 32 else (4 if d % 64 == 0 and d >= 512 else 8))
    else:
        assert mat_groups(mat, d) == 1
    x = np.random.default_rng(d).standard_normal((n, d)).astype(np.float32)
    got = gpu_product(mat, x, normalized)
    want = oracle_product(orc, mat, ei, n, x, normalized)
    assert orc.max_rel_err(got, want) <= TOL_CBM
    assert np.array_equal(got, want)                       # same order, same FMAs: in fact bit-exact
    assert orc.max_rel_err(got, oracle_product(orc, mat, ei, n, x, normalized, groups=1)) <= TOL_CBM
    assert orc.max_rel_err(got, orc.dense_product(ei, n, x, normalized)) <= TOL_CSR
    if normalized:                                         # gathering m[col] instead of streaming +-m[col]
        mat2 = cbm_matrix(torch.from_numpy(ei), None, alpha=1, normalized=True)
        mat2.stream_coefficients = False
        assert np.array_equal(gpu_product(mat2, x, True), got)
    mat.relayout = False                                   # no workspace: row-major gather / one wave per row
    got2 = gpu_product(mat, x, normalized)
    assert np.array_equal(got2, oracle_product(orc, mat, ei, n, x, normalized))
    assert orc.max_rel_err(got2, got) <= 1e-5


@pytest.mark.parametrize("name,scale,alphas", [("c1", 1.0, (0,)), ("c2", 0.5, (0, 8)), ("c3", 0.05, (0, 16))])
def test_workloads_against_oracle(orc, name, scale, alphas, spmm_kernel):
    w = graphs.workload(name, scale=scale)
    x = w.features(0).numpy()
    for alpha in alphas:
        say("workload", name, scale, alpha)
        mat = cbm_matrix(torch.from_numpy(w.edge_index), None, alpha=alpha, normalized=w.normalized)
        got = gpu_product(mat, x, w.normalized)
        # (1) the oracle's own build (its own arborescence): the reference-style CPU path end to end
        fmt = orc.build_format(w.edge_index, w.n, alpha)
        m = orc.col_multiplier(w.edge_index, w.n) if w.normalized else None
        crow, col, val = orc.deltas_csr(fmt, w.n, m)
        want = orc.spmm_update(crow, col, val, fmt["mst_row"], fmt["mst_col"], x, m, threads=4)
        assert orc.max_rel_err(got, want) <= TOL_CBM
        # (2) plain CSR A @ X on the CPU
        ei = w.edge_index
        order = np.lexsort((ei[1], ei[0]))
        rp = np.concatenate([[0], np.cumsum(np.bincount(ei[0], minlength=w.n))]).astype(np.int32)
        vals = (m[ei[0][order]] * m[ei[1][order]]).astype(np.float32) if w.normalized else None
        csr = orc.csr_spmm(rp, ei[1][order], vals, x, threads=4)
        assert orc.max_rel_err(got, csr) <= TOL_CSR
        # (3) the GPU CSR baseline computes the same thing
        yd = torch.empty((w.n, x.shape[1]), device="cuda")
        csr_spmm(torch.from_numpy(rp).cuda(), torch.from_numpy(ei[1][order].astype(np.int32)).cuda(),
                 None if vals is None else torch.from_numpy(vals).cuda(), torch.from_numpy(x).cuda(), yd)
        assert orc.max_rel_err(yd.cpu().numpy(), csr) <= 1e-5
        g = groups_for(x.shape[1], workspace=brings_workspace(True, ei.shape[1], w.n, x.shape[1]))
        assert np.array_equal(yd.cpu().numpy(), csr if g == 1 else orc.csr_spmm(rp, ei[1][order], vals, x, threads=4, groups=g))


@pytest.mark.parametrize("normalized", [False, True])
@pytest.mark.parametrize("kind", ["staircases", "sbm"])
def test_short_rows_summed_in_batches(orc, kind, normalized):
    """cbm_schedule_rows_batched + CBM_SPMM_SCHED_BATCHED: rows of at most ``batch_rows`` entries are summed by
    one lane group each, several rows per wavefront, entries strictly in order.  Against the oracle in that
    order, bit for bit, for every limit (0 = off, 8 = one chunk, 16, 64 = every row of these graphs' short
    part in up to 8 chunks), on 128-byte slabs from the copy, the 64-byte half slab (d = 41), 128- and
    256-byte slabs gathered in place (d = 64 / 512 without a copy), with streamed, sign-only and gathered
    coefficients; the CSR baseline takes the same schedules."""
    if kind == "staircases":
        ei = graphs.staircases(30, 70, 6, 2.0, seed=1)           # most delta rows hold 1 .. 6 entries
        n = int(ei.max()) + 1
    else:
        n = 700
        ei = graphs.sbm(n, 10, 0.3, 0.01, seed=5)                  # delta rows of 10 .. 40 entries
    if normalized:
        ei = graphs.add_self_loops(ei, n)
    mat = cbm_matrix(torch.from_numpy(ei), None, alpha=0 if kind == "staircases" else 1, normalized=normalized)
    mat.single_launch_max_bytes = 0
    lens = np.diff(mat.rowptr.numpy())
    assert (lens > 8).any() and ((lens <= 8).any() if kind == "staircases" else (lens <= 64).all())
    for d in (41, 64, 100, 256, 512):
        x = np.random.default_rng(d).standard_normal((n, d)).astype(np.float32)
        results = {}
        for limit in (0, 8, 16, 64):
            for relayout in (True, False):
                mat.batch_rows, mat.relayout = limit, relayout
                if not relayout and mat_groups(mat, d) == 1:
                    continue                                       # one wavefront per row: no slabs, no batches
                for stream in ((True, False) if (normalized and not relayout) else (True,)):
                    mat.stream_coefficients = stream
                    say("batched rows", kind, normalized, "d", d, "limit", limit, "copy", relayout, "stream", stream)
                    got = gpu_product(mat, x, normalized)
                    want = oracle_product(orc, mat, ei, n, x, normalized)
                    assert np.array_equal(got, want)
                    results[(limit, relayout, stream)] = got
        mat.stream_coefficients, mat.relayout = True, True
        assert not np.array_equal(results[(0, True, True)], results[(64, True, True)])      # the order does differ
        assert orc.max_rel_err(results[(64, True, True)], orc.dense_product(ei, n, x, normalized)) <= TOL_CBM
    # the CSR baseline on a batched schedule: same rule
    from cbm4gnn_amd.cbm import schedule_rows
    order = np.lexsort((ei[1], ei[0]))
    rp = np.concatenate([[0], np.cumsum(np.bincount(ei[0], minlength=n))]).astype(np.int32)
    col = ei[1][order].astype(np.int32)
    m = orc.col_multiplier(ei, n) if normalized else None
    vals = (m[ei[0][order]] * m[col]).astype(np.float32) if normalized else None
    x = np.random.default_rng(3).standard_normal((n, 96)).astype(np.float32)
    xd = torch.from_numpy(x).cuda()
    for limit in (0, 8, 64):
        sched = schedule_rows(torch.from_numpy(rp), batch=limit).cuda()
        assert sched.shape[0] == n + (1 if limit else 0)
        yd = torch.full((n, 96), float("nan"), device="cuda")
        csr_spmm(torch.from_numpy(rp).cuda(), torch.from_numpy(col).cuda(), None if vals is None else torch.from_numpy(vals).cuda(),
                 xd, yd, sched)
        g = groups_for(96, workspace=brings_workspace(True, col.shape[0], n, 96))
        assert g > 1
        assert np.array_equal(yd.cpu().numpy(), grouped_spmm(orc, rp, col, vals, x, g, seq_upto=limit))
    with pytest.raises(ValueError):
        csr_spmm(torch.from_numpy(rp).cuda(), torch.from_numpy(col).cuda(), None, xd, yd, sched[:-2])


def test_small_x_is_gathered_in_place(orc, monkeypatch):
    """While all of X is at most 8 MB the copy must repay one more dependent launch: rows then need 96 entries on
    average, not 24.  Same matrix under both rules: different kernels, each bit-exact against its order model."""
    from cbm4gnn_amd import cbm as cbm_mod
    n, d = 3000, 128
    ei = graphs.add_self_loops(graphs.sbm(n, 30, 0.4, 0.002, seed=8), n)
    mat = cbm_matrix(torch.from_numpy(ei), None, alpha=0, normalized=True)
    assert 24 * n <= mat.nnz < 96 * n
    x = np.random.default_rng(8).standard_normal((n, d)).astype(np.float32)
    xd = torch.from_numpy(x).cuda()
    results = []
    for small_bytes in (8 << 20, 0):
        monkeypatch.setattr(cbm_mod, "_SMALL_X_BYTES", small_bytes)
        say("small X rule", small_bytes)
        assert cbm_mod._wants_workspace(xd, xd, mat.nnz) == (small_bytes == 0)
        got = gpu_product(mat, x, True)
        assert np.array_equal(got, oracle_product(orc, mat, ei, n, x, True))
        results.append(got)
    assert orc.max_rel_err(results[0], results[1]) <= 1e-6 and not np.array_equal(results[0], results[1])
    assert cbm_mod._wants_workspace(torch.empty((n, 41), device="cuda"), torch.empty((n, 41), device="cuda"), mat.nnz)   # odd widths always


def test_reference_test_matmul_correctness(orc):
    # tests/test_matmul_correctness.py:30-61 restated with a seed: ER(25, 0.5), alpha=3, d=10,
    # integer features, CBM product == COO product at atol=rtol=1e-4; CPU tensors in and out
    for seed in range(4):
        ei = torch.from_numpy(graphs.erdos_renyi(25, 0.5, seed))
        feats = torch.randint(0, 10, (25, 10), generator=torch.Generator().manual_seed(seed)).float()
        vals = torch.ones(ei.size(1))
        want = torch.sparse_coo_tensor(ei.long(), vals, (25, 25)) @ feats
        say("reference test", seed)
        c = cbm_matrix(ei, vals, alpha=3)
        torch.testing.assert_close(want, c.seq_torch_csr_matmul(feats), atol=1e-4, rtol=1e-4)
        torch.testing.assert_close(want, c.omp_torch_csr_matmul(feats), atol=1e-4, rtol=1e-4)
        out = torch.empty(25, 10)
        c.omp_mkl_csr_spmm_update(feats, out)
        assert torch.equal(want, out)


# ---------------------------------------------------------------- each entry point --------
def test_update_only_entry_points(orc):
    n, d = 900, 72
    ei = graphs.add_self_loops(graphs.sbm(n, 12, 0.25, 0.01, seed=7), n)
    x = np.random.default_rng(7).standard_normal((n, d)).astype(np.float32)
    for normalized in (False, True):
        say("update-only", normalized)
        mat = cbm_matrix(torch.from_numpy(ei), None, alpha=0, normalized=normalized)
        mat.single_launch_max_bytes = 0                    # the product below is compared with SpMM + walk, step by step
        # spmm alone == Delta (diag m) X
        z = torch.empty((n, d), device="cuda")
        mat.omp_mkl_csr_spmm(torch.from_numpy(x).cuda(), z)
        m = orc.col_multiplier(ei, n) if normalized else None
        z_ref = oracle_delta_spmm(orc, mat, ei, n, x, normalized)
        assert np.array_equal(z.cpu().numpy(), z_ref)
        # update alone on that Z == the oracle's walk (plain or fused) on the same Z
        y = z.clone()
        (mat.omp_mkl_csr_fused_update if normalized else mat.omp_mkl_csr_update)(y)
        ref = z_ref.copy()
        if normalized:
            orc.update_fused(mat.mst_row.numpy(), mat.mst_col.numpy(), m, ref)
        else:
            orc.update_plain(mat.mst_row.numpy(), mat.mst_col.numpy(), ref)
        assert np.array_equal(y.cpu().numpy(), ref)
        # and spmm_update in one call agrees with the two-step result
        assert np.array_equal(gpu_product(mat, x, normalized), ref)
        # seq_/avx twins are the same code
        y2 = z.clone()
        (mat.seq_mkl_csr_fused_update if normalized else mat.omp_avx_csr_update)(y2)
        assert torch.equal(y, y2)


def test_narrow_levels_use_the_single_workgroup_kernel(orc):
    # a hand-made tree: 40 levels of 3 rows each under one root child (narrow, but not a chain)
    n, d = 121, 72
    parent = np.full(n, -1, np.int64)
    for v in range(1, n):
        parent[v] = 0 if v <= 3 else v - 3
    kids = [[] for _ in range(n + 1)]
    for v in range(n):
        kids[n if parent[v] < 0 else parent[v]].append(v)
    mst_col = torch.tensor(sum(kids, []), dtype=torch.int32)
    mst_row = torch.tensor(np.concatenate([[0], np.cumsum([len(k) for k in kids])]), dtype=torch.int32)
    from cbm import cbm_mkl_cpp as cbm_
    rng = np.random.default_rng(0)
    z = rng.standard_normal((n, d)).astype(np.float32)
    m = (rng.random(n).astype(np.float32) + 0.5)
    say("narrow levels, plain")
    y = torch.from_numpy(z.copy()).cuda()
    cbm_.omp_s_update_csr_int32(mst_row, mst_col, y)
    assert np.array_equal(y.cpu().numpy(), orc.update_plain(mst_row.numpy(), mst_col.numpy(), z.copy()))
    say("narrow levels, normalised")
    y = torch.from_numpy(z.copy()).cuda()
    cbm_.omp_s_fused_update_csr_int32(mst_row, mst_col, torch.from_numpy(m), y)
    assert np.array_equal(y.cpu().numpy(), orc.update_fused(mst_row.numpy(), mst_col.numpy(), m, z.copy()))


def test_deep_chain_uses_the_chain_kernel(orc):
    # 150-deep staircase chain: the run of single-row levels goes through the chain kernel
    # (register-carried running row, more than two 64-level stretches)
    ei = graphs.sbm_with_chain(n=1500, blocks=24, p_in=1.0, mean_deg=80.0, chain=150, base=48, seed=0)
    n = 1500
    for normalized, d in ((False, 512), (True, 96), (True, 41), (False, 10), (True, 1100)):
        e2 = graphs.add_self_loops(ei, n) if normalized else ei
        mat = cbm_matrix(torch.from_numpy(e2), None, alpha=0, normalized=normalized)
        mat.subtree_walk = mat.stream_multiply = "off"     # this test is about the level plan's chain kernel
        assert mat.n_levels >= 151
        widths = np.diff(mat.level_off.numpy())
        assert (widths[-120:] == 1).all()
        say("deep chain", normalized, d, "levels", mat.n_levels)
        x = np.random.default_rng(1).standard_normal((n, d)).astype(np.float32)
        got = gpu_product(mat, x, normalized)
        want = oracle_product(orc, mat, e2, n, x, normalized)
        assert np.array_equal(got, want)
        assert orc.max_rel_err(got, orc.dense_product(e2, n, x, normalized)) <= TOL_CSR


def test_chain_lengths_around_the_stretch_size(orc):
    # the chain kernel walks stretches of 64 levels in two halves of 32: runs of single-row levels that end
    # inside the first half, around a half's end and around a stretch's end
    n = 900
    runs = set()
    for chain in (12, 38, 39, 40, 41, 71, 72, 73, 74, 106):
        ei = graphs.sbm_with_chain(n=n, blocks=16, p_in=1.0, mean_deg=60.0, chain=chain, base=40, seed=7)
        for normalized, d in ((False, 96), (True, 41)):
            e2 = graphs.add_self_loops(ei, n) if normalized else ei
            mat = cbm_matrix(torch.from_numpy(e2), None, alpha=0, normalized=normalized)
            mat.subtree_walk = mat.stream_multiply = "off" # the level plan's chain kernel
            widths = np.diff(mat.level_off.numpy())
            run = int(np.argmax(widths[::-1] != 1)) if (widths != 1).any() else len(widths)
            runs.add(run)
            say("chain of", chain, normalized, d, "levels", mat.n_levels, "single-row run", run)
            x = np.random.default_rng(chain).standard_normal((n, d)).astype(np.float32)
            got = gpu_product(mat, x, normalized)
            want = oracle_product(orc, mat, e2, n, x, normalized)
            assert np.array_equal(got, want)
    assert {33, 64, 65} <= runs and min(runs) < 32 and max(runs) > 90, runs


def _walk_graph(kind):
    if kind == "bushy":
        n = 900
        return graphs.sbm(n, 9, 0.4, 0.01, seed=3), n
    if kind == "chain":
        n = 1500
        return graphs.sbm_with_chain(n=n, blocks=24, p_in=1.0, mean_deg=80.0, chain=150, base=48, seed=0), n
    if kind == "staircases":
        ei = graphs.staircases(30, 70, 6, 2.0, seed=1)
        return ei, int(ei.max()) + 1
    if kind == "bipartite":                                # identical rows on either side: empty delta rows
        u, v = np.meshgrid(np.arange(40), 40 + np.arange(500), indexing="ij")
        e = np.stack([u.ravel(), v.ravel()])
        return np.concatenate([e, e[::-1]], 1).astype(np.int32), 540
    n = 1200
    return graphs.duplication(n, 0.7, 3, 8, seed=2), n


@pytest.mark.parametrize("normalized", [False, True])
@pytest.mark.parametrize("kind", ["bushy", "chain", "staircases", "duplication"])
def test_subtree_walk_equals_the_level_walk_and_the_oracle(orc, kind, normalized):
    """cbm_propagate_subtrees_f32: the rows below a level walked by subtrees in one launch (a wavefront per bin
    of subtrees and 64 columns, parent values carried in a register / LDS slots).  Per row the arithmetic is
    that of the level-by-level walk, so the product must be bit-identical to it -- and to the oracle on the
    product's tree -- for every cut level, width (one to eighteen 64-column slices, ragged last slice,
    d % 8 != 0 for the division tail) and for trees that are bushy (slots in use), one long chain (bins of
    more than two stretches), many chains (deep and wide) and a duplication graph."""
    ei, n = _walk_graph(kind)
    if normalized:
        ei = graphs.add_self_loops(ei, n)
    mat = cbm_matrix(torch.from_numpy(ei), None, alpha=0, normalized=normalized)
    mat.single_launch_max_bytes = 0
    mat.path_walk_max_bytes = 0
    mat.stream_multiply = "off"                            # the SpMM and the walk apart
    assert mat.n_levels >= 3
    slots = mat._host_walk_plan(0, 64)["n_slots"]
    assert (slots >= 2) if kind in ("bushy", "duplication") else True
    mul = mat.omp_mkl_csr_fused_spmm_update if normalized else mat.omp_mkl_csr_spmm_update
    upd = mat.omp_mkl_csr_fused_update if normalized else mat.omp_mkl_csr_update
    for d in (1, 19, 64, 100, 256, 1100):
        x = np.random.default_rng(d).standard_normal((n, d)).astype(np.float32)
        xd = torch.from_numpy(x).cuda()
        mat.subtree_walk = "off"
        want = torch.full_like(xd, float("nan")); mul(xd, want)
        z = torch.empty_like(xd); mat.omp_mkl_csr_spmm(xd, z)            # the SpMM alone, for the update-only calls
        want_upd = z.clone(); upd(want_upd)
        if d in (19, 256):
            assert np.array_equal(want.cpu().numpy(), oracle_product(orc, mat, ei, n, x, normalized))
        for cut in ("on", 0, 1, mat.n_levels - 2):
            say("subtree walk", kind, normalized, "d", d, "cut", cut, "levels", mat.n_levels, "slots", slots)
            mat.subtree_walk = cut
            plan = mat.walk_plan(d)
            assert plan is not None and (cut == "on" or plan["cut"] == cut)
            got = torch.full_like(xd, float("nan")); mul(xd, got)
            assert torch.equal(got, want)
            # update-only entry point, in place on a matrix whose rows are further apart than d
            wide = torch.full((n, d + 5), 3.0, device="cuda")
            wide[:, :d] = z
            upd(wide[:, :d])
            assert torch.equal(wide[:, :d], want_upd) and bool((wide[:, d:] == 3.0).all())
        if d == 100:                                                     # the ReLU is a pass after the walk
            relu = torch.full_like(xd, float("nan"))
            mat._run_spmm_update(xd, relu, use_m=normalized, relu=True)
            assert float(want.min()) < 0 and torch.equal(relu, want.clamp_min(0.0))
    # the automatic choice follows the cost estimate; deep trees take the subtree walk
    mat.subtree_walk = "auto"
    auto = mat.walk_plan(256)
    if mat.n_levels > 16:
        assert auto is not None
    if auto is not None:
        assert mat._subtree_plan_cost_us(auto, 256) <= 0.8 * mat._level_plan_cost_us(256)


def test_subtree_walk_on_hand_made_trees(orc):
    """Trees the builder rarely produces, through the C ABI alone: a complete binary tree (a slot per level of
    the path), a random recursive tree (bushy, ~20 levels) and a caterpillar (a long spine with a leaf at
    every row: every row keeps its value for one child) -- plan from cbm_walk_plan_build, walk by
    cbm_propagate_subtrees_f32, against cbm_propagate_f32 on the same arrays and the oracle's walk."""
    from cbm4gnn_amd.cbm import tree_levels
    lib, host = _lib.hip_lib(), _lib.host_lib()
    rng = np.random.default_rng(5)
    trees = {}
    n = 2047
    trees["binary"] = np.concatenate([[-1], (np.arange(1, n) - 1) // 2])
    n = 5000
    par = np.full(n, -1, np.int64)
    par[40:] = (rng.random(n - 40) * np.arange(40, n)).astype(np.int64)          # 40 children of the root
    trees["recursive"] = par
    n = 1201
    par = np.full(n, -1, np.int64)
    par[1:601] = np.arange(0, 600)                                                # spine 0 .. 600
    par[601:] = np.arange(0, 600)                                                 # a leaf at every spine row
    trees["caterpillar"] = par
    p = lambda t: C.c_void_p(t.data_ptr())
    for name, par in trees.items():
        n = par.shape[0]
        kids = [[] for _ in range(n + 1)]
        for v in range(n):
            kids[n if par[v] < 0 else par[v]].append(v)
        mst_col = np.array(sum(kids, []), np.int32)
        mst_row = np.concatenate([[0], np.cumsum([len(k) for k in kids])]).astype(np.int32)
        parent, order, level_off = (torch.from_numpy(a) for a in tree_levels(mst_row, mst_col))
        levels = level_off.numel() - 1
        m = (rng.random(n).astype(np.float32) + 0.5)
        for d, norm in ((72, True), (130, False)):
            z = rng.standard_normal((n, d)).astype(np.float32)
            want = (orc.update_fused(mst_row, mst_col, m, z.copy()) if norm else orc.update_plain(mst_row, mst_col, z.copy()))
            md = torch.from_numpy(m).cuda() if norm else None
            dev = [t.cuda() for t in (parent, order, level_off)]
            flags = _lib.CBM_PROP_SCALE_ROOTS if norm else 0
            y0 = torch.from_numpy(z).cuda()
            assert lib.cbm_propagate_f32(p(dev[0]), p(dev[1]), p(dev[2]), p(level_off), levels, p(md) if norm else None, p(y0),
                                         n, d, d, flags, None) == 0
            assert np.array_equal(y0.cpu().numpy(), want)
            for cut in (0, 2):
                plan = _lib.CbmWalkPlan()
                assert host.cbm_walk_plan_build(p(parent), p(order), p(level_off), n, levels, cut, 64, C.byref(plan)) == 0
                say("hand-made tree", name, "d", d, norm, "cut", cut, "levels", levels, "slots", plan.n_slots, "bins", plan.n_bins)
                if name == "binary":
                    assert plan.n_slots >= levels - 2 - cut
                ent = torch.from_numpy(np.ctypeslib.as_array(plan.entries, shape=(2 * plan.n_entries,)).copy()).cuda()
                off = torch.from_numpy(np.ctypeslib.as_array(plan.bin_off, shape=(plan.n_bins + 1,)).copy()).cuda()
                w = _lib.CbmWalkDev(plan.cut, plan.n_entries, plan.n_bins, plan.n_slots, ent.data_ptr(), off.data_ptr())
                host.cbm_walk_plan_free(C.byref(plan))
                y = torch.from_numpy(z).cuda()
                assert lib.cbm_propagate_subtrees_f32(C.byref(w), p(dev[0]), p(dev[1]), p(dev[2]), p(level_off), levels,
                                                      p(md) if norm else None, p(y), n, d, d, flags, None) == 0
                assert torch.equal(y, y0), (name, d, norm, cut)


def test_subtree_walk_status_codes():
    lib = _lib.hip_lib()
    ei = graphs.add_self_loops(graphs.staircases(8, 20, 6, 2.0, seed=4))
    mat = cbm_matrix(torch.from_numpy(ei), None, alpha=0, normalized=True)
    n, d = mat.num_rows, 64
    y = torch.zeros((n, d), device="cuda")
    st = mat._device_arrays(y.device)
    plan = mat._host_walk_plan(0, d)
    good = mat._walk_struct(st, plan)
    p = lambda t: C.c_void_p(t.data_ptr())
    call = lambda w, flags=0, levels=mat.n_levels: lib.cbm_propagate_subtrees_f32(
        C.byref(w) if w is not None else None, p(st["parent"]), p(st["order"]), p(st["level_off"]), p(mat.level_off), levels,
        p(st["m"]), p(y), n, d, d, flags, None)
    say("subtree walk status codes")
    assert call(good) == 0
    assert call(None) == _lib.CBM_ERR_NULL
    assert call(good, flags=64) == 6                                     # unknown flag
    bad = _lib.CbmWalkDev(mat.n_levels, good.n_entries, good.n_bins, good.n_slots, good.entries, good.bin_off)
    assert call(bad) == _lib.CBM_ERR_SHAPE                               # cut beyond the last level
    bad = _lib.CbmWalkDev(0, good.n_entries, good.n_bins, 40, good.entries, good.bin_off)
    assert call(bad) == _lib.CBM_ERR_SHAPE                               # more slots than a wavefront has
    bad = _lib.CbmWalkDev(0, good.n_entries, good.n_bins, good.n_slots, None, good.bin_off)
    assert call(bad) == _lib.CBM_ERR_NULL
    torch.cuda.synchronize()


@pytest.mark.parametrize("normalized", [False, True])
@pytest.mark.parametrize("kind", ["staircases", "bushy", "chain", "duplication", "bipartite"])
def test_stream_multiply_against_oracle(orc, kind, normalized):
    """cbm_spmm_update_subtrees_f32: the whole multiply in one launch, every subtree walked depth-first and every
    row's delta entries summed on the way, strictly in entry order with fma(+-1 or +-m[col], x, acc) -- the
    reference's per-entry arithmetic -- then the walk step of the level-by-level walk.  Bit for bit the oracle's
    in-order product on the same tree, for widths of one to eighteen 64-column slices (ragged last slice,
    d % 8 != 0 for the division tail), trees that are deep and wide, bushy (slots in use), one long chain (a bin
    of many stretches, rows of hundreds of entries that span stretches) and rows with no delta entry at all;
    with the ReLU in the store; on matrices whose rows are further apart than d."""
    ei, n = _walk_graph(kind)
    if normalized:
        ei = graphs.add_self_loops(ei, n)
    mat = cbm_matrix(torch.from_numpy(ei), None, alpha=0, normalized=normalized)
    mat.single_launch_max_bytes = 0
    mat.stream_multiply = "on"
    assert mat.n_levels >= 2
    plan = mat.stream_plan(64)
    lens = np.diff(mat.rowptr.numpy())
    if kind == "bipartite" and not normalized:
        assert int((lens == 0).sum()) >= 400
    if kind == "chain":
        assert plan["heaviest_bin"] > 2000 and int(lens.max()) > 64     # many stretches; rows that span stretches
    if kind in ("bushy", "duplication"):
        assert plan["n_slots"] >= 2
    for d in (1, 19, 41, 64, 100, 128, 258, 1100):
        say("stream multiply", kind, normalized, "d", d, "levels", mat.n_levels, "bins", plan["n_bins"], "slots", plan["n_slots"],
            "heaviest bin", plan["heaviest_bin"])
        assert takes_stream(mat, d)
        x = np.random.default_rng(d).standard_normal((n, d)).astype(np.float32)
        got = gpu_product(mat, x, normalized)
        want = oracle_product(orc, mat, ei, n, x, normalized)
        assert np.array_equal(got, want)
        assert orc.max_rel_err(got, orc.dense_product(ei, n, x, normalized)) <= TOL_CBM
        if d in (41, 128):
            xd = torch.from_numpy(x).cuda()
            relu = torch.full_like(xd, float("nan"))
            mat._run_spmm_update(xd, relu, use_m=normalized, relu=True)
            assert float(got.min()) < 0 and np.array_equal(relu.cpu().numpy(), np.maximum(got, 0.0))
            # rows of X and Y further apart than d: the columns beyond stay as they were
            wide_x = torch.full((n, d + 3), float("nan"), device="cuda"); wide_x[:, :d] = xd
            wide_y = torch.full((n, d + 7), 3.0, device="cuda")
            mat._run_spmm_update(wide_x[:, :d], wide_y[:, :d], use_m=normalized)
            assert np.array_equal(wide_y[:, :d].cpu().numpy(), got) and bool((wide_y[:, d:] == 3.0).all())
    # integer features: every summation order is exact, so the SpMM + walk path returns the same bits
    xi = np.random.default_rng(1).integers(-4, 5, size=(n, 72)).astype(np.float32)
    if not normalized:
        got = gpu_product(mat, xi, False)
        mat.stream_multiply = "off"
        assert np.array_equal(gpu_product(mat, xi, False), got)


def test_stream_multiply_on_hand_made_trees(orc):
    """Trees the builder rarely produces and delta rows no builder made, through the C ABI alone
    (cbm_walk_stream_build + cbm_spmm_update_subtrees_f32): a complete binary tree (a slot per level of the path),
    a random recursive tree and a caterpillar, rows of 0 .. 200 random signed entries -- against the oracle's
    in-order SpMM followed by its walk, bit for bit, plain and normalised."""
    from cbm4gnn_amd.cbm import tree_levels
    lib, host = _lib.hip_lib(), _lib.host_lib()
    rng = np.random.default_rng(11)
    trees = {}
    n = 2047
    trees["binary"] = np.concatenate([[-1], (np.arange(1, n) - 1) // 2])
    n = 5000
    par = np.full(n, -1, np.int64)
    par[40:] = (rng.random(n - 40) * np.arange(40, n)).astype(np.int64)
    trees["recursive"] = par
    n = 1201
    par = np.full(n, -1, np.int64)
    par[1:601] = np.arange(0, 600)
    par[601:] = np.arange(0, 600)
    trees["caterpillar"] = par
    p = lambda t: C.c_void_p(t.data_ptr())
    for name, par in trees.items():
        n = par.shape[0]
        kids = [[] for _ in range(n + 1)]
        for v in range(n):
            kids[n if par[v] < 0 else par[v]].append(v)
        mst_col = np.array(sum(kids, []), np.int32)
        mst_row = np.concatenate([[0], np.cumsum([len(k) for k in kids])]).astype(np.int32)
        parent, order, level_off = (torch.from_numpy(a) for a in tree_levels(mst_row, mst_col))
        levels = level_off.numel() - 1
        lens = rng.choice([0, 1, 2, 3, 7, 64, 70, 200], size=n, p=[.2, .2, .2, .15, .15, .04, .04, .02])
        rowptr = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
        cols = np.concatenate([np.sort(rng.choice(n, size=l, replace=False)) for l in lens]).astype(np.int32)
        sign = np.where(rng.integers(0, 2, size=cols.size) == 1, -1.0, 1.0).astype(np.float32)
        idx = (cols.astype(np.uint32) | ((sign < 0).astype(np.uint32) << 31)).astype(np.uint32)
        m = (rng.random(n).astype(np.float32) + 0.5)
        plan = _lib.CbmWalkStream()
        rp_t, idx_t = torch.from_numpy(rowptr), torch.from_numpy(idx.view(np.int32))
        assert host.cbm_walk_stream_build(p(rp_t), p(idx_t), p(parent), p(order), p(level_off), n, levels, 256, C.byref(plan)) == 0
        gidx = torch.from_numpy(np.ctypeslib.as_array(plan.gidx, shape=(plan.n_elems,)).astype(np.int32)).cuda()
        ginfo = torch.from_numpy(np.ctypeslib.as_array(plan.ginfo, shape=(2 * plan.n_elems,)).copy()).cuda()
        goff = torch.from_numpy(np.ctypeslib.as_array(plan.bin_goff, shape=(plan.n_bins + 1,)).copy()).cuda()
        ws = _lib.CbmWalkStreamDev(n, plan.n_bins, plan.n_slots, plan.n_elems, gidx.data_ptr(), ginfo.data_ptr(), goff.data_ptr())
        say("hand-made tree, stream", name, "levels", levels, "slots", plan.n_slots, "bins", plan.n_bins, "entries", plan.n_elems)
        if name == "binary":
            assert plan.n_slots >= levels - 2
        host.cbm_walk_stream_free(C.byref(plan))
        for d, norm in ((72, True), (130, False), (41, True)):
            x = rng.standard_normal((n, d)).astype(np.float32)
            val = sign * m[cols] if norm else sign
            z = orc.csr_spmm(rowptr, cols, val.astype(np.float32), x)                 # strictly in entry order
            want = orc.update_fused(mst_row, mst_col, m, z) if norm else orc.update_plain(mst_row, mst_col, z)
            xd, y = torch.from_numpy(x).cuda(), torch.full((n, d), float("nan"), device="cuda")
            md = torch.from_numpy(m).cuda() if norm else None
            assert lib.cbm_spmm_update_subtrees_f32(C.byref(ws), p(md) if norm else None, p(xd), p(y), n, d, d, d, 0, None) == 0
            assert np.array_equal(y.cpu().numpy(), want), (name, d, norm)


def test_stream_multiply_status_codes():
    lib = _lib.hip_lib()
    ei = graphs.add_self_loops(graphs.staircases(8, 20, 6, 2.0, seed=4))
    mat = cbm_matrix(torch.from_numpy(ei), None, alpha=0, normalized=True)
    mat.stream_multiply = "on"
    n, d = mat.num_rows, 64
    x = torch.randn((n, d), device="cuda")
    y = torch.zeros((n, d), device="cuda")
    st = mat._device_arrays(y.device)
    good = mat._stream_struct(st, mat.stream_plan(d))
    p = lambda t: C.c_void_p(t.data_ptr())
    call = lambda w, xx=x, flags=0, rows=n: lib.cbm_spmm_update_subtrees_f32(
        C.byref(w) if w is not None else None, p(st["m"]), p(xx), p(y), rows, d, d, d, flags, None)
    say("stream multiply status codes")
    assert call(good) == 0
    assert call(None) == _lib.CBM_ERR_NULL
    assert call(good, xx=y) == _lib.CBM_ERR_SHAPE                        # X must not be Y
    assert call(good, flags=_lib.CBM_PROP_SCALE_ROOTS) == 6              # only the ReLU flag
    assert call(good, rows=n - 1) == _lib.CBM_ERR_SHAPE                  # a plan of another matrix
    bad = _lib.CbmWalkStreamDev(n, good.n_bins, 40, good.n_elems, good.gidx, good.ginfo, good.bin_goff)
    assert call(bad) == _lib.CBM_ERR_SHAPE                               # more slots than a wavefront has
    bad = _lib.CbmWalkStreamDev(n, good.n_bins, good.n_slots, good.n_elems, None, good.ginfo, good.bin_goff)
    assert call(bad) == _lib.CBM_ERR_NULL
    torch.cuda.synchronize()


def test_strided_rows_and_cpu_staging(orc):
    n, d = 300, 48
    ei = graphs.erdos_renyi(n, 0.1, 5)
    mat = cbm_matrix(torch.from_numpy(ei), None, alpha=1)
    x = np.random.default_rng(2).standard_normal((n, d)).astype(np.float32)
    want = oracle_product(orc, mat, ei, n, x, False)
    say("strided")
    xbig = torch.zeros((n, d + 5), device="cuda"); xbig[:, :d] = torch.from_numpy(x).cuda()
    ybig = torch.full((n, d + 9), 7.0, device="cuda")
    mat.omp_mkl_csr_spmm_update(xbig[:, :d], ybig[:, :d])        # ld = d+5 / d+9, unaligned for float4
    assert np.array_equal(ybig[:, :d].cpu().numpy(), want)
    assert (ybig[:, d:] == 7.0).all()                            # nothing written beyond the d columns
    say("strided, slab kernel")                                 # d = 64 with ld = 68 / 72: float4-addressable
    d2 = 64
    x2 = np.random.default_rng(3).standard_normal((n, d2)).astype(np.float32)
    want2 = oracle_product(orc, mat, ei, n, x2, False, groups=mat_groups(mat, d2, 68))
    xbig = torch.zeros((n, 68), device="cuda"); xbig[:, :d2] = torch.from_numpy(x2).cuda()
    ybig = torch.full((n, 72), 7.0, device="cuda")
    mat.omp_mkl_csr_spmm_update(xbig[:, :d2], ybig[:, :d2])
    assert np.array_equal(ybig[:, :d2].cpu().numpy(), want2)
    assert (ybig[:, d2:] == 7.0).all()
    say("cpu staging")
    y = torch.empty(n, d)
    mat.omp_mkl_csr_spmm_update(torch.from_numpy(x), y)
    assert np.array_equal(y.numpy(), want)


def test_autograd_backward_matches_dense(orc):
    n, d = 200, 24
    und = graphs.add_self_loops(graphs.erdos_renyi(n, 0.08, 9), n)
    directed = und[:, (und[0] * 7 + und[1] * 3) % 5 != 0]          # drop ~20% of entries: not symmetric
    directed = graphs.add_self_loops(directed, n)
    for ei, normalized in ((und, True), (und, False), (directed, False), (directed, True)):
        say("autograd", ei.shape[1], normalized)
        mat = cbm_matrix(torch.from_numpy(ei), None, alpha=0, normalized=normalized)
        x = torch.randn((n, d), generator=torch.Generator().manual_seed(1)).cuda().requires_grad_(True)
        g = torch.randn((n, d), generator=torch.Generator().manual_seed(2)).cuda()
        y = mat.matmul(x)
        y.backward(g)
        a = orc.dense_adjacency(ei, n)
        if normalized:
            m = a.sum(axis=1) ** -0.5
            a = m[:, None] * a * m[None, :]
        assert orc.max_rel_err(y.detach().cpu().numpy(), a @ x.detach().cpu().numpy().astype(np.float64)) <= TOL_CSR
        assert orc.max_rel_err(x.grad.cpu().numpy(), a.T @ g.cpu().numpy().astype(np.float64)) <= TOL_CSR


def test_shim_functions_match_cbm_matrix(orc):
    from cbm import cbm_mkl_cpp as cbm_
    n, d = 120, 20
    ei_np = graphs.add_self_loops(graphs.erdos_renyi(n, 0.2, 3), n)
    ei = torch.from_numpy(ei_np)
    x = torch.randn((n, d), generator=torch.Generator().manual_seed(0))
    say("shim")
    for normalized in (False, True):
        c = cbm_matrix(ei, None, alpha=2, normalized=normalized)
        c.relayout = False                                 # the shim brings no workspace: same summation order
        want = gpu_product(c, x.numpy(), normalized)
        mul = c.col_multiplier
        data = (cbm_.from_coo_int32_t_v2_(ei[0], ei[1], torch.ones(ei.size(1)), mul, n, n, 2) if normalized
                else cbm_.from_coo_int32_t_v1_(ei[0], ei[1], torch.ones(ei.size(1)), n, n, 2))
        mst_row, mst_col, r, cidx, v = data
        assert torch.equal(mst_row, c.mst_row) and torch.equal(mst_col, c.mst_col)
        deltas = torch.sparse_coo_tensor(torch.stack((r, cidx)).long(), v, (n, n)).coalesce().to_sparse_csr()
        rb = deltas.crow_indices()[:-1].to(torch.int32); re = deltas.crow_indices()[1:].to(torch.int32)
        col = deltas.col_indices().to(torch.int32); val = deltas.values()
        y = torch.empty(n, d)
        if normalized:
            cbm_.omp_s_fused_spmm_update_csr_int32(rb, re, col, val, x, mst_row, mst_col, mul, y)
        else:
            cbm_.omp_s_spmm_update_csr_int32(rb, re, col, val, x, mst_row, mst_col, y)
        assert np.array_equal(y.numpy(), want)
        y2 = torch.empty(n, d)
        cbm_.seq_s_spmm_csr_int32(rb, re, col, val, x, y2)
        (cbm_.seq_s_fused_update_csr_int32(mst_row, mst_col, mul, y2) if normalized
         else cbm_.omp_s_update_avx_int32(mst_row, mst_col, y2))
        assert np.array_equal(y2.numpy(), want)
    with pytest.raises(RuntimeError, match="kInt32"):
        cbm_.seq_s_update_csr_int32(mst_row.long(), mst_col, y)


def test_c_abi_status_codes_on_device_calls():
    lib = _lib.hip_lib()
    n, d = 8, 4
    x = torch.zeros((n, d), device="cuda"); y = torch.zeros((n, d), device="cuda")
    rp = torch.zeros(n + 1, dtype=torch.int32, device="cuda"); idx = torch.zeros(1, dtype=torch.int32, device="cuda")
    p = lambda t: C.c_void_p(t.data_ptr())
    say("status codes")
    assert lib.cbm_spmm_f32(None, p(idx), 0, None, None, None, None, p(x), p(y), None, 0, n, d, d, d, None) == 1
    assert lib.cbm_spmm_f32(p(rp), p(idx), 0, None, None, None, None, p(x), p(y), None, 0, n, d, d - 1, d, None) == 3
    assert lib.cbm_spmm_f32(p(rp), p(idx), 0, None, p(x), None, None, p(x), p(y), None, 0, n, d, d, d, None) == 1   # coef without m
    assert lib.cbm_spmm_f32(p(rp), p(idx), 0, None, None, None, None, p(x), p(x), None, 0, n, d, d, d, None) == 3   # in place
    assert lib.cbm_spmm_f32(p(rp), p(idx), 0, None, None, None, None, p(x), p(y), None, 0, n, d, d, d, None) == 0   # empty rows -> zeros
    assert lib.cbm_spmm_f32(p(rp), p(idx), 0, None, None, None, None, p(x), p(y), None, 1, n, d, d, d, None) == 1   # WORKSPACE_READY without a workspace
    lo = (C.c_int32 * 2)(0, n - 1)                      # does not cover n rows
    par = torch.full((n,), -1, dtype=torch.int32, device="cuda"); order = torch.arange(n, dtype=torch.int32, device="cuda")
    assert lib.cbm_propagate_f32(p(par), p(order), p(rp), lo, 1, None, p(y), n, d, d, 0, None) == 3
    lo = (C.c_int32 * 2)(0, n)
    assert lib.cbm_propagate_f32(p(par), p(order), p(rp), lo, 1, None, p(y), n, d, d, 0, None) == 0
    assert lib.cbm_spmm_update_f32(p(rp), p(idx), 0, None, None, p(par), None, p(order), p(rp), lo, 1, p(x), p(x), None, n, d, d, d, 0, None) == 3
    torch.cuda.synchronize()
    assert (y == 0).all()
    # row intersections: (rowptr, col, colptr_t, row_t, after, row_nnz, n, alpha, groups, ticket, pairs, capacity, n_pairs, stream)
    i64 = torch.zeros(n + 1, dtype=torch.int64, device="cuda"); i32 = torch.zeros(n, dtype=torch.int32, device="cuda")
    tick = torch.zeros(1, dtype=torch.int32, device="cuda"); cnt = torch.zeros(1, dtype=torch.int64, device="cuda")
    ri = lambda *a: lib.cbm_row_intersections(*a)
    assert lib.cbm_row_intersections_groups() >= 8
    assert ri(None, p(i32), p(i64), p(i32), p(i64), p(i32), n, 0, 8, p(tick), None, 0, p(cnt), None) == 1
    assert ri(p(i64), p(i32), p(i64), p(i32), p(i64), p(i32), n, 0, 0, p(tick), None, 0, p(cnt), None) == 3      # no workgroups
    assert ri(p(i64), p(i32), p(i64), p(i32), p(i64), p(i32), n, 0, 8, p(tick), None, 4, p(cnt), None) == 1      # room but no buffer
    assert ri(p(i64), p(i32), p(i64), p(i32), p(i64), p(i32), 0, 0, 8, p(tick), None, 0, p(cnt), None) == 0      # nothing to do
    assert ri(p(i64), p(i32), p(i64), p(i32), p(i64), p(i32), n, 0, 8, p(tick), None, 0, p(cnt), None) == 0      # n empty rows: no pair
    torch.cuda.synchronize()
    assert int(cnt) == 0 and int(tick) >= n


@pytest.mark.parametrize("fused", [True, False])
@pytest.mark.parametrize("alpha,directed,normalized", [(2, False, True), (10_000, False, True), (2, True, True),
                                                       (2, False, False)])
def test_two_layer_gcn_forward_backward_matches_dense(orc, fused, alpha, directed, normalized):
    """The GCN epoch harness (Linear -> CBM aggregate -> ReLU -> Linear -> CBM aggregate, cross
    entropy) against the same model written with a dense normalised adjacency in torch fp64.
    ``fused``: the layer as one autograd function (Linear output gathered in place from a padded
    buffer, ReLU in the multiply's epilogue -- alpha = 10 000 gives the flat tree where it is
    the SpMM's epilogue, alpha = 2 a deeper tree where it is a pass after the walk -- and its
    gradient folded into the slab-major copy of the backward multiply); ``directed``: the backward
    multiply runs on the transposed operator; ``normalized=False``: the plain adjacency, whose
    Linear output the fused layer lets the SpMM gather in place."""
    from cbm4gnn_amd.gcn import CBMGCNLayer, CSRGCNLayer, TwoLayerGCN, build_operator, csr_operator
    n, f_in, hidden, classes = 300, 37, 128, 41
    ei_np = graphs.add_self_loops(graphs.sbm(n, 6, 0.3, 0.02, seed=11), n)
    if directed:
        keep = (np.random.default_rng(5).random(ei_np.shape[1]) > 0.3) | (ei_np[0] == ei_np[1])
        ei_np = np.ascontiguousarray(ei_np[:, keep])
    ei = torch.from_numpy(ei_np)
    say("gcn harness", fused, alpha, directed, normalized)
    op = build_operator(ei, alpha=alpha, normalized=normalized)
    assert (op.n_levels == 1) == (alpha == 10_000) and op.is_symmetric == (not directed)
    torch.manual_seed(1)
    model = TwoLayerGCN(CBMGCNLayer(f_in, hidden, op, fused=fused, relu=fused),
                        CBMGCNLayer(hidden, classes, op, fused=fused), relu_between=not fused).cuda()
    x = torch.randn((n, f_in), generator=torch.Generator().manual_seed(2)).cuda()
    y = torch.randint(0, classes, (n,), generator=torch.Generator().manual_seed(3)).cuda()
    a = torch.from_numpy(orc.dense_adjacency(np.stack([ei_np[1], ei_np[0]]), n)).double().cuda()
    m = a.sum(dim=1).pow(-0.5)
    a_hat = m[:, None] * a * m[None, :] if normalized else a
    for epoch in range(2):                                  # the second pass runs on the cached buffers
        model.zero_grad(set_to_none=True)
        xin = x.clone().requires_grad_(True)
        logits = model(xin)
        loss = torch.nn.functional.cross_entropy(logits, y)
        loss.backward()
        w1 = model.first_layer.lin.weight.detach().double().requires_grad_(True)
        w2 = model.last_layer.lin.weight.detach().double().requires_grad_(True)
        xr = x.double().requires_grad_(True)
        ref = a_hat @ ((a_hat @ (xr @ w1.t())).relu() @ w2.t())
        ref_loss = torch.nn.functional.cross_entropy(ref, y)
        ref_loss.backward()
        assert float((logits.detach().double() - ref).abs().max() / ref.abs().max()) <= TOL_CBM
        assert abs(float(loss.detach()) - float(ref_loss.detach())) <= 1e-4 * abs(float(ref_loss.detach()))
        for got, want in ((model.first_layer.lin.weight.grad, w1.grad), (model.last_layer.lin.weight.grad, w2.grad),
                          (xin.grad, xr.grad)):
            assert float((got.double() - want).abs().max() / want.abs().max()) <= 1e-3
    if fused:
        b = model.first_layer._cache
        # plain operator: the Linear output sits in a padded buffer and is gathered in place; a
        # normalised one keeps the copy (scaled by m on the way)
        assert b["h_in_place"] == (not normalized) and b["h"].stride(0) == (hidden if normalized else hidden + 32)
        assert float(b["y"].min()) == 0.0                                               # the ReLU was applied
        assert not model.last_layer._cache["h_in_place"]                                # width 41 takes the copy
    # the CSR-baseline model computes the same thing
    vals = op.col_multiplier[ei[0].long()] * op.col_multiplier[ei[1].long()] if normalized else None
    fwd = csr_operator(torch.stack([ei[1], ei[0]]), n, vals, x.device)
    bwd = fwd if not directed else csr_operator(ei, n, vals, x.device)
    torch.manual_seed(1)
    base = TwoLayerGCN(CSRGCNLayer(f_in, hidden, fwd, bwd), CSRGCNLayer(hidden, classes, fwd, bwd)).cuda()
    base_loss = torch.nn.functional.cross_entropy(base(x), y)
    assert abs(float(base_loss.detach()) - float(loss.detach())) <= 1e-5 * abs(float(loss.detach()))


def test_fused_gcn_layer_refuses_a_backward_whose_buffers_were_overwritten(orc):
    """The fused layer keeps one output buffer per layer (as the reference caches its output,
    cbm_message_passing.py:26-29): backward of a call whose output a later forward has overwritten must
    raise -- for the layer's own ReLU mask (call counter) and for the next layer's saved input (autograd
    version of the buffer) -- while the ordinary forward/backward sequence gives the dense gradient."""
    from cbm4gnn_amd.gcn import CBMGCNLayer, TwoLayerGCN, build_operator
    n, f_in, hidden, classes = 200, 19, 64, 7
    ei_np = graphs.add_self_loops(graphs.sbm(n, 4, 0.3, 0.02, seed=12), n)
    op = build_operator(torch.from_numpy(ei_np), alpha=1, normalized=True)
    torch.manual_seed(3)
    model = TwoLayerGCN(CBMGCNLayer(f_in, hidden, op, relu=True), CBMGCNLayer(hidden, classes, op), relu_between=False).cuda()
    x1 = torch.randn((n, f_in), generator=torch.Generator().manual_seed(4)).cuda()
    x2 = torch.randn((n, f_in), generator=torch.Generator().manual_seed(5)).cuda()
    say("fused gcn layer: second forward before backward")
    first = model(x1).square().sum()
    with torch.no_grad():
        model(x2)                                           # e.g. an evaluation pass in between
    with pytest.raises(RuntimeError):
        first.backward()
    # only the FIRST layer runs again: the second layer's saved input lives in the first layer's buffer
    model.zero_grad(set_to_none=True)
    second = model(x1).square().sum()
    with torch.no_grad():
        model.first_layer(x2)
    with pytest.raises(RuntimeError):
        second.backward()
    # forward -> backward, twice on different inputs: gradients of the dense fp64 model each time
    a = torch.from_numpy(orc.dense_adjacency(np.stack([ei_np[1], ei_np[0]]), n)).double().cuda()
    m = a.sum(dim=1).pow(-0.5)
    a_hat = m[:, None] * a * m[None, :]
    for x in (x1, x2):
        model.zero_grad(set_to_none=True)
        model(x).square().sum().backward()
        w1 = model.first_layer.lin.weight.detach().double().requires_grad_(True)
        w2 = model.last_layer.lin.weight.detach().double().requires_grad_(True)
        (a_hat @ ((a_hat @ (x.double() @ w1.t())).relu() @ w2.t())).square().sum().backward()
        for got, want in ((model.first_layer.lin.weight.grad, w1.grad), (model.last_layer.lin.weight.grad, w2.grad)):
            assert float((got.double() - want).abs().max() / want.abs().max()) <= 1e-3
    # the un-fused composition allocates per call and may interleave
    torch.manual_seed(3)
    loose = TwoLayerGCN(CBMGCNLayer(f_in, hidden, op, fused=False), CBMGCNLayer(hidden, classes, op, fused=False)).cuda()
    out1 = loose(x1).square().sum()
    loose(x2)
    out1.backward()
    w1 = loose.first_layer.lin.weight.detach().double().requires_grad_(True)
    w2 = loose.last_layer.lin.weight.detach().double().requires_grad_(True)
    (a_hat @ ((a_hat @ (x1.double() @ w1.t())).relu() @ w2.t())).square().sum().backward()
    assert float((loose.first_layer.lin.weight.grad.double() - w1.grad).abs().max() / w1.grad.abs().max()) <= 1e-3


def test_relu_epilogue_and_masked_copy_through_the_c_abi(orc):
    """CBM_UPDATE_RELU on a flat and on a deeper tree equals max(multiply, 0) bit for bit, for
    widths on both SpMM kernels; cbm_relayout_slabs_masked_f32 holds x where the mask is positive."""
    from cbm4gnn_amd.cbm import relayout_slabs
    n = 700
    ei = graphs.add_self_loops(graphs.sbm(n, 10, 0.3, 0.01, seed=13), n)
    for alpha in (1, 10_000):
        mat = cbm_matrix(torch.from_numpy(ei), None, alpha=alpha, normalized=True)
        for d in (41, 128, 200):
            say("relu epilogue", alpha, d)
            x = torch.randn((n, d), generator=torch.Generator().manual_seed(d)).cuda()
            want = torch.empty_like(x); mat._run_spmm_update(x, want, use_m=True)
            got = torch.full_like(x, float("nan")); mat._run_spmm_update(x, got, use_m=True, relu=True)
            assert float(want.min()) < 0.0 and torch.equal(got, want.clamp_min(0.0))
            mat.relayout = False                            # wave-per-row / row-major gather
            got2 = torch.full_like(x, float("nan")); mat._run_spmm_update(x, got2, use_m=True, relu=True)
            want2 = torch.empty_like(x); mat._run_spmm_update(x, want2, use_m=True)
            assert torch.equal(got2, want2.clamp_min(0.0))
            mat.relayout = True
            mask = torch.randn((n, d), generator=torch.Generator().manual_seed(d + 1)).cuda()
            ws = relayout_slabs(x, mask=mask)
            assert torch.equal(ws, relayout_slabs(torch.where(mask > 0, x, torch.zeros_like(x))))
            m_dev = mat._device_arrays(x.device)["m"]
            ws = relayout_slabs(x, mask=mask, scale=m_dev)
            assert torch.equal(ws, relayout_slabs(torch.where(mask > 0, x, torch.zeros_like(x)), scale=m_dev))
            via_copy = torch.empty_like(x)
            mat._run_spmm_update(torch.full_like(x, float("nan")), via_copy, use_m=True, workspace=ws, workspace_ready=True,
                                 workspace_prescaled=True)
            direct = torch.empty_like(x)
            mat._run_spmm_update(torch.where(mask > 0, x, torch.zeros_like(x)), direct, use_m=True, workspace=torch.empty_like(ws))
            assert torch.equal(via_copy, direct)


def test_path_walk_equals_the_level_by_level_walk(orc):
    """cbm_spmm_update_paths_f32 (one launch after the SpMM: every row sums down its own ancestor path)
    returns what the level-by-level walk returns, bit for bit: plain and normalised, with and without the
    ReLU, widths with a scalar tail (d mod 8 != 0), a strided destination, the deepest tree it takes;
    deeper and flat trees are handed to the level plan."""
    from cbm4gnn_amd.cbm import _ptr
    n = 900
    ei = graphs.add_self_loops(graphs.sbm(n, 6, 0.6, 0.01, seed=21), n)
    for normalized in (False, True):
        for max_levels in (None, _lib.CBM_PATH_MAX_LEVELS, 3):
            mat = cbm_matrix(torch.from_numpy(ei), None, alpha=0, normalized=normalized, max_levels=max_levels)
            say("path walk", normalized, max_levels, "levels", mat.n_levels)
            assert mat.n_levels >= 3
            for d in (10, 41, 128, 1028):
                x = torch.randn((n, d), generator=torch.Generator().manual_seed(d)).cuda()
                for relu in (False, True):
                    mat.path_walk_max_bytes = 0
                    want = torch.empty_like(x); mat._run_spmm_update(x, want, use_m=normalized, relu=relu)
                    mat.path_walk_max_bytes = 64 << 20
                    assert mat._walks_paths(n, d) == (mat.n_levels <= _lib.CBM_PATH_MAX_LEVELS)
                    got = torch.full((n, d + 8), float("nan"), device="cuda")[:, :d]
                    mat._run_spmm_update(x, got, use_m=normalized, relu=relu)
                    assert torch.equal(got, want)
            # and against the oracle, end to end
            x = np.random.default_rng(5).standard_normal((n, 64)).astype(np.float32)
            assert np.array_equal(gpu_product(mat, x, normalized), oracle_product(orc, mat, ei, n, x, normalized))
    # the C-ABI: overlapping scratch is refused, depths out of range fall back without touching the scratch
    mat = cbm_matrix(torch.from_numpy(ei), None, alpha=0, normalized=False, max_levels=4)
    st = mat._device_arrays(torch.device("cuda", 0))
    d = 64
    x = torch.randn((n, d), generator=torch.Generator().manual_seed(1)).cuda()
    y = torch.empty_like(x)
    lib = _lib.hip_lib()
    assert lib.cbm_spmm_update_paths_scratch_floats(n, d, 4) == n * d
    assert lib.cbm_spmm_update_paths_scratch_floats(n, 41, 4) == n * 44
    assert lib.cbm_spmm_update_paths_scratch_floats(n, d, 1) == 0
    assert lib.cbm_spmm_update_paths_scratch_floats(n, d, _lib.CBM_PATH_MAX_LEVELS + 1) == 0

    def call(scratch, n_levels=mat.n_levels, level_off=mat.level_off):
        return lib.cbm_spmm_update_paths_f32(
            _ptr(st["rowptr"]), _ptr(st["idx"]), mat.nnz, None, None, _ptr(st["parent"]), _ptr(st["sched"]), _ptr(st["order"]),
            _ptr(st["level_off"]), _ptr(level_off), n_levels, _ptr(x), _ptr(y), None, scratch, n, d, d, d, 0, None)
    assert call(C.c_void_p(y.data_ptr() + 64)) == _lib.CBM_ERR_SHAPE
    assert call(C.c_void_p(x.data_ptr())) == _lib.CBM_ERR_SHAPE
    assert call(None) == _lib.CBM_ERR_NULL
    scratch = torch.full((n * d,), 7.0, device="cuda")
    assert call(_ptr(scratch)) == 0
    torch.cuda.synchronize()
    want = torch.empty_like(x); mat.path_walk_max_bytes = 0; mat._run_spmm_update(x, want, use_m=False)
    assert torch.equal(y, want) and float(scratch.min()) != 7.0
    flat = cbm_matrix(torch.from_numpy(ei), None, alpha=10_000, normalized=False)
    assert flat.n_levels == 1
    fs = flat._device_arrays(torch.device("cuda", 0))
    scratch.fill_(7.0)
    rc = lib.cbm_spmm_update_paths_f32(
        _ptr(fs["rowptr"]), _ptr(fs["idx"]), flat.nnz, None, None, _ptr(fs["parent"]), _ptr(fs["sched"]), _ptr(fs["order"]),
        _ptr(fs["level_off"]), _ptr(flat.level_off), 1, _ptr(x), _ptr(y), None, _ptr(scratch), n, d, d, d, 0, None)
    torch.cuda.synchronize()
    assert rc == 0 and float(scratch.min()) == 7.0 and float(scratch.max()) == 7.0
    want = torch.empty_like(x); flat._run_spmm_update(x, want, use_m=False)
    assert torch.equal(y, want)


def test_one_launch_product_for_small_shallow_trees(orc):
    """``cbm_spmm_update_single_f32``: small products on shallow, sparse trees run as ONE launch in which
    every row gathers its own delta entries and those of its ancestors.  Bit for bit what one wavefront per
    row + the level-by-level walk return (entries in order, the reference's fma(+-m[c], x, acc)), with the
    ReLU, widths with a scalar tail, a strided destination; the policy leaves large products, deep or
    dense trees and flat trees alone; the C ABI refuses what it cannot do."""
    from cbm4gnn_amd.cbm import _ptr
    lib = _lib.hip_lib()
    n = 1200
    ei = graphs.add_self_loops(graphs.sbm(n, 40, 0.2, 0.002, seed=3), n)        # few rows find a parent
    for normalized in (False, True):
        mat = cbm_matrix(torch.from_numpy(ei), None, alpha=2, normalized=normalized)
        say("one launch", normalized, "levels", mat.n_levels, "path ratio", round(mat._path_gather_ratio(), 3))
        assert 2 <= mat.n_levels <= _lib.CBM_PATH_MAX_LEVELS and 1.0 < mat._path_gather_ratio() <= 1.5
        for d in (10, 41, 64, 200):
            assert mat._single_launch(n, d) and mat_groups(mat, d, update=True) == 1
            x = np.random.default_rng(d).standard_normal((n, d)).astype(np.float32)
            got = gpu_product(mat, x, normalized)
            assert np.array_equal(got, oracle_product(orc, mat, ei, n, x, normalized))
            assert np.array_equal(got, oracle_product(orc, mat, ei, n, x, normalized, groups=1, prescaled=False))
            assert orc.max_rel_err(got, orc.dense_product(ei, n, x, normalized)) <= TOL_CBM
            xd = torch.from_numpy(x).cuda()
            # the same through one wavefront per row + the level walk
            mat.single_launch_max_bytes = 0
            assert lib.cbm_set_spmm_kernel(1) == 0
            try:
                two = torch.empty_like(xd); mat._run_spmm_update(xd, two, use_m=normalized)
            finally:
                assert lib.cbm_set_spmm_kernel(0) == 0
                mat.single_launch_max_bytes = 4 << 20
            assert np.array_equal(two.cpu().numpy(), got)
            r = torch.full((n, d + 8), float("nan"), device="cuda")[:, :d]
            mat._run_spmm_update(xd, r, use_m=normalized, relu=True)
            assert np.array_equal(r.cpu().numpy(), np.maximum(got, 0.0))
        assert not mat._single_launch(n, 1024)              # 4.9 MB of output: the launches are no longer what costs
    flat = cbm_matrix(torch.from_numpy(ei), None, alpha=10 ** 6)
    assert flat.n_levels == 1 and not flat._single_launch(n, 64)
    dense_tree = cbm_matrix(torch.from_numpy(graphs.add_self_loops(graphs.sbm(n, 6, 0.6, 0.01, seed=21), n)), None, alpha=0,
                            max_levels=8)
    assert dense_tree._path_gather_ratio() > 1.5 and not dense_tree._single_launch(n, 64)
    # C ABI
    mat = cbm_matrix(torch.from_numpy(ei), None, alpha=2)
    st = mat._device_arrays(torch.device("cuda", 0))
    x = torch.randn((n, 64), device="cuda"); y = torch.full_like(x, 3.0)
    call = lambda xx, yy, levels=mat.n_levels, flags=0: lib.cbm_spmm_update_single_f32(
        _ptr(st["rowptr"]), _ptr(st["idx"]), None, None, _ptr(st["parent"]), levels, _ptr(xx), _ptr(yy), n, 64, 64, 64, flags, None)
    assert call(x, x) == _lib.CBM_ERR_SHAPE and call(x, y, levels=_lib.CBM_PATH_MAX_LEVELS + 1) == 6 and call(x, y, flags=64) == 6
    assert call(None, y) == _lib.CBM_ERR_NULL
    torch.cuda.synchronize()
    assert bool((y == 3.0).all())
    assert call(x, y) == 0
    want = torch.empty_like(x); mat._run_spmm_update(x, want, use_m=False)
    assert torch.equal(y, want)


def test_degenerate_shapes(orc):
    # empty rows, a single-row matrix, d = 1, more slabs than rows
    ei = np.array([[0, 1, 2, 4, 2], [0, 2, 1, 2, 4]], np.int32)      # row 3 is empty
    for d in (1, 32, 256):
        say("degenerate", d)
        x = np.random.default_rng(d).standard_normal((5, d)).astype(np.float32)
        for normalized in (False, True):
            if normalized:
                e2 = graphs.add_self_loops(ei, 5)                     # no zero degrees under normalisation
            else:
                e2 = ei
            mat = cbm_matrix(torch.from_numpy(e2), None, alpha=0, normalized=normalized)
            got = gpu_product(mat, x, normalized)
            assert orc.max_rel_err(got, orc.dense_product(e2, 5, x, normalized)) <= 1e-6
            if not normalized:
                assert (got[3] == 0).all()
    one = cbm_matrix(torch.tensor([[0], [0]], dtype=torch.int32), None, alpha=0)
    x = torch.arange(64, dtype=torch.float32).reshape(1, 64).cuda()
    y = torch.empty_like(x)
    one.omp_mkl_csr_spmm_update(x, y)
    assert torch.equal(x, y)
    with pytest.raises(ValueError):
        one.omp_mkl_csr_spmm_update(x, x)                             # in place is refused


def _oracle_levels(parent):
    """Number of tree levels from the oracle's parent array (-1 or N = child of the virtual root)."""
    parent = np.asarray(parent, np.int64)
    n = parent.shape[0]
    level = np.where((parent < 0) | (parent >= n), 0, -1)
    while (level < 0).any():
        known = (level < 0) & (level[np.clip(parent, 0, n - 1)] >= 0)
        assert known.any()
        level[known] = level[parent[known]] + 1
    return int(level.max()) + 1


def test_alpha_tuner_reports_every_alpha_and_picks_the_fastest(orc):
    """Every candidate alpha is held against the ORACLE, not only against this library's own CSR kernel
    (the reference's searcher asserts each candidate against an independent product,
    alpha_searcher/spmm_cpu_parallel.py:116-124): delta entries = the oracle builder's arborescence weight,
    candidate count and compression ratio = the oracle's, and the product the tuner timed = dense fp64."""
    from cbm4gnn_amd.tuner import tune_alpha
    w = graphs.workload("c2", scale=0.25)
    n, d = w.n, 64
    say("alpha tuner")
    x = np.random.default_rng(5).standard_normal((n, d)).astype(np.float32)
    dense = orc.dense_product(w.edge_index, n, x, True)
    best, rows = tune_alpha(w.edge_index, d, alphas=(0, 4, 10_000), normalized=True, iters=10, warmup=2,
                            x=x, reference=dense, reference_tolerance=TOL_CBM)
    assert [r["alpha"] for r in rows] == [0, 4, 10_000]
    for r in rows:
        o = orc.build_format(w.edge_index, n, r["alpha"])
        assert r["nnz_delta"] == o["nnz"] == o["msa_weight"] and r["n_candidates"] == o["n_candidates"]
        assert r["compression_ratio"] == pytest.approx(orc.compression_ratio(n, w.edge_index.shape[1], o["nnz"]))
        # equal-weight arborescences may differ in depth between two algorithms; flat is flat for both
        assert (r["tree_levels"] == 1) == (_oracle_levels(o["parent"]) == 1)
        assert r["max_rel_err_vs_reference"] is not None and r["max_rel_err_vs_reference"] <= TOL_CBM
        assert r["max_rel_err_vs_gpu_csr"] <= TOL_CSR
    assert rows[-1]["tree_levels"] == 1 and rows[-1]["compression_ratio"] < 1.0      # flat tree: delta = A
    assert rows[0]["compression_ratio"] > 1.2
    assert best in (0, 4, 10_000)
    fastest = min(r["cbm_ms"] for r in rows)
    assert next(r for r in rows if r["alpha"] == best)["cbm_ms"] <= 1.02 * fastest
    # the chosen alpha, multiplied once more outside the tuner: in the oracle's order bit for bit, dense at 1e-4
    mat = cbm_matrix(torch.from_numpy(w.edge_index), None, alpha=best, normalized=True)
    got = gpu_product(mat, x, True)
    assert np.array_equal(got, oracle_product(orc, mat, w.edge_index, n, x, True))
    assert orc.max_rel_err(got, dense) <= TOL_CBM
    # a reference that is NOT the product is refused (the check can fail)
    with pytest.raises(AssertionError):
        tune_alpha(w.edge_index, d, alphas=(10_000,), normalized=True, iters=2, warmup=1, x=x, reference=dense * 1.01)


def test_shared_slab_major_copy(orc):
    """cbm_relayout_slabs_f32 once, then two different matrices multiply the same X from it."""
    from cbm4gnn_amd.cbm import relayout_slabs
    n, d = 600, 128
    ei = graphs.add_self_loops(graphs.sbm(n, 6, 0.3, 0.01, seed=4), n)
    x = torch.randn((n, d), generator=torch.Generator().manual_seed(4)).cuda()
    say("shared relayout")
    ws = relayout_slabs(x)
    assert ws is not None and ws.numel() == n * d
    # the copy is what it says: W[s][r][:] = X[r][32 s : 32 s + 32]
    assert torch.equal(ws.view(d // 32, n, 32).permute(1, 0, 2).reshape(n, d), x)
    for alpha in (0, 1000):
        mat = cbm_matrix(torch.from_numpy(ei), None, alpha=alpha, normalized=True)
        # the plain copy: the entries carry +-m[col], as when the multiply gathers from X in place
        mat.relayout = False
        want = torch.empty_like(x); mat._run_spmm(x, want, use_m=True, scale_roots=True)
        mat.relayout = True
        got = torch.empty_like(x); mat._run_spmm(torch.zeros_like(x), got, use_m=True, scale_roots=True,
                                                 workspace=ws, workspace_ready=True)     # X itself is not read
        assert torch.equal(got, want)
        # the copy scaled by m, which is what the multiply makes for itself
        want = torch.empty_like(x); mat._run_spmm(x, want, use_m=True, scale_roots=True)
        wm = relayout_slabs(x, scale=mat._device_arrays(x.device)["m"])
        assert torch.equal(wm.view(d // 32, n, 32).permute(1, 0, 2).reshape(n, d), x * mat.col_multiplier.cuda()[:, None])
        got = torch.empty_like(x); mat._run_spmm(torch.zeros_like(x), got, use_m=True, scale_roots=True,
                                                 workspace=wm, workspace_ready=True, workspace_prescaled=True)
        assert torch.equal(got, want)
    x41 = torch.randn((n, 41), generator=torch.Generator().manual_seed(5)).cuda()
    # odd width: one full slab, then the last 9 columns zero-padded to a 64-byte half slab behind it
    w41 = relayout_slabs(x41)
    assert w41.numel() == n * 48
    assert torch.equal(w41[:n * 32].view(n, 32), x41[:, :32])
    half = w41[n * 32:].view(n, 16)
    assert torch.equal(half[:, :9], x41[:, 32:]) and float(half[:, 9:].abs().max()) == 0.0
    # 100 columns: three full slabs do not split evenly over 8 XCDs, so four zero-padded full slabs
    x100 = torch.randn((n, 100), generator=torch.Generator().manual_seed(6)).cuda()
    w100 = relayout_slabs(x100)
    assert w100.numel() == n * 128
    back = w100.view(4, n, 32).permute(1, 0, 2).reshape(n, 128)
    assert torch.equal(back[:, :100], x100) and float(back[:, 100:].abs().max()) == 0.0


def test_launch_size_does_not_change_results(orc):
    """The slab kernel is persistent: how many wavefronts it is launched with (automatic from the
    mean row length, or fixed through cbm_set_spmm_occupancy) changes which wavefront computes a
    row, never the order in which a row's entries are summed."""
    lib = _lib.hip_lib()
    n = 3000
    ei = graphs.add_self_loops(graphs.sbm(n, 3, 0.3, 0.002, seed=6), n)       # rows average ~300 entries
    mat = cbm_matrix(torch.from_numpy(ei), None, alpha=0, normalized=True)
    assert mat.nnz_a >= 256 * n
    x = torch.randn((n, 128), generator=torch.Generator().manual_seed(6)).cuda()
    say("occupancy hook")
    want = torch.empty_like(x); mat.omp_mkl_csr_fused_spmm_update(x, want)
    assert lib.cbm_set_spmm_occupancy(9) == 3 and lib.cbm_set_spmm_occupancy(-1) == 3
    try:
        for waves in (1, 3, 8):
            assert lib.cbm_set_spmm_occupancy(waves) == 0
            got = torch.full_like(x, float("nan")); mat.omp_mkl_csr_fused_spmm_update(x, got)
            assert torch.equal(got, want), waves
    finally:
        assert lib.cbm_set_spmm_occupancy(0) == 0
    ref = oracle_product(orc, mat, ei, n, x.cpu().numpy(), True)
    assert np.array_equal(want.cpu().numpy(), ref)


def test_gpu_row_intersections_build_the_same_format(monkeypatch):
    """builder="gpu": cbm_row_intersections + cbm_builder_finish give exactly the arrays of the
    all-host build, also when the first pair buffer is too small and a second pass is needed."""
    from cbm4gnn_amd import cbm as cbm_mod
    cases = [(graphs.add_self_loops(graphs.sbm(600, 6, 0.5, 0.02, seed=1), 600), 0),
             (graphs.add_self_loops(graphs.erdos_renyi(300, 0.3, 2), 300), 3),
             (graphs.workload("c2", scale=0.25).edge_index, 0),
             (graphs.workload("c1").edge_index, 0),
             (np.array([[0, 1, 2], [0, 1, 2]], np.int32), 0)]                       # self loops only: no pair at all
    for tiny_buffer in (False, True):
        if tiny_buffer:                                     # 8 pairs of room: the second, exactly sized pass runs
            monkeypatch.setattr(cbm_mod, "_first_pair_capacity", lambda nnz: 8)
        for k, (ei, alpha) in enumerate(cases):
            say("gpu builder case", k, "tiny buffer", tiny_buffer)
            a = cbm_matrix(torch.from_numpy(ei), None, alpha=alpha)
            b = cbm_matrix(torch.from_numpy(ei), None, alpha=alpha, builder="gpu")
            assert a.n_candidates == b.n_candidates and a.nnz == b.nnz
            for name in ("rowptr", "idx", "parent", "order", "level_off", "mst_row", "mst_col"):
                assert torch.equal(getattr(a, name), getattr(b, name)), (k, name)
            assert "gpu_intersections" in b.build_seconds


def test_reference_message_passing_call_pattern():
    """The way the reference's layers drive the matrix (gnns/message_passing/cbm_message_passing.py:16-60,
    tests/test_message_passing.py:53-98 restated with seeds): cbm_matrix of the TRANSPOSED int32 edge
    list with unit values, alpha = 2, built once; one cached output buffer on x's device, overwritten
    by every call; the result is the scatter-add of source features into target rows."""
    for seed in range(3):
        ei = torch.from_numpy(graphs.erdos_renyi(25, 0.75, seed)).long()
        x = torch.randint(0, 10, (25, 10), generator=torch.Generator().manual_seed(seed)).float().cuda()
        native = torch.zeros(25, 10, device="cuda").index_add_(0, ei[1].cuda(), x[ei[0].cuda()])   # out[target] += x[source]
        ei_t = torch.stack([ei[1], ei[0]], dim=0).to(torch.int32)
        say("message passing pattern", seed)
        a_t = cbm_matrix(ei_t, torch.ones(ei.size(1), dtype=x.dtype), normalized=False, alpha=2)
        out = torch.empty((int(ei.max()) + 1, x.size(1)), dtype=x.dtype, device=x.device)
        for call in (a_t.seq_mkl_csr_spmm_update, a_t.omp_mkl_csr_spmm_update):
            out.fill_(float("nan"))
            assert call(x, out) is None
            torch.testing.assert_close(out, native, atol=1e-4, rtol=1e-4)
            assert torch.equal(out, native)                  # integer features: exact
        # two hops through the same cached buffer, as stacked layers of equal width do
        a_t.omp_mkl_csr_spmm_update(x, out)
        hop2 = torch.empty_like(out)
        a_t.omp_mkl_csr_spmm_update(out, hop2)
        want2 = torch.zeros(25, 10, device="cuda").index_add_(0, ei[1].cuda(), native[ei[0].cuda()])
        assert torch.equal(hop2, want2)
        # matmul-returning variants (CBM*TorchCSR* layers)
        torch.testing.assert_close(a_t.seq_torch_csr_matmul(x), native, atol=1e-4, rtol=1e-4)
        torch.testing.assert_close(a_t.omp_torch_csr_matmul(x), native, atol=1e-4, rtol=1e-4)
        # normalised flavour: GCN weights deg^-1/2[target] * deg^-1/2[source] on the self-looped graph
        # (gnns/utility.py:25-43), fused into the matrix by normalized=True
        n = 25
        loops = torch.arange(n).repeat(2, 1)
        ei_l = torch.cat([ei[:, ei[0] != ei[1]], loops], dim=1)
        deg = torch.zeros(n).index_add_(0, ei_l[1], torch.ones(ei_l.size(1)))
        w = (deg.pow(-0.5)[ei_l[0]] * deg.pow(-0.5)[ei_l[1]]).cuda()
        native_n = torch.zeros(n, 10, device="cuda").index_add_(0, ei_l[1].cuda(), x[ei_l[0].cuda()] * w[:, None])
        a_n = cbm_matrix(torch.stack([ei_l[1], ei_l[0]]).to(torch.int32), torch.ones(ei_l.size(1)), normalized=True, alpha=2)
        out_n = torch.empty_like(out)
        for call in (a_n.seq_mkl_csr_fused_spmm_update, a_n.omp_mkl_csr_fused_spmm_update):
            out_n.fill_(float("nan"))
            call(x, out_n)
            torch.testing.assert_close(out_n, native_n, atol=1e-4, rtol=1e-4)


def test_alias_free_row_stride_needs_no_copy(orc):
    """X whose row stride is an odd number of 128-byte lines is gathered in place: the library asks
    for no workspace, and the result is bit-identical to the one through the slab-major copy."""
    lib = _lib.hip_lib()
    n, d = 700, 256
    ei = graphs.add_self_loops(graphs.sbm(n, 7, 0.3, 0.01, seed=9), n)
    mat = cbm_matrix(torch.from_numpy(ei), None, alpha=1, normalized=True)
    mat.single_launch_max_bytes = 0                        # this test is about the slab kernel's gather, not the one-launch product
    assert mat.nnz >= 24 * n
    x = torch.randn((n, d), generator=torch.Generator().manual_seed(9)).cuda()
    xp = torch.zeros((n, d + 32), device="cuda")[:, :d]
    xp.copy_(x)
    assert xp.stride(0) == 288 and xp.data_ptr() % 128 == 0
    y = torch.empty_like(x)
    p = lambda t: C.c_void_p(t.data_ptr())
    assert lib.cbm_spmm_workspace_floats(n, d, 256, 256, p(x), p(y)) == n * d
    assert lib.cbm_spmm_workspace_floats(n, d, 288, 256, p(xp), p(y)) == 0
    assert lib.cbm_spmm_workspace_floats(n, d, 320, 256, p(xp), p(y)) == n * d      # 10 lines per row: even again
    say("alias-free stride")
    want = torch.empty_like(x); mat.omp_mkl_csr_fused_spmm_update(x, want)
    got = torch.full_like(x, float("nan")); mat.omp_mkl_csr_fused_spmm_update(xp, got)
    # same summation order; the in-place gather multiplies by +-m[col] per entry, the copy is scaled by m
    assert np.array_equal(got.cpu().numpy(), oracle_product(orc, mat, ei, n, x.cpu().numpy(), True, groups=8, prescaled=False))
    assert np.array_equal(want.cpu().numpy(), oracle_product(orc, mat, ei, n, x.cpu().numpy(), True, groups=8, prescaled=True))
    assert orc.max_rel_err(got.cpu().numpy(), want.cpu().numpy()) <= 1e-6
    plain = cbm_matrix(torch.from_numpy(ei), None, alpha=1)                         # no m: bit-identical either way
    want = torch.empty_like(x); plain.omp_mkl_csr_spmm_update(x, want)
    got = torch.full_like(x, float("nan")); plain.omp_mkl_csr_spmm_update(xp, got)
    assert torch.equal(got, want)


@pytest.mark.parametrize("normalized", [False, True])
def test_depth_limited_trees_multiply_like_the_oracle(orc, normalized):
    """max_levels re-attaches deep rows to the root: a different (heavier, shallower) but valid
    format; the product is the same matrix, bit for bit against the oracle on the product's tree."""
    ei = graphs.sbm_with_chain(n=1500, blocks=24, p_in=1.0, mean_deg=80.0, chain=64, base=48, seed=0)
    n = 1500
    if normalized:
        ei = graphs.add_self_loops(ei, n)
    x = np.random.default_rng(11).standard_normal((n, 96)).astype(np.float32)
    dense = orc.dense_product(ei, n, x, normalized)
    levels = []
    for limit in (None, 8, 3, 1):
        say("depth limit", limit, normalized)
        mat = cbm_matrix(torch.from_numpy(ei), None, alpha=0, normalized=normalized, max_levels=limit)
        levels.append(mat.n_levels)
        got = gpu_product(mat, x, normalized)
        assert np.array_equal(got, oracle_product(orc, mat, ei, n, x, normalized))
        assert orc.max_rel_err(got, dense) <= TOL_CSR
    assert levels[0] > 8 and levels[1:] == [8, 3, 1]


def test_tuner_sweeps_depth_limits(orc):
    from cbm4gnn_amd.tuner import tune_alpha
    w = graphs.workload("c2", scale=0.25)
    say("tuner with depth limits")
    x = np.random.default_rng(6).standard_normal((w.n, 64)).astype(np.float32)
    dense = orc.dense_product(w.edge_index, w.n, x, True)
    best, rows = tune_alpha(w.edge_index, 64, alphas=(0, 10_000), normalized=True, iters=10, warmup=2, max_levels=(None, 3),
                            x=x, reference=dense, reference_tolerance=TOL_CBM)
    assert [(r["alpha"], r["max_levels"]) for r in rows] == [(0, None), (0, 3), (10_000, None), (10_000, 3)]
    assert rows[1]["tree_levels"] <= 3 < rows[0]["tree_levels"] and rows[1]["nnz_delta"] >= rows[0]["nnz_delta"]
    assert sum(r["best"] for r in rows) == 1 and next(r for r in rows if r["best"])["alpha"] == best
    assert all(r["max_rel_err_vs_reference"] <= TOL_CBM for r in rows)
    o = orc.build_format(w.edge_index, w.n, 0)
    assert rows[0]["nnz_delta"] == o["msa_weight"] and rows[2]["nnz_delta"] == w.edge_index.shape[1]
    # a depth-limited format is heavier than the optimum but still the same matrix: every row rebuilt from it
    limited = cbm_matrix(torch.from_numpy(w.edge_index), None, alpha=0, normalized=True, max_levels=3)
    assert limited.nnz == rows[1]["nnz_delta"]
    assert orc.check_format(w.edge_index, w.n, limited.rowptr.numpy(), limited.idx.numpy().view(np.uint32),
                            limited.mst_row.numpy(), limited.mst_col.numpy())


def test_plain_methods_on_a_normalised_matrix_apply_the_right_scaling_only(orc):
    """The reference's delta values on a ``normalized=True`` matrix are +-m[col] (cbm.py:56-66 with
    the v2 builder), so its un-fused calls (``*_spmm_update``, ``*_torch_csr_matmul``) return
    A diag(m) X, and ``*_csr_spmm`` followed by ``*_csr_update`` is the same thing in two steps.
    Oracle: SpMM with values +-m[col], then the plain walk."""
    n, d = 800, 96
    ei = graphs.add_self_loops(graphs.sbm(n, 10, 0.3, 0.01, seed=21), n)
    mat = cbm_matrix(torch.from_numpy(ei), None, alpha=1, normalized=True)
    assert mat.n_levels >= 2
    x = np.random.default_rng(21).standard_normal((n, d)).astype(np.float32)
    m = orc.col_multiplier(ei, n)
    col, sign = mat.columns()
    z = oracle_delta_spmm(orc, mat, ei, n, x, True)
    want = orc.update_plain(mat.mst_row.numpy(), mat.mst_col.numpy(), z.copy())
    a = orc.dense_adjacency(ei, n).astype(np.float64)
    dense = a @ (m.astype(np.float64)[:, None] * x.astype(np.float64))
    assert orc.max_rel_err(want, dense) <= TOL_CBM
    xd = torch.from_numpy(x).cuda()
    say("plain methods on a normalised matrix")
    for name in ("seq_mkl_csr_spmm_update", "omp_mkl_csr_spmm_update", "omp_mkl_csr_spmm_update_v2"):
        yd = torch.full_like(xd, float("nan"))
        getattr(mat, name)(xd, yd)
        assert np.array_equal(yd.cpu().numpy(), want), name
    two = torch.full_like(xd, float("nan"))
    mat.omp_mkl_csr_spmm(xd, two)
    assert np.array_equal(two.cpu().numpy(), z)
    mat.omp_mkl_csr_update(two)
    assert np.array_equal(two.cpu().numpy(), want)
    # deltas @ x (the torch route of cbm.py:255-265) + update agrees to rounding
    mixed = (mat.deltas.to(xd.device) @ xd).contiguous()
    mat.seq_mkl_csr_update(mixed)
    assert orc.max_rel_err(mixed.cpu().numpy(), want) <= 1e-5
    # the matmul-returning twins, and their gradient diag(m) A^T g
    xg = xd.clone().requires_grad_(True)
    y = mat.omp_torch_csr_matmul(xg)
    assert np.array_equal(y.detach().cpu().numpy(), want)
    g = torch.randn((n, d), generator=torch.Generator().manual_seed(3)).cuda()
    (y * g).sum().backward()
    want_g = m.astype(np.float64)[:, None] * (a.T @ g.cpu().numpy().astype(np.float64))
    assert orc.max_rel_err(xg.grad.cpu().numpy(), want_g) <= TOL_CBM
    # and the fused calls still give diag(m) A diag(m) X
    yf = torch.empty_like(xd); mat.omp_mkl_csr_fused_spmm_update(xd, yf)
    assert orc.max_rel_err(yf.cpu().numpy(), orc.dense_product(ei, n, x, True)) <= TOL_CBM


def test_changing_a_cached_setting_takes_effect():
    """``stream_coefficients`` and ``col_multiplier`` feed device arrays that are cached per device;
    changing either after a multiply must not leave the old arrays in use."""
    n, d = 500, 64
    ei = graphs.add_self_loops(graphs.sbm(n, 5, 0.3, 0.01, seed=8), n)
    mat = cbm_matrix(torch.from_numpy(ei), None, alpha=1, normalized=True)
    mat.single_launch_max_bytes = 0                        # the one-launch product gathers m[col] and never expands coef
    x = torch.randn((n, d), generator=torch.Generator().manual_seed(8)).cuda()
    say("cached settings")
    mat.relayout = False                                    # gather in place: the entries' coefficients are used
    y1 = torch.empty_like(x); mat.omp_mkl_csr_fused_spmm_update(x, y1)
    assert mat._device_arrays(x.device)["coef"] is not None
    mat.stream_coefficients = False
    y2 = torch.empty_like(x); mat.omp_mkl_csr_fused_spmm_update(x, y2)
    assert mat._device_arrays(x.device)["coef"] is None and torch.equal(y1, y2)
    mat.col_multiplier = mat.col_multiplier * 2.0           # diag(2m) A diag(2m) = 4 x the product, exactly
    y3 = torch.empty_like(x); mat.omp_mkl_csr_fused_spmm_update(x, y3)
    assert torch.equal(y3, 4.0 * y1)


@pytest.mark.parametrize("symmetric", [True, False])
def test_a_loaded_format_multiplies_like_the_built_one(tmp_path, symmetric):
    """save() -> load() -> multiply and backward: bit-equal to the freshly built matrix, including
    the depth limit and (directed graphs) the transposed operator of the backward pass."""
    n, d = 900, 72
    ei = graphs.add_self_loops(graphs.sbm(n, 9, 0.3, 0.01, seed=31), n)
    if not symmetric:                                       # drop a third of the directed edges
        keep = (np.random.default_rng(31).random(ei.shape[1]) > 0.33) | (ei[0] == ei[1])
        ei = np.ascontiguousarray(ei[:, keep])
    built = cbm_matrix(torch.from_numpy(ei), None, alpha=1, normalized=True, max_levels=3)
    assert built.is_symmetric == symmetric and 2 <= built.n_levels <= 3
    path = str(tmp_path / "fmt")
    built.save(path)
    loaded = cbm_matrix.load(path)
    assert loaded.max_levels == 3
    # the cache file keyed by the edge fingerprint: the same graph in another edge order is loaded, not rebuilt
    perm = np.random.default_rng(1).permutation(ei.shape[1])
    cached = cbm_matrix.from_cache(path, torch.from_numpy(np.ascontiguousarray(ei[:, perm])), alpha=1, normalized=True,
                                   max_levels=3)
    assert cached.builder is None and torch.equal(cached.idx, built.idx)
    say("loaded format", symmetric)
    x = torch.randn((n, d), generator=torch.Generator().manual_seed(31)).cuda()
    g = torch.randn((n, d), generator=torch.Generator().manual_seed(32)).cuda()
    out = []
    for mat in (built, loaded, cached):
        y = torch.full_like(x, float("nan")); mat.omp_mkl_csr_fused_spmm_update(x, y)
        yp = torch.full_like(x, float("nan")); mat.omp_mkl_csr_spmm_update(x, yp)
        xg = x.clone().requires_grad_(True)
        (mat.matmul(xg) * g).sum().backward()
        out.append((y, yp, xg.grad))
    for a, b, c in zip(*out):
        assert torch.isfinite(a).all() and torch.equal(a, b) and torch.equal(a, c)
    if not symmetric:
        t_built, t_loaded = built.transposed(), loaded.transposed()
        assert t_loaded.max_levels == 3
        for name in ("rowptr", "idx", "parent", "order", "level_off"):
            assert torch.equal(getattr(t_built, name), getattr(t_loaded, name)), name


def test_gpu_built_format_counts_equal_the_oracle_build(orc):
    """builder="gpu" on the 4,096-node SBM and the duplication graph at a quarter of its size: the
    number of candidate edges and the weight of the arborescence (delta non-zeros) equal those of
    the oracle's own build (its own candidate scan, its own Chu-Liu/Edmonds)."""
    for name, scale, alpha in (("c1", 1.0, 0), ("c2", 0.25, 0), ("c2", 0.25, 8)):
        w = graphs.workload(name, scale=scale)
        say("gpu build vs oracle build", name, scale, alpha)
        mat = cbm_matrix(torch.from_numpy(w.edge_index), None, alpha=alpha, builder="gpu")
        fmt = orc.build_format(w.edge_index, w.n, alpha)
        assert mat.n_candidates == fmt["n_candidates"]
        assert mat.nnz == fmt["nnz"] == int(fmt["d_row"].shape[0])
        assert orc.check_format(w.edge_index, w.n, mat.rowptr.numpy(), mat.idx.numpy().view(np.uint32),
                                mat.mst_row.numpy(), mat.mst_col.numpy())


@pytest.mark.parametrize("normalized", [False, True])
@pytest.mark.parametrize("alpha", [0, 10 ** 6])
def test_tiled_multiply_against_oracle(orc, normalized, alpha, tiled_fused):
    """``tiling="on"``: local blocks gathered from LDS tiles, the rest from the slab-major copy by the same
    kernel (in column order) or by the slab kernel first (8 interleaved partial sums).  Bit for
    bit against the oracle in the documented order -- (remote entries) + (local entries one after the
    other in storage order) -- for signed deltas (alpha = 0) and a flat tree of
    all-positive entries (alpha huge), widths on both store paths, with and without the ReLU, the
    SpMM alone, and the un-fused methods."""
    n = 3000
    ei = graphs.add_self_loops(graphs.sbm(n, 30, 0.6, 0.002, seed=5), n)
    mat = cbm_matrix(torch.from_numpy(ei), None, alpha=alpha, normalized=normalized, tiling="on")
    mat.tile_min_block_entries = 1000
    assert mat.is_tiled()
    info = mat.tiling_info
    assert info["nnz_local"] > 0 and info["nnz_remote"] > 0 and info["has_negative"] == (alpha == 0)
    assert (mat.n_levels > 2) == (alpha == 0)
    off = cbm_matrix(torch.from_numpy(ei), None, alpha=alpha, normalized=normalized, tiling="off")
    for d in (41, 128, 200):
        say("tiled", normalized, alpha, d)
        x = np.random.default_rng(d).standard_normal((n, d)).astype(np.float32)
        got = gpu_product(mat, x, normalized)
        want = oracle_product(orc, mat, ei, n, x, normalized)
        assert np.array_equal(got, want)
        assert orc.max_rel_err(got, orc.dense_product(ei, n, x, normalized)) <= TOL_CBM
        assert orc.max_rel_err(got, gpu_product(off, x, normalized)) <= 1e-5
        xd = torch.from_numpy(x).cuda()
        z = torch.full_like(xd, float("nan")); mat.omp_mkl_csr_spmm(xd, z)                  # the SpMM alone
        assert np.array_equal(z.cpu().numpy(), oracle_delta_spmm(orc, mat, ei, n, x, normalized))
        r = torch.full_like(xd, float("nan")); mat._run_spmm_update(xd, r, use_m=normalized, relu=True)
        assert np.array_equal(r.cpu().numpy(), np.maximum(want, 0.0)) and float(r.min()) == 0.0
        if normalized:                                      # un-fused: A diag(m) X
            p = torch.full_like(xd, float("nan")); mat.omp_mkl_csr_spmm_update(xd, p)
            zz = oracle_delta_spmm(orc, mat, ei, n, x, True)
            assert np.array_equal(p.cpu().numpy(), orc.update_plain(mat.mst_row.numpy(), mat.mst_col.numpy(), zz))
    # backward of matmul runs on the same path (the graph is symmetric)
    xg = torch.from_numpy(x).cuda().requires_grad_(True)
    g = torch.randn((n, 200), generator=torch.Generator().manual_seed(1)).cuda()
    (mat.matmul(xg) * g).sum().backward()
    assert orc.max_rel_err(xg.grad.cpu().numpy(), orc.dense_product(ei, n, g.cpu().numpy(), normalized)) <= TOL_CBM


def hub_graph(n, per_row, seed):
    """Directed graph with one hub ROW: row 0 is adjacent to every column; every other row has a
    self loop and ``per_row`` random columns.  (The hub is a row only: column 0 stays ordinary.)"""
    rng = np.random.default_rng(seed)
    rows = np.concatenate([np.zeros(n, np.int64), np.repeat(np.arange(1, n), per_row), np.arange(1, n)])
    cols = np.concatenate([np.arange(n), rng.integers(0, n, size=(n - 1) * per_row), np.arange(1, n)])
    ei = np.unique(np.stack([rows, cols]), axis=1)
    return np.ascontiguousarray(ei.astype(np.int32))


@pytest.mark.parametrize("normalized", [False, True])
def test_hub_row_is_cut_into_pieces(orc, normalized):
    """A 200,000-entry hub row (and a second, 5,000-entry one): the schedule cuts them into pieces
    of 2,048 entries that different wavefronts gather; the piece sums are added in order.  Bit for
    bit against the oracle in that order, for both store paths, with the ReLU, and the SpMM alone."""
    n = 200_000
    ei = hub_graph(n, 6, seed=3)
    second = np.stack([np.full(5000, 7, np.int32), np.arange(1000, 6000, dtype=np.int32)])   # row 7 gets 5,000 more
    ei = np.ascontiguousarray(np.unique(np.concatenate([ei, second], axis=1), axis=1))
    mat = cbm_matrix(torch.from_numpy(ei), None, alpha=0, normalized=normalized)
    lens = np.diff(mat.rowptr.numpy())
    assert lens.max() > 190_000 and (lens > mat.split_chunk).sum() >= 2
    assert mat.has_cut_rows() and not mat.is_tiled()
    for d in (64, 41):
        say("hub row", normalized, d)
        x = np.random.default_rng(d).standard_normal((n, d)).astype(np.float32)
        got = gpu_product(mat, x, normalized)
        want = oracle_product(orc, mat, ei, n, x, normalized)
        assert np.array_equal(got, want)
        # anchors that share no code with the oracle's SpMM: the hub row itself and a sample, in fp64
        rows = np.concatenate([[0, 7], np.random.default_rng(1).choice(n, 200, replace=False)])
        m = orc.col_multiplier(ei, n).astype(np.float64) if normalized else np.ones(n)
        order = np.lexsort((ei[1], ei[0]))
        rp = np.concatenate([[0], np.cumsum(np.bincount(ei[0], minlength=n))])
        cs = ei[1][order]
        for r in rows:
            c = cs[rp[r]:rp[r + 1]]
            ref = m[r] * (m[c][:, None] * x[c].astype(np.float64)).sum(axis=0)
            assert np.abs(got[r] - ref).max() <= TOL_CBM * max(np.abs(ref).max(), 1e-3)
        xd = torch.from_numpy(x).cuda()
        r_ = torch.full_like(xd, float("nan")); mat._run_spmm_update(xd, r_, use_m=normalized, relu=True)
        assert np.array_equal(r_.cpu().numpy(), np.maximum(want, 0.0))
        z = torch.full_like(xd, float("nan")); mat.omp_mkl_csr_spmm(xd, z)
        assert np.array_equal(z.cpu().numpy(), oracle_delta_spmm(orc, mat, ei, n, x, normalized))
    # never cut: same product to rounding, and the cut version is the faster one by far
    whole = cbm_matrix(torch.from_numpy(ei), None, alpha=0, normalized=normalized)
    whole.split_chunk = 0
    assert not whole.has_cut_rows()
    assert orc.max_rel_err(gpu_product(whole, x, normalized), got) <= 1e-5


@pytest.mark.parametrize("normalized", [False, True])
def test_rows_cut_at_column_blocks(orc, normalized):
    """``column_blocks = 3`` (with and without the chunk cut on top): every row is gathered in pieces, one
    per third of X it touches, scheduled block by block; the piece sums are added in column order.  Bit for
    bit against the oracle in that order, signed deltas and a deep tree included, both store paths, with
    the ReLU, and the SpMM alone; the automatic choice leaves a matrix of this size alone."""
    n = 3000
    ei = graphs.add_self_loops(graphs.sbm(n, 30, 0.6, 0.05, seed=17), n)
    auto = cbm_matrix(torch.from_numpy(ei), None, alpha=0, normalized=normalized, tiling="off")
    assert not auto.has_cut_rows() and auto._host_tiling() is False
    for alpha, chunk in ((0, 2048), (10 ** 6, 64)):
        mat = cbm_matrix(torch.from_numpy(ei), None, alpha=alpha, normalized=normalized, tiling="off")
        mat.column_blocks, mat.split_chunk = 3, chunk
        assert mat.has_cut_rows() and not mat.is_tiled() and mat._host_tiling()["col_blocks"] == 3
        st = mat._device_arrays(torch.device("cuda", 0))["tiled"]
        assert st["n_long"] > 0.9 * n and st["n_pieces"] >= 2 * st["n_long"]
        for d in (41, 128):
            say("column blocks", normalized, alpha, chunk, d)
            x = np.random.default_rng(d).standard_normal((n, d)).astype(np.float32)
            got = gpu_product(mat, x, normalized)
            want = oracle_product(orc, mat, ei, n, x, normalized)
            assert np.array_equal(got, want)
            assert orc.max_rel_err(got, orc.dense_product(ei, n, x, normalized)) <= TOL_CBM
            assert orc.max_rel_err(got, gpu_product(auto, x, normalized)) <= 1e-5
            xd = torch.from_numpy(x).cuda()
            z = torch.full_like(xd, float("nan")); mat.omp_mkl_csr_spmm(xd, z)
            assert np.array_equal(z.cpu().numpy(), oracle_delta_spmm(orc, mat, ei, n, x, normalized))
            r_ = torch.full_like(xd, float("nan")); mat._run_spmm_update(xd, r_, use_m=normalized, relu=True)
            assert np.array_equal(r_.cpu().numpy(), np.maximum(want, 0.0))


def test_tiled_blocks_and_cut_rows_together(orc):
    """Local blocks (a dense community among the first 2,000 nodes) and a hub row whose entries are
    mostly remote and get cut: remote pieces -> combine -> local kernel (adds, scales, ReLU)."""
    n = 20_000
    hub = hub_graph(n, 4, seed=9)
    dense = graphs.sbm(2000, 1, 0.3, 0.0, seed=9)
    ei = np.ascontiguousarray(np.unique(np.concatenate([hub, dense], axis=1), axis=1).astype(np.int32))
    for normalized in (False, True):
        mat = cbm_matrix(torch.from_numpy(ei), None, alpha=10 ** 6, normalized=normalized, tiling="on")
        mat.tile_min_block_entries = 1500
        assert mat.is_tiled() and mat.has_cut_rows()
        th = mat._host_tiling()
        assert int(np.diff(th["rowptr_r"].numpy()).max()) > 4 * mat.split_chunk and mat.tiling_info["nnz_local"] > 100_000
        for d in (96, 41):
            say("tiled + cut", normalized, d)
            x = np.random.default_rng(d).standard_normal((n, d)).astype(np.float32)
            got = gpu_product(mat, x, normalized)
            assert np.array_equal(got, oracle_product(orc, mat, ei, n, x, normalized))
            assert orc.max_rel_err(got[:3000], orc.csr_spmm(*_normalised_csr(orc, ei, n, normalized), x)[:3000]) <= TOL_CBM
            xd = torch.from_numpy(x).cuda()
            r_ = torch.full_like(xd, float("nan")); mat._run_spmm_update(xd, r_, use_m=normalized, relu=True)
            assert np.array_equal(r_.cpu().numpy(), np.maximum(got, 0.0))


def _normalised_csr(orc, ei, n, normalized):
    order = np.lexsort((ei[1], ei[0]))
    rp = np.concatenate([[0], np.cumsum(np.bincount(ei[0], minlength=n))]).astype(np.int32)
    col = ei[1][order].astype(np.int32)
    if not normalized:
        return rp, col, None
    m = orc.col_multiplier(ei, n)
    return rp, col, (m[ei[0][order]] * m[col]).astype(np.float32)


def test_status_codes_of_the_plan_based_entry_points():
    """cbm_spmm_tiled_f32 / cbm_spmm_update_tiled_f32 / the scaled and masked copies refuse bad
    arguments with a status code before anything is enqueued."""
    lib = _lib.hip_lib()
    n, d = 3000, 64
    ei = graphs.add_self_loops(graphs.sbm(n, 30, 0.6, 0.002, seed=5), n)
    mat = cbm_matrix(torch.from_numpy(ei), None, alpha=0, normalized=True, tiling="on")
    mat.tile_min_block_entries = 1000
    dev = torch.device("cuda")
    st = mat._device_arrays(dev)
    assert st["tiled"] is not None
    ts = mat._tiled_struct(st, True)
    x = torch.randn((n, d), device=dev)
    y = torch.full((n, d), 5.0, device=dev)
    ws = torch.empty(mat.workspace_floats(n, d, dev), device=dev)
    p = lambda t: C.c_void_p(t.data_ptr()) if t is not None else None
    say("plan status codes")
    call = lambda t, m, xx, yy, w, flags, nn=n, dd=d, ldx=d, ldy=d: lib.cbm_spmm_tiled_f32(
        C.byref(t) if t is not None else None, p(m), p(xx), p(yy), p(w), flags, nn, dd, ldx, ldy, None)
    m = st["m"]
    assert call(None, m, x, y, ws, 0) == 1                          # no plan
    assert call(ts, m, x, y, None, 0) == 1                          # the workspace is required
    assert call(ts, m, x, y, ws, 0, ldx=d - 1) == 3                 # stride below the width
    assert call(ts, m, x, y, ws, 0, nn=n - 300) == 3                # the plan was made for another row count
    assert call(ts, m, x, x, ws, 0) == 3                            # in place
    assert call(ts, m, x, y, x, 0) == 3                             # workspace overlaps X
    assert call(ts, m, x, y, ws, 64) == 6                           # unknown flag
    assert call(ts, m, x, y, ws, _lib.CBM_SPMM_WORKSPACE_READY) == 6         # with m, a ready copy must be the scaled one
    assert call(ts, None, x, y, ws, _lib.CBM_SPMM_WORKSPACE_READY | _lib.CBM_SPMM_WORKSPACE_PRESCALED) == 6
    assert call(ts, m, x, y, ws, _lib.CBM_SPMM_WORKSPACE_PRESCALED) == 6     # PRESCALED without READY
    bad = _lib.CbmTilingDev.from_buffer_copy(ts); bad.tile_rows = 777
    assert call(bad, m, x, y, ws, 0) == 3
    bad = _lib.CbmTilingDev.from_buffer_copy(ts); bad.n_long = 2; bad.long_rows = None
    assert call(bad, m, x, y, ws, 0) == 1
    torch.cuda.synchronize()
    assert bool((y == 5.0).all())                                   # none of the refused calls wrote anything
    assert call(ts, m, x, y, ws, 0) == 0
    lo = mat.level_off
    upd = lambda flags: lib.cbm_spmm_update_tiled_f32(C.byref(ts), p(m), p(st["parent"]), p(st["order"]), p(st["level_off"]),
                                                      p(lo), mat.n_levels, p(x), p(y), p(ws), n, d, d, d, flags, None)
    assert upd(128) == 6 and upd(0) == 0
    assert lib.cbm_spmm_update_tiled_f32(C.byref(ts), p(m), None, p(st["order"]), p(st["level_off"]), p(lo), mat.n_levels,
                                         p(x), p(y), p(ws), n, d, d, d, 0, None) == 1
    # copies
    assert lib.cbm_relayout_slabs_scaled_f32(p(x), None, p(ws), n, d, d, None) == 1
    assert lib.cbm_relayout_slabs_scaled_f32(p(x), p(m), p(x), n, d, d, None) == 3
    assert lib.cbm_relayout_slabs_masked_f32(p(x), None, p(m), p(ws), n, d, d, d, None) == 1
    assert lib.cbm_relayout_slabs_masked_f32(p(x), p(y), None, p(y), n, d, d, d, None) == 3      # copy over its own mask
    assert lib.cbm_relayout_slabs_masked_f32(p(x), p(y), None, p(ws), n, d, d, d - 1, None) == 3
    assert lib.cbm_spmm_tiled_workspace_floats(C.byref(ts), n, d) == n * d
    assert lib.cbm_spmm_tiled_workspace_floats(None, n, d) == 0
    torch.cuda.synchronize()
    # a workspace that is too small for the Python layer's own check
    with pytest.raises(ValueError, match="workspace"):
        mat._run_spmm_update(x, y, use_m=True, workspace=torch.empty(16, device=dev))
