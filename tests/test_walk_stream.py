"""Host side of the one-launch multiply by subtrees (no GPU): ``cbm_walk_stream_build`` lays the delta entries
of every row end to end in the order the walk visits the rows; a NumPy interpreter of that stream -- the
accumulator / register / slot semantics the kernel has -- must reproduce the oracle's product on the same
matrix, and the layout must keep what the kernel relies on."""
import ctypes as C

import numpy as np
import pytest
import torch

from cbm4gnn_amd import _lib, graphs
from cbm4gnn_amd.cbm import cbm_matrix

LOAD_ONLY = _lib.CBM_WALK_LOAD_ONLY
LAST, DUMMY, COL = _lib.CBM_STREAM_LAST, _lib.CBM_STREAM_DUMMY, _lib.CBM_STREAM_COL_MASK


def interpret(plan, x):
    """The plain product as one wavefront per bin computes it: ``acc`` sums a row's entries in stream order,
    ``run`` = value of the row just finished, slots = values of rows with two or more children; the rows that
    end inside a stretch of 64 entries are looked up at the head of that stretch.  float64 on integer
    features: exact."""
    gidx, ginfo, goff = plan["gidx"].numpy().view(np.uint32), plan["ginfo"].numpy(), plan["bin_goff"].numpy()
    y = np.full(x.shape, np.nan)
    written = np.zeros(x.shape[0], np.int32)
    for b in range(plan["n_bins"]):
        first, count = int(goff[b]), int(goff[b + 1] - goff[b])
        run, slots, acc = None, {}, np.zeros(x.shape[1])
        for base in range(0, count, 64):
            rs = 0
            for k in range(min(64, count - base)):
                p = int(gidx[first + base + k])
                if not p & DUMMY:
                    acc = acc + (-1.0 if p >> 31 else 1.0) * x[p & COL]
                if p & LAST:
                    row, ctl = ginfo[first + base + rs]
                    rs += 1
                    src, dst = ctl & 63, (ctl >> 8) & 63
                    run = acc if src == LOAD_ONLY else acc + (run if src == 0 else slots[src])
                    y[row] = run
                    written[row] += 1
                    if dst:
                        assert 1 <= dst <= plan["n_slots"]
                        slots[dst] = run
                    acc = np.zeros(x.shape[1])
    return y, written


def check_stream_shape(mat, plan):
    """What the layout promises: every row exactly once, its entries the row's delta entries in order (one
    stand-in for an empty row), bins padded to whole stretches of 64, heads = the children of the root, a row's
    parent is the row before it or sits in the slot named, bins hold whole subtrees, every slot of ``ginfo`` names
    a valid row."""
    gidx, ginfo, goff = plan["gidx"].numpy().view(np.uint32), plan["ginfo"].numpy(), plan["bin_goff"].numpy()
    rp, idx, parent = mat.rowptr.numpy(), mat.idx.numpy().view(np.uint32), mat.parent.numpy()
    n = mat.num_rows
    lens = np.diff(rp)
    assert plan["n_elems"] == gidx.size == ginfo.shape[0]
    assert 0 <= gidx.size - int(np.maximum(lens, 1).sum()) < 64 * plan["n_bins"]          # the padding of the bins
    assert goff[0] == 0 and goff[-1] == gidx.size and (np.diff(goff) > 0).all() and goff.size == plan["n_bins"] + 1
    assert (goff % 64 == 0).all()
    # the heaviest bin: entries + CBM_STREAM_ROW_COST per row
    rows_in = lambda b: int((gidx[goff[b]:goff[b + 1]] & LAST != 0).sum())
    real_in = lambda b: int(goff[b + 1] - goff[b]) - pad_of(b)
    def pad_of(b):
        seg = gidx[goff[b]:goff[b + 1]]
        last = int(np.flatnonzero(seg & LAST)[-1])
        return seg.size - 1 - last
    assert plan["heaviest_bin"] == max(real_in(b) + _lib.CBM_STREAM_ROW_COST * rows_in(b) for b in range(plan["n_bins"]))
    assert int((gidx & LAST != 0).sum()) == n
    assert ginfo[:, 0].min() >= 0 and ginfo[:, 0].max() < n
    seen = np.zeros(n, np.int32)
    for b in range(plan["n_bins"]):
        first, count = int(goff[b]), int(goff[b + 1] - goff[b])
        prev, slot_row, cur, first_src, last_col = None, {}, [], None, None
        for base in range(0, count, 64):
            rs = 0
            for k in range(min(64, count - base)):
                p = int(gidx[first + base + k])
                cur.append(p)
                if p & LAST:
                    row, ctl = (int(v) for v in ginfo[first + base + rs])
                    rs += 1
                    if lens[row] == 0:
                        assert cur == [row | DUMMY | LAST]
                    else:
                        want = idx[rp[row]:rp[row + 1]].tolist()
                        assert [q & ~LAST for q in cur] == want and not any(q & DUMMY for q in cur)
                        assert all(not q & LAST for q in cur[:-1])
                    src, dst = ctl & 63, (ctl >> 8) & 63
                    first_src = src if first_src is None else first_src
                    if src == LOAD_ONLY:
                        assert parent[row] < 0
                    elif src == 0:
                        assert parent[row] == prev
                    else:
                        assert slot_row[src] == parent[row]
                    if dst:
                        slot_row[dst] = row
                        assert (parent == row).sum() >= 2
                    seen[row] += 1
                    last_col = p & COL
                    prev, cur = row, []
            # the slots of this stretch that no row landed in: the bin's first row, control word 0
            for q in range(rs, min(64, count - base)):
                assert tuple(ginfo[first + base + q]) == (ginfo[first, 0], 0)
        assert cur == [last_col] * len(cur) and len(cur) < 64      # after its last row only the padding
        assert first_src == LOAD_ONLY                               # and starts with a child of the root
    assert (seen == 1).all()


def bipartite(a, b):
    """Complete bipartite graph: the rows of one side are identical, so all but one have an empty delta row."""
    u, v = np.meshgrid(np.arange(a), a + np.arange(b), indexing="ij")
    e = np.stack([u.ravel(), v.ravel()])
    return np.concatenate([e, e[::-1]], 1).astype(np.int32)


def cases():
    yield "stairs", graphs.add_self_loops(graphs.staircases(6, 30, 4, 2.0, seed=1))
    yield "stairs-clean", graphs.staircases(9, 12, 3, 0.0, seed=2)
    yield "bipartite", bipartite(5, 70)
    yield "sbm", graphs.sbm(300, 3, 0.5, 0.01, seed=3)
    yield "er", graphs.erdos_renyi(150, 0.3, 4)
    yield "dup", graphs.add_self_loops(graphs.duplication(400, seed=5))


@pytest.mark.parametrize("name,ei", list(cases()), ids=[c[0] for c in cases()])
@pytest.mark.parametrize("target_d", [64, 100_000])
def test_stream_layout_and_interpretation(orc, name, ei, target_d):
    """``target_d``: the width the bins are sized for (a huge one: the fewest, largest bins)."""
    n = int(ei.max()) + 1
    mat = cbm_matrix(torch.from_numpy(ei), None, alpha=0)
    assert mat.n_levels >= 2
    plan = mat._host_stream(target_d)
    assert plan
    check_stream_shape(mat, plan)
    if name == "bipartite":
        assert int((plan["gidx"].numpy().view(np.uint32) & DUMMY != 0).sum()) >= 60
    x = np.random.default_rng(0).integers(-8, 9, size=(n, 3)).astype(np.float64)
    y, written = interpret(plan, x)
    assert (written == 1).all()
    assert np.array_equal(y, orc.dense_product(ei, n, x.astype(np.float32), False))


def test_stream_policy():
    ei = graphs.add_self_loops(graphs.staircases(40, 60, 8, 2.0, seed=0))
    mat = cbm_matrix(torch.from_numpy(ei), None, alpha=0, normalized=True)
    assert mat.n_levels > 20
    # by estimate: short bins, many bytes at a large width; at a small one the longest bin decides
    assert mat.stream_plan(4096) is not None
    assert mat.stream_plan(8) is None
    mat.stream_multiply = "on"
    assert mat.stream_plan(8) is not None and mat.stream_plan(8)["n_elems"] >= int(np.maximum(np.diff(mat.rowptr.numpy()), 1).sum())
    mat.stream_multiply = "off"
    assert mat.stream_plan(4096) is None
    mat.stream_multiply = "sometimes"
    with pytest.raises(ValueError):
        mat.stream_plan(64)
    # a flat tree has nothing to walk; a matrix with cut rows goes through its plan-based multiply
    flat = cbm_matrix(torch.from_numpy(ei), None, alpha=1 << 30, normalized=True)
    flat.stream_multiply = "on"
    assert flat.stream_plan(256) is None
    cut = cbm_matrix(torch.from_numpy(ei), None, alpha=0, normalized=True)
    cut.stream_multiply, cut.split_chunk = "on", 64
    if cut.has_cut_rows():
        assert cut.stream_plan(256) is None


def test_stream_build_rejects_bad_input():
    ei = graphs.add_self_loops(graphs.staircases(3, 10, 3, 1.0, seed=0))
    mat = cbm_matrix(torch.from_numpy(ei), None, alpha=0)
    n = mat.num_rows
    arrays = {k: getattr(mat, k).numpy().copy() for k in ("rowptr", "idx", "parent", "order", "level_off")}

    def build(**changed):
        a = {**arrays, **changed}
        p = _lib.CbmWalkStream()
        rc = _lib.host_lib().cbm_walk_stream_build(
            a["rowptr"].ctypes.data, a["idx"].ctypes.data, a["parent"].ctypes.data, a["order"].ctypes.data,
            a["level_off"].ctypes.data, changed.get("n", n), mat.n_levels, changed.get("bins", 64), C.byref(p))
        _lib.host_lib().cbm_walk_stream_free(C.byref(p))
        return rc

    assert build() == 0
    bad = arrays["rowptr"].copy(); bad[3] = bad[4] + 1
    assert build(rowptr=bad) != 0
    bad = arrays["idx"].copy(); bad[5] = n
    assert build(idx=bad) != 0
    bad = arrays["parent"].copy(); bad[np.flatnonzero(bad >= 0)[0]] = -1          # a row one level too deep for "root child"
    assert build(parent=bad) != 0
    bad = arrays["order"].copy(); bad[0] = bad[1]
    assert build(order=bad) != 0
    assert build(bins=0) != 0
    assert build(n=0) != 0


@pytest.mark.parametrize("seed", range(8))
def test_random_trees_and_random_delta_rows(seed):
    """Arrays no builder made: a random recursive tree (bushy or nearly a chain), delta rows of 0 .. 200 random
    signed entries (rows that span several stretches, runs of empty rows), every bin target from one bin to one
    subtree per bin -- the layout must hold and the interpreted stream must equal the sum down every row's
    ancestor path computed directly."""
    import types

    from cbm4gnn_amd.cbm import tree_levels
    rng = np.random.default_rng(seed)
    n = int(rng.choice([1, 2, 63, 64, 65, 500, 1500]))
    roots = int(rng.integers(1, max(2, n // 4) + 1))
    par = np.full(n, -1, np.int64)
    stretch = float(rng.choice([0.0, 0.9, 0.995]))                   # how much a row prefers the row just before it
    for v in range(roots, n):
        par[v] = v - 1 if rng.random() < stretch else int(rng.integers(0, v))
    kids = [[] for _ in range(n + 1)]
    for v in range(n):
        kids[n if par[v] < 0 else par[v]].append(v)
    mst_col = np.array(sum(kids, []), np.int32)
    mst_row = np.concatenate([[0], np.cumsum([len(k) for k in kids])]).astype(np.int32)
    parent, order, level_off = tree_levels(mst_row, mst_col)
    lens = rng.choice([0, 0, 1, 2, 3, 7, 64, 70, 200], size=n, p=[.15, .1, .2, .2, .15, .1, .04, .04, .02])
    lens = np.minimum(lens, n)
    rowptr = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    cols = np.concatenate([np.sort(rng.choice(n, size=l, replace=False)) for l in lens] + [np.empty(0, np.int64)]).astype(np.uint32)
    idx = (cols | (rng.integers(0, 2, size=cols.size).astype(np.uint32) << 31)).astype(np.uint32)
    x = rng.integers(-8, 9, size=(n, 2)).astype(np.float64)
    # the product directly: a row's own signed sum plus its parent's value, parents first
    want = np.zeros((n, 2))
    for v in order:
        e = idx[rowptr[v]:rowptr[v + 1]]
        own = (np.where(e >> 31, -1.0, 1.0)[:, None] * x[e & COL]).sum(0) if e.size else 0.0
        want[v] = own + (want[parent[v]] if parent[v] >= 0 else 0.0)
    mat = types.SimpleNamespace(rowptr=torch.from_numpy(rowptr), idx=torch.from_numpy(idx.view(np.int32)),
                                parent=torch.from_numpy(np.asarray(parent, np.int32)), num_rows=n)
    for bins in (1, 7, 100_000):
        p = _lib.CbmWalkStream()
        a = [np.ascontiguousarray(t, np.int32) for t in (parent, order, level_off)]
        rc = _lib.host_lib().cbm_walk_stream_build(rowptr.ctypes.data, idx.ctypes.data, a[0].ctypes.data, a[1].ctypes.data,
                                                   a[2].ctypes.data, n, len(level_off) - 1, bins, C.byref(p))
        assert rc == 0
        try:
            take = lambda ptr, count: torch.from_numpy(np.ctypeslib.as_array(ptr, shape=(count,)).astype(np.int32, copy=True))
            plan = {"n_bins": int(p.n_bins), "n_slots": int(p.n_slots), "n_elems": int(p.n_elems), "heaviest_bin": int(p.heaviest_bin),
                    "gidx": take(p.gidx, p.n_elems), "ginfo": take(p.ginfo, 2 * p.n_elems).view(-1, 2),
                    "bin_goff": take(p.bin_goff, p.n_bins + 1)}
        finally:
            _lib.host_lib().cbm_walk_stream_free(C.byref(p))
        assert plan["n_bins"] == 1 if bins == 1 else plan["n_bins"] >= 1
        check_stream_shape(mat, plan)
        y, written = interpret(plan, x)
        assert (written == 1).all() and np.array_equal(y, want)
