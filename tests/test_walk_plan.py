"""Host side of the walk by subtrees (no GPU): ``cbm_walk_plan_build`` lays the rows below a level out as
depth-first sequences with control words; a NumPy interpreter of those sequences -- the same register / slot
semantics the kernel has -- must reproduce the reference-style walk of the oracle on the same tree."""
import ctypes as C

import numpy as np
import pytest
import torch

from cbm4gnn_amd import _lib, graphs
from cbm4gnn_amd.cbm import cbm_matrix

LOAD_ONLY = _lib.CBM_WALK_LOAD_ONLY


def interpret(plan, m, y):
    """Walk ``y`` in place as one wavefront per bin would: ``run`` = value of the row just finished, slots =
    values of rows with two or more children.  fp32, the arithmetic of the fused walk for ``m`` given
    (FMA body for columns below d - d % 8, division tail), a plain add otherwise."""
    entries, bin_off = plan["entries"].numpy(), plan["bin_off"].numpy()
    d = y.shape[1]
    dv = d - d % 8
    written = np.zeros(y.shape[0], np.int32)
    for b in range(plan["n_bins"]):
        run, mu = None, None
        slots = {}
        for row, ctl in entries[bin_off[b]:bin_off[b + 1]]:
            src, dst = ctl & 63, (ctl >> 8) & 63
            mv = np.float32(1) if m is None else m[row]
            if src == LOAD_ONLY:
                run = y[row].copy()
            else:
                a, ma = (run, mu) if src == 0 else slots[src]
                z = y[row]
                if m is None:
                    run = (z + a).astype(np.float32)
                else:
                    inv = np.float32(1) / ma
                    body = (np.float32(np.float64(a[:dv]) * np.float64(inv) + np.float64(z[:dv]))).astype(np.float32) * mv
                    tail = ((z[dv:] + a[dv:] / ma).astype(np.float32) * mv).astype(np.float32)
                    run = np.concatenate([body, tail]).astype(np.float32)
                y[row] = run
                written[row] += 1
            mu = mv
            if dst:
                assert 1 <= dst <= plan["n_slots"]
                slots[dst] = (run.copy(), mv)
    return written


def check_plan_shape(mat, plan, cut):
    """What the layout promises: every row below the cut exactly once as a computed entry, heads = the rows of
    level ``cut`` with children, a computed row's parent is the row before it or sits in the slot named,
    bins hold whole tasks, longest first."""
    entries, bin_off = plan["entries"].numpy(), plan["bin_off"].numpy()
    parent, order, lo = mat.parent.numpy(), mat.order.numpy(), mat.level_off.numpy()
    n = mat.num_rows
    level = np.empty(n, np.int64)
    level[order] = np.repeat(np.arange(mat.n_levels), np.diff(lo))
    has_child = np.zeros(n, bool)
    has_child[parent[parent >= 0]] = True
    heads = entries[(entries[:, 1] & 63) == LOAD_ONLY, 0]
    assert sorted(heads.tolist()) == sorted(np.flatnonzero((level == cut) & has_child).tolist())
    body = entries[(entries[:, 1] & 63) != LOAD_ONLY, 0]
    assert sorted(body.tolist()) == np.flatnonzero(level > cut).tolist()
    assert bin_off[0] == 0 and bin_off[-1] == entries.shape[0] == plan["n_entries"] and (np.diff(bin_off) > 0).all()
    assert ((entries[bin_off[:-1], 1] & 63) == LOAD_ONLY).all()                 # a bin starts with a head
    assert int(np.diff(bin_off).max()) == plan["longest_bin"]
    slot_row = {}
    for b in range(plan["n_bins"]):
        prev = None
        for row, ctl in entries[bin_off[b]:bin_off[b + 1]]:
            src, dst = ctl & 63, (ctl >> 8) & 63
            if src == 0:
                assert parent[row] == prev
            elif src != LOAD_ONLY:
                assert slot_row[src] == parent[row]
            if dst:
                slot_row[dst] = row
                assert (parent == row).sum() >= 2
            prev = row


@pytest.mark.parametrize("normalized", [False, True])
@pytest.mark.parametrize("graph", ["sbm", "chain", "staircases", "dup"])
def test_plan_interpreted_equals_the_oracle_walk(orc, graph, normalized):
    if graph == "sbm":
        n = 900
        ei = graphs.sbm(n, 9, 0.4, 0.01, seed=3)
    elif graph == "chain":
        n = 1500
        ei = graphs.sbm_with_chain(n=n, blocks=24, p_in=1.0, mean_deg=80.0, chain=64, base=48, seed=0)
    elif graph == "staircases":
        ei = graphs.staircases(12, 20, 6, 2.0, seed=1)
        n = int(ei.max()) + 1
    else:
        n = 1200
        ei = graphs.duplication(n, 0.7, 3, 8, seed=2)
    if normalized:
        ei = graphs.add_self_loops(ei, n)
    mat = cbm_matrix(torch.from_numpy(ei), None, alpha=0, normalized=normalized)
    assert mat.n_levels >= 3
    d = 19                                                     # d % 8 != 0: body and tail of the fused walk
    z = np.random.default_rng(7).standard_normal((n, d)).astype(np.float32)
    m = orc.col_multiplier(ei, n) if normalized else None
    z0 = z.copy()
    if normalized:                                             # children of the root are scaled before the walk
        roots = mat.parent.numpy() < 0
        z0[roots] = (z0[roots] * m[roots, None]).astype(np.float32)
    want = (orc.update_fused(mat.mst_row.numpy(), mat.mst_col.numpy(), m, z.copy()) if normalized
            else orc.update_plain(mat.mst_row.numpy(), mat.mst_col.numpy(), z.copy()))
    level_of = np.empty(n, np.int64)
    level_of[mat.order.numpy()] = np.repeat(np.arange(mat.n_levels), np.diff(mat.level_off.numpy()))
    for cut in (0, 1, mat.n_levels - 2):
        plan = mat._host_walk_plan(cut, d)
        check_plan_shape(mat, plan, cut)
        y = z0.copy()
        above = level_of <= cut
        y[above] = want[above]                                 # levels 1 .. cut were walked level by level before
        written = interpret(plan, m, y)
        assert np.array_equal(written, (~above).astype(np.int32))
        assert np.array_equal(y, want), (graph, normalized, cut)
    # slots stay few: children are visited lightest first
    assert mat._host_walk_plan(0, d)["n_slots"] <= int(np.log2(n)) + 1


def test_plan_bins_pack_small_tasks_and_keep_long_ones_alone():
    ei = graphs.add_self_loops(graphs.staircases(40, 30, 6, 2.0, seed=2))
    mat = cbm_matrix(torch.from_numpy(ei), None, alpha=0, normalized=True)
    p = _lib.CbmWalkPlan()
    host = _lib.host_lib()
    ptr = lambda t: C.c_void_p(t.data_ptr())
    sizes = {}
    for target in (1, 16, 4096):
        assert host.cbm_walk_plan_build(ptr(mat.parent), ptr(mat.order), ptr(mat.level_off), mat.num_rows, mat.n_levels, 0,
                                        target, C.byref(p)) == 0
        off = np.ctypeslib.as_array(p.bin_off, shape=(p.n_bins + 1,)).copy()
        sizes[target] = np.diff(off)
        assert p.n_entries == off[-1]
        host.cbm_walk_plan_free(C.byref(p))
    assert sizes[1].shape[0] == 1                                               # everything in one bin
    assert sizes[4096].shape[0] > sizes[16].shape[0] > 1
    assert sizes[4096].min() >= 2 and (np.diff(sizes[4096][:-1]) <= 32).all()  # longest first, up to the packing
    # bad input
    assert host.cbm_walk_plan_build(ptr(mat.parent), ptr(mat.order), ptr(mat.level_off), mat.num_rows, mat.n_levels,
                                    mat.n_levels, 8, C.byref(p)) == _lib.CBM_ERR_SHAPE
    assert host.cbm_walk_plan_build(None, ptr(mat.order), ptr(mat.level_off), mat.num_rows, mat.n_levels, 0, 8,
                                    C.byref(p)) == _lib.CBM_ERR_NULL
    bad = mat.parent.clone(); bad[int(mat.order[-1])] = -1                       # a deep row claims to hang off the root
    assert host.cbm_walk_plan_build(ptr(bad), ptr(mat.order), ptr(mat.level_off), mat.num_rows, mat.n_levels, 0, 8,
                                    C.byref(p)) == _lib.CBM_ERR_SHAPE


def test_walk_policy_by_estimate():
    """"auto" takes the subtree walk for a deep and wide tree and leaves shallow trees to the one-launch path
    walk; "off" and a forced cut do what they say."""
    deep = cbm_matrix(torch.from_numpy(graphs.add_self_loops(graphs.staircases(60, 40, 6, 2.0, seed=3))), None, alpha=0,
                      normalized=True)
    assert deep.n_levels > 16
    plan = deep.walk_plan(256)
    assert plan is not None and plan["cut"] == 0 and plan["n_bins"] > 1
    deep.subtree_walk = "off"
    assert deep.walk_plan(256) is None
    deep.subtree_walk = 2
    assert deep.walk_plan(256)["cut"] == 2
    shallow = cbm_matrix(torch.from_numpy(graphs.add_self_loops(graphs.sbm(600, 6, 0.4, 0.01, seed=1), 600)), None, alpha=0,
                         normalized=True)
    # "auto" follows the estimate, whatever the depth (a multiply the one-launch path walk takes does not ask)
    assert 2 <= shallow.n_levels <= 16
    auto, level_cost = shallow.walk_plan(128), shallow._level_plan_cost_us(128)
    shallow.subtree_walk = "on"
    forced = shallow.walk_plan(128)
    assert forced is not None
    assert (auto is not None) == (shallow._subtree_plan_cost_us(forced, 128) <= 0.8 * level_cost)
    flat = cbm_matrix(torch.from_numpy(graphs.erdos_renyi(50, 0.3, 1)), None, alpha=10_000)
    flat.subtree_walk = "on"
    assert flat.walk_plan(64) is None


def test_auto_finds_a_deeper_cut_when_the_top_of_the_tree_is_narrow():
    """One child of the root, 4 rows below it, 256 below those, then 256 chains of 100 rows: walked from the
    root's child the whole tree is ONE sequence; below level 2 it is 256 independent ones.  The estimate must
    pick that cut (levels 1 and 2 level by level, the rest in one launch)."""
    from cbm4gnn_amd.cbm import tree_levels
    par = [-1] + [0] * 4 + [1 + i // 64 for i in range(256)]
    first_chain = len(par)
    for depth in range(100):
        par += [first_chain - 256 + i if depth == 0 else first_chain + (depth - 1) * 256 + i for i in range(256)]
    par = np.array(par, np.int64)
    n = par.shape[0]
    kids = [[] for _ in range(n + 1)]
    for v in range(n):
        kids[n if par[v] < 0 else par[v]].append(v)
    mst_col = np.array(sum(kids, []), np.int32)
    mst_row = np.concatenate([[0], np.cumsum([len(k) for k in kids])]).astype(np.int32)
    parent, order, level_off = tree_levels(mst_row, mst_col)
    mat = cbm_matrix.__new__(cbm_matrix)
    mat.num_rows, mat.n_levels = n, level_off.shape[0] - 1
    mat.parent, mat.order, mat.level_off = (torch.from_numpy(a) for a in (parent, order, level_off))
    mat._walk_plans, mat.subtree_walk = {}, "auto"
    assert mat.n_levels == 103
    plan = mat.walk_plan(256)
    assert plan is not None and plan["cut"] == 2 and plan["longest_bin"] <= 2 * 101 and plan["n_entries"] == 256 * 101
    assert mat._subtree_plan_cost_us(plan, 256) < 0.2 * mat._level_plan_cost_us(256)
    sizes = mat._subtree_sizes()
    assert sizes[0] == n and (sizes[1:5] == 1 + 64 * 101).all() and sizes[-1] == 1
    # a forced cut of 0 is still honoured (one bin, one long sequence)
    mat.subtree_walk = 0
    assert mat.walk_plan(256)["n_bins"] == 1


def _fake_matrix(par):
    """A ``cbm_matrix`` shell holding only a tree (what the walk plan reads)."""
    from cbm4gnn_amd.cbm import tree_levels
    n = par.shape[0]
    kids = [[] for _ in range(n + 1)]
    for v in range(n):
        kids[n if par[v] < 0 else par[v]].append(v)
    mst_col = np.array(sum(kids, []), np.int32)
    mst_row = np.concatenate([[0], np.cumsum([len(k) for k in kids])]).astype(np.int32)
    parent, order, level_off = tree_levels(mst_row, mst_col)
    mat = cbm_matrix.__new__(cbm_matrix)
    mat.num_rows, mat.n_levels = n, level_off.shape[0] - 1
    mat.parent, mat.order, mat.level_off = (torch.from_numpy(a) for a in (parent, order, level_off))
    mat.mst_row, mat.mst_col = torch.from_numpy(mst_row), torch.from_numpy(mst_col)
    mat._walk_plans, mat.subtree_walk = {}, "auto"
    return mat


@pytest.mark.parametrize("seed", range(12))
def test_plans_of_random_trees_walk_like_the_oracle(orc, seed):
    """Random forests of every shape the builder can produce and some it rarely does -- random recursive trees
    (bushy, ~2 ln n levels), brooms (a chain ending in a star), caterpillars, forests of stars, near-binary trees,
    single rows -- at every cut level: the plan's layout invariants hold and its interpretation equals the
    oracle's walk (plain and fused) bit for bit."""
    rng = np.random.default_rng(100 + seed)
    n = int(rng.choice([1, 2, 17, 200, 1500]))
    kind = ["recursive", "broom", "caterpillar", "stars", "binary", "forest"][seed % 6]
    roots = int(rng.integers(1, max(2, n // 10 + 1)))
    par = np.full(n, -1, np.int64)
    for v in range(roots, n):
        if kind == "recursive" or kind == "forest":
            par[v] = int(rng.integers(0, v))
        elif kind == "broom":
            par[v] = v - roots if v < n // 2 else int(rng.integers(max(roots, n // 2 - roots), max(roots + 1, n // 2)))
        elif kind == "caterpillar":
            par[v] = v - 2 * roots if (v - roots) % 2 == 0 and v >= 3 * roots else max(v - roots - (v - roots) % 2 * roots, 0) if v >= 2 * roots else v - roots
        elif kind == "stars":
            par[v] = v % roots
        else:
            par[v] = (v - roots) // 2 if (v - roots) // 2 < v else 0
    par = np.minimum(par, np.arange(n) - 1)                    # a parent always precedes its child: no cycles
    par[:roots] = -1
    mat = _fake_matrix(par)
    d = int(rng.choice([1, 8, 19]))
    z = rng.standard_normal((n, d)).astype(np.float32)
    m = (rng.random(n).astype(np.float32) + 0.5)
    for fused in (False, True):
        want = (orc.update_fused(mat.mst_row.numpy(), mat.mst_col.numpy(), m, z.copy()) if fused
                else orc.update_plain(mat.mst_row.numpy(), mat.mst_col.numpy(), z.copy()))
        z0 = z.copy()
        if fused:
            rt = mat.parent.numpy() < 0
            z0[rt] = (z0[rt] * m[rt, None]).astype(np.float32)
        level_of = np.empty(n, np.int64)
        level_of[mat.order.numpy()] = np.repeat(np.arange(mat.n_levels), np.diff(mat.level_off.numpy()))
        for cut in sorted({0, mat.n_levels // 2, max(mat.n_levels - 2, 0)}):
            if cut >= mat.n_levels:
                continue
            plan = mat._host_walk_plan(cut, d)
            assert plan, (kind, n, cut)
            if plan["n_entries"]:
                check_plan_shape(mat, plan, cut)
            y = z0.copy()
            above = level_of <= cut
            y[above] = want[above]
            written = interpret(plan, m if fused else None, y)
            assert np.array_equal(written, (~above).astype(np.int32))
            assert np.array_equal(y, want), (kind, n, fused, cut)
    # the estimate-driven choice never fails to produce a usable answer
    mat.subtree_walk = "on"
    chosen = mat.walk_plan(64)
    assert chosen is None or 0 <= chosen["cut"] < mat.n_levels
