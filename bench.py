#!/usr/bin/env python3
"""Benchmark of the CBM multiply on one MI355X.

    python bench.py [--gpus 1] [--steps 50] [--warmup 5] [--workload c3] [--alpha 16] [--d 256]

A "step" is one CBM multiply  Y = A_hat X  (delta SpMM + tree propagation through the C ABI)
on fixed device buffers; the format is built once, outside the timed region, as in the
reference's protocol (``benchmark/parallel/benchmark_spmm_cpu.py:119-151``: 50 timed calls on
fixed x, y).  Default workload: the 100k-node Chung-Lu + cliques graph, GCN-normalised, alpha=16,
feature width 256.  Prints ONE JSON line.  The default run also carries, in the same line,

  * ``gcn_epoch``        the 2-layer GCN forward + backward epoch on the 233k-node SBM (c4), with
                         CBM aggregation and with the hand-written GPU CSR layers;
  * ``other_workloads``  one compact row each for the duplication graph (c2, alpha 0 and 8), the
                         4,096-node SBM (c1) and the dense-community graph with the deep chain (c5);
  * ``cpu_baseline``     the reference-style CPU path on the host cores of the same box, all
                         threads and one thread (``benchmark/sequential/benchmark_spmm_cpu.py:1-11``):
                         MKL ``mkl_sparse_s_mm`` (reached through torch's libtorch_cpu.so, handle
                         re-created per call like the reference) + the OpenMP tree walk of the oracle;
  * ``gpu_vendor_csr``   the CSR product of the same matrix through ``torch.sparse.mm`` (hipSPARSE), an
                         outside anchor for the hand-written GPU CSR baseline.

``--only-multiply`` skips the extra sections (GCN epoch, other workloads, vendor CSR); ``--gcn`` and ``--sweep`` run one of them alone.
"""
from __future__ import annotations

import argparse
import contextlib
import glob
import hashlib
import json
import os
import re
import statistics
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0
KERNEL_SOURCE = os.path.join(ROOT, "cbm4gnn_amd", "csrc", "cbm_kernels.hip")


def kernel_source_hash():
    with open(KERNEL_SOURCE, "rb") as f:
        return hashlib.sha256(f.read()).hexdigest()[:16]


def measured_traffic(workload, alpha, d):
    """HBM-side bytes per launch of the dominant kernel from the counter summaries under
    ``profiles/``.  Counters cannot be read from inside this process; a summary records them as

        traffic-record: workload=c3 alpha=16 d=256 kernel=<instantiation> fetch_bytes=.. write_bytes=.. kernels_sha256=..

    where ``kernels_sha256`` is the hash of the kernel source the counters were taken on.  A record
    taken on another version of the kernels is reported as stale and contributes no number."""
    want = {"workload": workload, "alpha": str(alpha), "d": str(d)}
    stale = None
    for path in sorted(glob.glob(os.path.join(ROOT, "profiles", "*.md"))):
        with open(path) as f:
            for line in f:
                if "traffic-record:" not in line:
                    continue
                rec = dict(kv.split("=", 1) for kv in re.findall(r"\S+=\S+", line.split("traffic-record:", 1)[1]))
                if any(rec.get(k) != v for k, v in want.items()):
                    continue
                src = {"file": os.path.relpath(path, ROOT), "kernel": rec.get("kernel"),
                       "kernels_sha256": rec.get("kernels_sha256")}
                if rec.get("kernels_sha256") != kernel_source_hash():
                    stale = src
                    continue
                return float(rec["fetch_bytes"]) + float(rec["write_bytes"]), src, False
    return None, stale, stale is not None


def algorithmic_bytes(n, nnz, d, norm, tree_edges, levels, n_edges_a):
    """Bytes one multiply must move under the gather model (no reuse of X rows assumed)."""
    b_spmm = 4 * (n + 1) + 4 * nnz * (1 + norm) + 4 * d * nnz + 4 * d * n
    b_prop = (4 * (2 * n + levels + 1) + 4 * n * norm + 4 * d * 3 * tree_edges) if tree_edges else 0
    b_csr = 4 * (n + 1) + 4 * n_edges_a * (1 + norm) + 4 * d * n_edges_a + 4 * d * n
    return b_spmm, b_prop, b_csr


def compulsory_bytes(n, nnz, d):
    """Lower bound: X read once, Y written once, every index once, three words per row."""
    return 4 * d * 2 * n + 4 * (nnz + 3 * n)


def time_gpu(fn, steps, warmup, torch):
    """(wall ms per step, GPU ms per step, median ms of per-call events).  The first two come from ONE
    loop of exactly ``steps`` calls issued back to back between two synchronisations (wall clock around
    the synchronisations, one event pair inside them); the median from a second loop of the same
    length with an event pair around every call (those records cost about 10 us per call, which is
    why that loop is not the one the per-step figures come from)."""
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    a.record()
    for _ in range(steps):
        fn()
    b.record()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3 / steps
    span_ms = a.elapsed_time(b) / steps
    starts = [torch.cuda.Event(enable_timing=True) for _ in range(steps)]
    ends = [torch.cuda.Event(enable_timing=True) for _ in range(steps)]
    for i in range(steps):
        starts[i].record()
        fn()
        ends[i].record()
    torch.cuda.synchronize()
    per_call = [s.elapsed_time(e) for s, e in zip(starts, ends)]
    return wall_ms, span_ms, statistics.median(per_call)


def time_gpu_back_to_back(fn, steps, torch):
    """GPU ms per call of ``steps`` calls between one pair of events (a longer loop than time_gpu's,
    for the workloads whose multiply takes tens of microseconds)."""
    fn()
    torch.cuda.synchronize()
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    a.record()
    for _ in range(steps):
        fn()
    b.record()
    torch.cuda.synchronize()
    return a.elapsed_time(b) / steps


def csr_of(edge_index, n, m=None):
    """(rowptr int32, col int32, val fp32 or None, order) of the CSR of a COO list, NumPy."""
    import numpy as np
    ei = edge_index
    order = np.lexsort((ei[1], ei[0]))
    rp = np.concatenate([[0], np.cumsum(np.bincount(ei[0], minlength=n))]).astype(np.int32)
    col = np.ascontiguousarray(ei[1][order].astype(np.int32))
    val = None
    if m is not None:
        val = (m[ei[0][order]] * m[col]).astype(np.float32)
    return rp, col, val


def vendor_csr_spmm(rp, col, val, xd, y_ref, steps, torch):
    """The same CSR product through the vendor library: ``torch.sparse.mm`` on a CSR tensor, which
    torch's ROCm build hands to hipSPARSE's SpMM.  An outside anchor for the hand-written GPU CSR
    baseline; returns None where this torch build cannot run it."""
    try:
        n = rp.shape[0] - 1
        values = torch.ones(col.shape[0], dtype=torch.float32) if val is None else torch.from_numpy(val)
        a = torch.sparse_csr_tensor(torch.from_numpy(rp), torch.from_numpy(col), values, size=(n, n)).to(xd.device)
        _, ms, med = time_gpu(lambda: torch.sparse.mm(a, xd), steps, 2, torch)
        err = float((torch.sparse.mm(a, xd) - y_ref).abs().max() / y_ref.abs().max())
        return {"what": "torch.sparse.mm(CSR, X) (hipSPARSE SpMM)", "ms": ms, "ms_median": med, "calls": steps,
                "max_rel_err_vs_gpu_csr": err}
    except Exception as e:          # noqa: BLE001 -- optional leg: report why it is absent
        return {"what": "torch.sparse.mm(CSR, X)", "error": f"{type(e).__name__}: {e}"[:200]}


def cpu_rows_fp64(rp, col, val, x, rows):
    """Rows ``rows`` of ``A_hat X`` in fp64 straight from the CSR arrays (SciPy): an anchor that
    shares no code with the kernels, cheap enough for every workload."""
    import numpy as np
    import scipy.sparse as sp
    cnt = (rp[rows + 1] - rp[rows]).astype(np.int64)
    take = np.repeat(rp[rows].astype(np.int64), cnt) + (np.arange(int(cnt.sum())) - np.repeat(np.cumsum(cnt) - cnt, cnt))
    sub = sp.csr_matrix((np.ones(take.shape[0]) if val is None else val[take].astype(np.float64), col[take],
                         np.concatenate([[0], np.cumsum(cnt)])), shape=(rows.shape[0], x.shape[0]))
    return sub @ x.astype(np.float64)


def cpu_baseline(w, mat, x, budget_s=20.0, max_iters=50, threads=0):
    """Reference-style CPU CBM and CPU CSR multiplies on this host (MKL SpMM + OpenMP walk), with
    all threads and with one thread."""
    import numpy as np
    import torch
    from oracle import cbm_oracle as orc

    n, d = x.shape
    all_threads = orc.max_threads()
    if threads > 0:                                           # --threads: the reference's num_threads knob
        all_threads = min(int(threads), all_threads)
        torch.set_num_threads(all_threads)
    ei = w.edge_index
    m = orc.col_multiplier(ei, n) if w.normalized else None
    col, sign = mat.columns()
    col = col.numpy().astype(np.int32)
    val = (sign.numpy() * (m[col] if m is not None else 1.0)).astype(np.float32)
    rp = mat.rowptr.numpy()
    rb, re = np.ascontiguousarray(rp[:-1]), np.ascontiguousarray(rp[1:])
    mst_row, mst_col = mat.mst_row.numpy(), mat.mst_col.numpy()
    arp, acol, aval = csr_of(ei, n, m)
    if aval is None:
        aval = np.ones(acol.shape[0], np.float32)
    arb, are = np.ascontiguousarray(arp[:-1]), np.ascontiguousarray(arp[1:])
    y = np.empty((n, d), np.float32)
    use_mkl = orc.mkl() is not None

    walk_ms = []

    def legs(threads, budget, iters):
        def spmm(b, e, c, v):
            if use_mkl:
                orc.mkl_csr_spmm(b, e, c, v, x, y)
            else:
                y[:] = orc.csr_spmm(np.concatenate([b, e[-1:]]), c, v, x, threads)

        def cbm_call():
            spmm(rb, re, col, val)
            t = time.perf_counter()
            if m is None:
                orc.update_plain(mst_row, mst_col, y, threads)
            else:
                orc.update_fused(mst_row, mst_col, m, y, threads)
            walk_ms.append((time.perf_counter() - t) * 1e3)

        def csr_call():
            spmm(arb, are, acol, aval)

        def run(fn):
            # 1 warm-up, as the reference -- unless one call alone takes a third of the leg's budget: then the
            # first call is a sample like the others (said in the report: warm-up 0)
            t = time.perf_counter(); fn(); first = (time.perf_counter() - t) * 1e3
            warm = 1
            ts = []
            if first * 1e-3 > budget / 6:
                ts, warm = [first], 0
            t_end = time.perf_counter() + budget / 2
            while len(ts) < iters and (not ts or time.perf_counter() < t_end):
                t = time.perf_counter(); fn(); ts.append((time.perf_counter() - t) * 1e3)
            return ts, warm

        del walk_ms[:]
        t_cbm, warm = run(cbm_call)
        walk = statistics.mean(walk_ms[-len(t_cbm):])
        y_cbm = y.copy()
        t_csr, _ = run(csr_call)
        return t_cbm, t_csr, y_cbm, walk, warm

    t_cbm, t_csr, y_cbm, walk, _ = legs(all_threads, budget_s, max_iters)
    torch.set_num_threads(1)                                  # OpenMP and MKL: the "sequential" protocol
    try:
        t_cbm1, t_csr1, _, _, warm1 = legs(1, budget_s / 2, 10)
    finally:
        torch.set_num_threads(all_threads)
    return {
        "cbm_ms_mean": statistics.mean(t_cbm), "cbm_ms_median": statistics.median(t_cbm),
        "csr_ms_mean": statistics.mean(t_csr), "csr_ms_median": statistics.median(t_csr),
        "walk_ms_mean": walk,
        "cbm_ms_1t": statistics.mean(t_cbm1), "csr_ms_1t": statistics.mean(t_csr1),
        "iters": [len(t_cbm), len(t_csr)], "iters_1t": [len(t_cbm1), len(t_csr1)], "warmup_1t": warm1, "threads": all_threads,
        "spmm": "mkl_sparse_s_mm via libtorch_cpu.so" if use_mkl else "hand OpenMP CSR SpMM (non-MKL stand-in)",
    }, y_cbm


def spmm_alone(mat, xd, normalized, steps, warmup, torch):
    """The delta SpMM launch of a multiply on its own -- the dominant kernel -- timed with the slab-major
    copy of X made once beforehand (that copy is timed separately).  Returns (copy ms, SpMM ms, Z, name of
    the kernel)."""
    from cbm4gnn_amd.cbm import _wants_workspace, relayout_slabs
    n, d = xd.shape
    zd = torch.empty_like(xd)
    scale = mat._device_arrays(xd.device)["m"] if normalized else None       # the step scales its copy by m
    ws, relayout_ms = None, 0.0
    if mat.relayout and (mat.is_tiled() or mat.has_cut_rows() or _wants_workspace(xd, zd, mat.nnz)):
        # room for the copy and, where the plan cuts rows into pieces, their sums behind it
        ws = torch.empty(mat.workspace_floats(n, d, xd.device), dtype=torch.float32, device=xd.device)
        relayout_slabs(xd, scale=scale, out=ws)
        _, relayout_ms, _ = time_gpu(lambda: relayout_slabs(xd, scale=scale, out=ws), steps, warmup, torch)
    fn = lambda: mat._run_spmm(xd, zd, use_m=normalized, scale_roots=normalized, workspace=ws,
                               workspace_ready=ws is not None, workspace_prescaled=ws is not None and scale is not None)
    _, spmm_ms, _ = time_gpu(fn, steps, warmup, torch)
    kernel = ("spmm_tiled_local" if mat.is_tiled() else
              "spmm_slab_per_xcd" if (ws is not None or d % 32 == 0) else "spmm_wave_per_row")
    return relayout_ms, spmm_ms, zd, kernel


def roofline_of(name, alpha, d, kernel, launch_ms, algorithmic, compulsory, scale=1.0):
    """The ``roofline`` object of one kernel launch.  ``frac``: algorithmic (gather-model, no reuse assumed)
    bytes over the launch time -- it exceeds 1 where rows of X are re-used out of L2 / the memory-side cache.
    ``frac_traffic``: counter-measured HBM-side bytes (a ``traffic-record:`` under profiles/, dropped as stale
    when taken on another version of the kernel source) over the same time: what the memory system really
    moved.  ``frac_compulsory``: the lower bound (X once, Y once, every index once) over the same time."""
    traffic, src, stale = measured_traffic(name, alpha, d) if scale == 1.0 else (None, None, False)
    achieved = algorithmic / (launch_ms * 1e-3) / 1e9
    return {"bound": "hbm", "kernel": kernel, "achieved": achieved, "peak": HBM_PEAK_GBPS, "unit": "GB/s",
            "frac": achieved / HBM_PEAK_GBPS, "traffic": traffic,
            "frac_traffic": (traffic / (launch_ms * 1e-3) / 1e9 / HBM_PEAK_GBPS) if traffic else None,
            "frac_compulsory": compulsory / (launch_ms * 1e-3) / 1e9 / HBM_PEAK_GBPS,
            "traffic_source": src, "traffic_stale": stale, "kernels_sha256": kernel_source_hash(),
            "algorithmic_bytes": algorithmic, "compulsory_bytes": compulsory, "avg_launch_ms": launch_ms}


FLAT_ALPHA = 1 << 30          # prunes every candidate pair: flat tree, delta matrix = A ("alpha = infinity")


def measure_multiply(w, alpha, d, args, torch, vendor=False, sample_rows=512, cpu=None, flat=True):
    """Build the format of workload ``w`` and time, on the same X: the CBM multiply; the hand-written GPU
    CSR baseline (generic fp32 values); the same graph as a FLAT-tree CBM (``flat_binary_ms``: alpha =
    infinity, so the delta matrix is A itself in the value-free packed format on the same best kernels --
    what the tree and its compression add is ``speedup_from_compression = flat_binary_ms / cbm_ms``, as the
    reference reports CBM against CSR, plot_results_alpha_vs_runtime.py:53-63); the dominant kernel alone
    (``roofline``); and, with ``cpu`` = a budget in seconds, the reference-style CPU legs.
    Returns (row dict, handles for the caller that wants more)."""
    import numpy as np

    from cbm4gnn_amd.cbm import DEFAULT_BATCH_ROWS, cbm_matrix, csr_spmm, schedule_rows

    t0 = time.perf_counter()
    mat = cbm_matrix(torch.from_numpy(w.edge_index), None, alpha=alpha, normalized=w.normalized, builder=args.builder,
                     max_levels=args.max_levels)
    t_build = time.perf_counter() - t0
    n, nnz, n_edges = w.n, mat.nnz, mat.nnz_a
    norm = int(w.normalized)
    tree_edges = n - int(mat.level_off[1])
    x = w.features(0, d)
    xd = x.cuda()
    yd = torch.empty_like(xd)
    mat.to(xd.device)
    step = (lambda: mat.omp_mkl_csr_fused_spmm_update(xd, yd)) if w.normalized else (lambda: mat.omp_mkl_csr_spmm_update(xd, yd))
    wall_ms, span_ms, med_ms = time_gpu(step, args.steps, args.warmup, torch)

    # hand-written GPU CSR baseline on A_hat (explicit values when normalised), same row scheduling
    m_np = mat.col_multiplier.numpy() if w.normalized else None
    rp, col, val = csr_of(w.edge_index, n, m_np)
    rp_d, col_d = torch.from_numpy(rp).cuda(), torch.from_numpy(col).cuda()
    val_d = None if val is None else torch.from_numpy(val).cuda()
    ycsr = torch.empty_like(xd)
    csr_sched = schedule_rows(torch.from_numpy(rp), batch=DEFAULT_BATCH_ROWS).to(xd.device)
    csr_step = lambda: csr_spmm(rp_d, col_d, val_d, xd, ycsr, csr_sched)
    _, csr_ms, _ = time_gpu(csr_step, args.steps, args.warmup, torch)
    # ten times as many calls where a call is short (launch gaps and clock ramps weigh on 20 calls of 20 us)
    reps, loop_ms, csr_loop_ms = args.steps, span_ms, csr_ms
    if span_ms < 0.2:
        reps = 10 * args.steps
        loop_ms, csr_loop_ms = time_gpu_back_to_back(step, reps, torch), time_gpu_back_to_back(csr_step, reps, torch)
    step()
    torch.cuda.synchronize()
    err_vs_csr = float((yd - ycsr).abs().max() / ycsr.abs().max())
    vendor_row = vendor_csr_spmm(rp, col, val, xd, ycsr, min(args.steps, 10), torch) if vendor else None
    # anchor that shares no code with the kernels: a sample of rows in fp64 from the edge list
    rows = np.sort(np.random.default_rng(0).choice(n, size=min(sample_rows, n), replace=False))
    want = cpu_rows_fp64(rp, col, val, x.numpy(), rows)
    got = yd[torch.from_numpy(rows).cuda()].cpu().numpy().astype(np.float64)
    err_vs_cpu_rows = float(np.abs(got - want).max() / np.abs(want).max())
    del rp_d, col_d, val_d, csr_sched

    # the same graph as a flat-tree CBM: value-free packed A on the same kernels
    if mat.n_levels == 1 and nnz == n_edges:
        flat_ms, flat_loop_ms = span_ms, loop_ms            # this format IS the flat one
    elif flat:
        fm = cbm_matrix(torch.from_numpy(w.edge_index), None, alpha=FLAT_ALPHA, normalized=w.normalized, builder=args.builder)
        assert fm.n_levels == 1 and fm.nnz == n_edges
        fm.to(xd.device)
        yf = torch.empty_like(xd)
        fstep = (lambda: fm.omp_mkl_csr_fused_spmm_update(xd, yf)) if w.normalized else (lambda: fm.omp_mkl_csr_spmm_update(xd, yf))
        _, flat_ms, _ = time_gpu(fstep, args.steps, args.warmup, torch)
        flat_loop_ms = time_gpu_back_to_back(fstep, reps, torch) if reps != args.steps else flat_ms
        del fm, yf
    else:
        flat_ms = flat_loop_ms = None

    b_spmm, b_prop, b_csr = algorithmic_bytes(n, nnz, d, norm, tree_edges, mat.n_levels, n_edges)
    b_min = compulsory_bytes(n, nnz, d)
    # the dominant kernel alone; a small product on a shallow tree is ONE launch that does everything
    if not mat.is_tiled() and not mat.has_cut_rows() and mat._single_launch(n, d):
        relayout_ms, spmm_ms, prop_ms, prop_how, kernel, slab = 0.0, span_ms, 0.0, None, "spmm_update_paths_wave_per_row", False
        roof = roofline_of(w.name, alpha, d, kernel, spmm_ms, b_spmm + b_prop, b_min, args.scale)
    elif streams_in_multiply(mat, n, d):
        # a deep tree with short delta rows: ONE launch sums the rows and walks the subtrees
        relayout_ms, spmm_ms, prop_ms, prop_how, kernel, slab = 0.0, span_ms, 0.0, None, "spmm_update_subtrees", False
        roof = roofline_of(w.name, alpha, d, kernel, spmm_ms, b_spmm + b_prop, b_min, args.scale)
    else:
        relayout_ms, spmm_ms, zd, kernel = spmm_alone(mat, xd, w.normalized, args.steps, args.warmup, torch)
        prop_ms, prop_how = 0.0, None
        if tree_edges and walks_paths_in_multiply(mat, n, d):
            # the path walk reads Z from a scratch the multiply fills: it cannot run on its own
            prop_ms, prop_how = max(span_ms - relayout_ms - spmm_ms, 0.0), "multiply minus copy and SpMM (the path walk runs only inside the multiply)"
        elif tree_edges:
            # the walk as the multiply runs it: the root children were scaled in the SpMM's epilogue
            _, prop_ms, _ = time_gpu(lambda: mat._run_propagate(zd, use_m=w.normalized, scale_roots=False), args.steps, args.warmup, torch)
            prop_how = "the walk's launches alone, in place on Z"
        slab = kernel != "spmm_wave_per_row"
        roof = roofline_of(w.name, alpha, d, kernel, spmm_ms, b_spmm, b_min, args.scale)
        del zd
    row = {
        "workload": f"{w.name}: {w.note}", "alpha": alpha, "d": d, "nodes": n, "nnz_A": n_edges, "nnz_delta": nnz,
        "compression_ratio": mat.compression_ratio(), "tree_levels": mat.n_levels, "tree_edges": tree_edges,
        "launches_per_multiply": launches_per_multiply(mat, n, d, copies_x=relayout_ms > 0.0),
        "cbm_ms": span_ms, "cbm_ms_median": med_ms, "gpu_csr_ms": csr_ms, "speedup_vs_gpu_csr": csr_ms / span_ms,
        "flat_binary_ms": flat_ms, "speedup_from_compression": (flat_ms / span_ms) if flat_ms else None,
        "cbm_ms_back_to_back": loop_ms, "gpu_csr_ms_back_to_back": csr_loop_ms,
        "flat_binary_ms_back_to_back": flat_loop_ms,
        "speedup_vs_gpu_csr_back_to_back": csr_loop_ms / loop_ms, "back_to_back_calls": reps,
        "kernel_ms": {"relayout_slabs": relayout_ms, "delta_spmm": spmm_ms, "propagate": prop_ms, "propagate_is": prop_how},
        "walk_share": prop_ms / (relayout_ms + spmm_ms + prop_ms) if prop_ms else 0.0,
        "cbm_GBps": (b_spmm + b_prop) / (span_ms * 1e-3) / 1e9,
        "edges_x_features_per_s": n_edges * d / (span_ms * 1e-3),
        "roofline": roof,
        "max_rel_err_vs_gpu_csr": err_vs_csr, "max_rel_err_vs_cpu_fp64_rows": err_vs_cpu_rows,
        "cpu_rows_checked": int(rows.shape[0]), "build_s": t_build,
    }
    if vendor_row is not None:
        row["gpu_vendor_csr"] = vendor_row
    if cpu:
        c, y_cpu = cpu_baseline(w, mat, x.numpy(), budget_s=cpu, threads=args.threads)
        row["cpu_baseline"] = cpu_baseline_object(c)
        got_all = yd.cpu().numpy()
        row["max_rel_err_vs_cpu_cbm"] = float(np.abs(got_all - y_cpu).max() / np.abs(y_cpu).max())
        del got_all, y_cpu
    extra = {"mat": mat, "x": x, "xd": xd, "yd": yd, "wall_ms": wall_ms, "span_ms": span_ms, "med_ms": med_ms,
             "csr_ms": csr_ms, "b": (b_spmm, b_prop, b_csr), "t_build": t_build, "tree_edges": tree_edges,
             "relayout_ms": relayout_ms, "spmm_ms": spmm_ms, "prop_ms": prop_ms, "slab": slab}
    return row, extra


def level_launches(lo, first_level, last_level):
    """Launches the level-by-level walk issues for levels first_level .. last_level - 1 (the library's plan:
    one per wide level, one per run of narrow levels, one per chain of at least four single-row levels)."""
    width = lambda l: lo[l + 1] - lo[l]

    def chain_end(l):
        while l < last_level and width(l) == 1:
            l += 1
        return l

    launches, l = 0, first_level
    while l < last_level:
        if width(l) == 1 and chain_end(l) - l >= 4:
            l = chain_end(l)
        elif width(l) <= 64:
            e = l + 1
            while e < last_level and width(e) <= 64 and chain_end(e) - e < 4:
                e += 1
            l = e
        else:
            l += 1
        launches += 1
    return launches


def streams_in_multiply(mat, n, d):
    """Whether a multiply of ``mat`` with an [n, d] matrix is the one-launch multiply by subtrees (the Python
    layer's rule: after the single launch of small products, for matrices neither tiled nor with cut rows)."""
    return (mat.n_levels > 1 and not (mat.is_tiled() or mat.has_cut_rows()) and not mat._single_launch(n, d)
            and mat.stream_plan(d) is not None)


def walks_paths_in_multiply(mat, n, d):
    """Whether a multiply of ``mat`` with an [n, d] matrix ends in the one-launch path walk (the Python
    layer's rule: untiled, no cut rows, a shallow tree, a product within the path walk's size limit)."""
    return mat.n_levels > 1 and not (mat.is_tiled() or mat.has_cut_rows()) and mat._walks_paths(n, d)


def launches_per_multiply(mat, n, d, copies_x=True):
    """Kernel launches one multiply of ``mat`` with an [n, d] matrix issues, by the rules the Python layer
    applies: one for a small product on a shallow tree, one for the multiply by subtrees of a deep tree with
    short delta rows; else the copy of X (``copies_x``: short rows and
    small X are gathered in place) + the SpMM (+ adding the pieces of cut rows), then the walk -- one launch
    for the path walk of a shallow tree, the levels above the cut + one for the walk by subtrees, or the
    level-by-level plan."""
    tiled_or_cut = mat.is_tiled() or mat.has_cut_rows()
    if not tiled_or_cut and mat._single_launch(n, d):
        return 1
    if streams_in_multiply(mat, n, d):
        return 1
    launches = (2 if copies_x or tiled_or_cut else 1) + (1 if mat.has_cut_rows() else 0)
    if mat.n_levels <= 1:
        return launches
    lo = mat.level_off.tolist()
    if walks_paths_in_multiply(mat, n, d):
        return launches + 1
    if mat.walk_plan(d) is not None:
        return launches + level_launches(lo, 1, mat.walk_plan(d)["cut"] + 1) + 1
    return launches + level_launches(lo, 1, mat.n_levels)


def cpu_baseline_object(cpu):
    return {
        "value": cpu["cbm_ms_mean"], "unit": "ms", "cores": cpu["threads"], "kind": "port",
        "sample": f"{cpu['iters'][0]} full multiplies of the same workload after 1 warm-up ({cpu['spmm']} + OpenMP tree walk); "
                  f"1-thread legs: {cpu['iters_1t'][0]} multiplies after {cpu['warmup_1t']} warm-up",
        "cbm_ms_median": cpu["cbm_ms_median"], "csr_ms_mean": cpu["csr_ms_mean"], "csr_ms_median": cpu["csr_ms_median"],
        "cbm_walk_ms_mean": cpu["walk_ms_mean"],
        "cbm_ms_1t": cpu["cbm_ms_1t"], "csr_ms_1t": cpu["csr_ms_1t"],
    }


def gcn_epoch(args, torch, workload="c4"):
    """2-layer GCN forward + backward (cross-entropy) with CBM aggregation.  Model and protocol
    follow benchmark/parallel/benchmark_gcn_cpu.py:70-103 (warm-up + timed passes, one cbm_matrix
    shared by both layers), plus the backward pass the reference lacks."""
    import numpy as np

    from cbm4gnn_amd import graphs
    from cbm4gnn_amd.gcn import CBMGCNLayer, CSRGCNLayer, TwoLayerGCN, build_operator, csr_operator, tuned_gemms

    t0 = time.perf_counter()
    w = graphs.workload(workload, scale=args.scale)
    t_gen = time.perf_counter() - t0
    alpha = args.alpha if (args.alpha is not None and args.gcn) else w.alphas[-1]
    hidden, classes = 128, 41
    ei = torch.from_numpy(w.edge_index)
    t0 = time.perf_counter()
    op = build_operator(ei, alpha=alpha, normalized=True, builder=args.builder)
    t_build = time.perf_counter() - t0
    dev = torch.device("cuda:0")
    op.to(dev)
    n = w.n
    g = torch.Generator().manual_seed(0)
    x = torch.randn((n, w.d), generator=g).to(dev)
    labels = torch.randint(0, classes, (n,), generator=g).to(dev)
    m = op.col_multiplier
    vals = m[ei[0].long()] * m[ei[1].long()]
    fwd = csr_operator(torch.stack([ei[1], ei[0]]), n, vals, dev)       # rows = targets, as the CBM operator
    bwd = fwd if op.is_symmetric else csr_operator(ei, n, vals, dev)

    def make(kind):
        torch.manual_seed(0)
        if kind == "csr":
            return TwoLayerGCN(CSRGCNLayer(w.d, hidden, fwd, bwd), CSRGCNLayer(hidden, classes, fwd, bwd)).to(dev)
        fused = kind == "cbm_fused"
        return TwoLayerGCN(CBMGCNLayer(w.d, hidden, op, fused=fused, relu=fused),
                           CBMGCNLayer(hidden, classes, op, fused=fused), relu_between=not fused).to(dev)

    label_col = labels[:, None]

    def epoch(net):
        net.zero_grad(set_to_none=True)
        # mean cross entropy, written as log-softmax + gather: torch's nll_loss kernels reduce the 233k rows
        # in one workgroup (0.34 ms forward + 0.21 ms backward per epoch, for all three models alike)
        loss = -torch.log_softmax(net(x), dim=1).gather(1, label_col).mean()
        loss.backward()
        return loss

    def run(net):
        for _ in range(args.warmup):
            epoch(net)
        torch.cuda.synchronize()
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        for _ in range(args.steps):
            loss = epoch(net)
        b.record()
        torch.cuda.synchronize()
        return a.elapsed_time(b) / args.steps, float(loss.detach())

    nets = {k: make(k) for k in ("cbm_fused", "cbm_unfused", "csr")}
    # the dense GEMMs of all three models alike run on the library solution torch's TunableOp measures
    # fastest per shape (tuned during the warm-up epochs); --no-gemm-tuning leaves hipBLASLt's default pick
    with contextlib.ExitStack() as stack:
        if not args.no_gemm_tuning:
            try:
                stack.enter_context(tuned_gemms())
            except Exception as exc:                       # a torch build without TunableOp: default picks
                print(f"bench.py: GEMM tuning unavailable ({exc}); dense GEMMs on the default pick", file=sys.stderr)
                args.no_gemm_tuning = True
        res = {k: run(v) for k, v in nets.items()}
    # aggregation alone: the 4 multiplies of an epoch (d = hidden and d = classes, forward and backward)
    agg = 0.0
    per_width, roof = {}, {}
    tree_edges = n - int(op.level_off[1])
    for dd in (hidden, classes):
        h = torch.randn((n, dd), device=dev)
        o = torch.empty_like(h)
        _, t, _ = time_gpu(lambda: op._run_spmm_update(h, o, use_m=True), args.steps, args.warmup, torch)
        per_width[str(dd)] = t
        agg += 2 * t
        # the dominant kernel of that multiply alone
        _, spmm_ms, z, kernel = spmm_alone(op, h, True, args.steps, args.warmup, torch)
        b_spmm, _, _ = algorithmic_bytes(n, op.nnz, dd, 1, tree_edges, op.n_levels, op.nnz_a)
        roof[str(dd)] = roofline_of(w.name, alpha, dd, kernel, spmm_ms, b_spmm, compulsory_bytes(n, op.nnz, dd), args.scale)
        del h, o, z
    base = nets["csr"]
    grad_err = {k: max(float((p.grad - q.grad).abs().max() / q.grad.abs().max())
                       for p, q in zip(nets[k].parameters(), base.parameters())) for k in ("cbm_fused", "cbm_unfused")}
    ms = res["cbm_fused"][0]
    return {
        "workload": f"{w.name}: {w.note}", "nodes": n, "nnz_A": op.nnz_a, "nnz_delta": op.nnz, "alpha": alpha,
        "in": w.d, "hidden": hidden, "classes": classes, "tree_levels": op.n_levels, "scale": args.scale,
        "steps": args.steps, "warmup": args.warmup,
        "gcn_epoch_ms": ms, "gcn_epoch_ms_unfused_layers": res["cbm_unfused"][0], "gcn_epoch_ms_gpu_csr": res["csr"][0],
        "speedup_vs_gpu_csr": res["csr"][0] / ms, "compression_ratio": op.compression_ratio(),
        "aggregation_ms_per_epoch": agg, "aggregation_share": agg / ms, "multiply_ms_by_width": per_width,
        "roofline_by_width": roof,
        "loss": res["cbm_fused"][1], "loss_unfused_layers": res["cbm_unfused"][1], "loss_gpu_csr": res["csr"][1],
        "max_rel_weight_grad_diff_vs_gpu_csr": grad_err,
        "dense_gemms": ("hipBLASLt default pick" if args.no_gemm_tuning else
                        "library solution picked per shape by torch.cuda.tunable during warm-up (all three models)"),
        "host_s": {"generate": t_gen, "build_format": t_build, "build_phases": op.build_seconds},
    }


def gcn_epoch_bench(args):
    import torch
    r = gcn_epoch(args, torch, args.workload if args.workload != "c3" else "c4")
    print(json.dumps({
        "metric": "2-layer GCN epoch ms (forward + backward, CBM aggregation)", "value": r["gcn_epoch_ms"], "unit": "ms",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": r["gcn_epoch_ms"],
        "higher_is_better": False, "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {k: r[k] for k in ("workload", "nodes", "nnz_A", "nnz_delta", "alpha", "in", "hidden", "classes",
                                     "tree_levels", "scale")},
        **{k: v for k, v in r.items() if k not in ("workload", "nodes", "nnz_A", "nnz_delta", "alpha", "in", "hidden",
                                                   "classes", "tree_levels", "scale", "steps", "warmup")}}))


def alpha_sweep_bench(args):
    """CBM multiply per alpha on one graph (default: the dense-community workload c5, d = 512):
    compression ratio, tree depth and runtime per alpha, as alpha_searcher/spmm_cpu_parallel.py:84-124
    does on the CPU.  Prints one JSON line with a row per alpha."""
    import numpy as np
    import torch

    from cbm4gnn_amd import graphs
    from cbm4gnn_amd.cbm import DEFAULT_BATCH_ROWS, cbm_matrix, csr_spmm, schedule_rows

    w = graphs.workload(args.workload if args.workload != "c3" else "c5", scale=args.scale)
    d = args.d or w.d
    n = w.n
    ei = torch.from_numpy(w.edge_index)
    xd = w.features(0, d).cuda()
    yd = torch.empty_like(xd)
    m_np = torch.bincount(ei[0].long(), minlength=n).float().pow(-0.5).numpy() if w.normalized else None
    rp_np, col_np, val_np = csr_of(w.edge_index, n, m_np)
    rp, col = torch.from_numpy(rp_np).cuda(), torch.from_numpy(col_np).cuda()
    val = None if val_np is None else torch.from_numpy(val_np).cuda()
    ycsr = torch.empty_like(xd)
    sched = schedule_rows(rp, batch=DEFAULT_BATCH_ROWS).to(xd.device)
    _, csr_ms, _ = time_gpu(lambda: csr_spmm(rp, col, val, xd, ycsr, sched), args.steps, args.warmup, torch)
    rows = []
    alphas = [args.alpha] if args.alpha is not None else list(w.alphas)
    for alpha in alphas:
        t0 = time.perf_counter()
        mat = cbm_matrix(ei, None, alpha=alpha, normalized=w.normalized, builder=args.builder, max_levels=args.max_levels)
        t_build = time.perf_counter() - t0
        mat.to(xd.device)
        step = (lambda: mat.omp_mkl_csr_fused_spmm_update(xd, yd)) if w.normalized else (lambda: mat.omp_mkl_csr_spmm_update(xd, yd))
        _, ms, _ = time_gpu(step, args.steps, args.warmup, torch)
        zd = torch.empty_like(xd)
        _, spmm_ms, _ = time_gpu(lambda: mat._run_spmm(xd, zd, use_m=w.normalized, scale_roots=w.normalized), args.steps, args.warmup, torch)
        tree_edges = n - int(mat.level_off[1])
        b_spmm, b_prop, b_csr = algorithmic_bytes(n, mat.nnz, d, int(w.normalized), tree_edges, mat.n_levels, mat.nnz_a)
        step(); torch.cuda.synchronize()
        widths = np.diff(mat.level_off.numpy())
        rows.append({"alpha": alpha, "compression_ratio": mat.compression_ratio(), "nnz_delta": mat.nnz,
                     "tree_levels": mat.n_levels, "tree_edges": tree_edges,
                     "level_widths": {"first": widths[:12].tolist(),
                                      "histogram": {int(k): int(v) for k, v in zip(*np.unique(widths, return_counts=True))}},
                     "cbm_ms": ms, "delta_spmm_ms": spmm_ms,
                     "propagate_ms": ms - spmm_ms, "cbm_GBps": (b_spmm + b_prop) / ms / 1e6,
                     "speedup_vs_gpu_csr": csr_ms / ms, "build_s": t_build, "build_phases": mat.build_seconds,
                     "max_rel_err_vs_gpu_csr": float((yd - ycsr).abs().max() / ycsr.abs().max())})
        del mat
    print(json.dumps({
        "metric": "CBM SpMM alpha sweep", "unit": "ms", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": f"{w.name}: {w.note}", "nodes": n, "nnz_A": int(ei.size(1)), "d": d, "scale": args.scale,
                   "mean_degree": ei.size(1) / n},
        "gpu_csr_ms": csr_ms, "gpu_csr_GBps": algorithmic_bytes(n, 0, d, int(w.normalized), 0, 1, int(ei.size(1)))[2] / csr_ms / 1e6,
        "rows": rows}))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="c3")
    ap.add_argument("--alpha", type=int, default=None)
    ap.add_argument("--d", type=int, default=None)
    ap.add_argument("--scale", type=float, default=1.0)
    ap.add_argument("--no-cpu", action="store_true", help="skip the cpu_baseline leg")
    ap.add_argument("--threads", type=int, default=0,
                    help="threads of the multi-threaded cpu_baseline leg (default: all host cores; the reference's "
                         "benchmarks fix 16, benchmark/parallel/benchmark_spmm_cpu.py:2)")
    ap.add_argument("--only-multiply", action="store_true",
                    help="skip the gcn_epoch, other_workloads and gpu_vendor_csr sections of the default run")
    ap.add_argument("--max-levels", type=int, default=None,
                    help="depth limit of the arborescence (default: none, as the reference)")
    ap.add_argument("--builder", choices=("auto", "host", "gpu"), default="auto",
                    help="where the format builder computes its row intersections (same format either way)")
    ap.add_argument("--probe", action="store_true",
                    help="counter run: 3 multiplies and 3 plain device copies of X (known size, for scaling "
                         "FETCH_SIZE / WRITE_SIZE), no timing, no JSON")
    ap.add_argument("--sweep", action="store_true",
                    help="alpha sweep (default workload c5): compression ratio and runtime per alpha")
    ap.add_argument("--no-gemm-tuning", action="store_true",
                    help="GCN epoch: leave the dense GEMMs on hipBLASLt's default pick instead of the solution "
                         "torch's TunableOp measures fastest per shape (applies to all three models alike)")
    ap.add_argument("--gcn", action="store_true",
                    help="measure the 2-layer GCN forward+backward epoch (default workload c4) instead of the multiply")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: this build has no multi-GPU path (every box has one GPU); "
                 "run with --gpus 1")
    import numpy as np
    import torch

    if not torch.cuda.is_available():
        sys.exit("bench.py needs a HIP device")
    if args.gcn or args.sweep:
        return gcn_epoch_bench(args) if args.gcn else alpha_sweep_bench(args)

    from cbm4gnn_amd import graphs

    t0 = time.perf_counter()
    w = graphs.workload(args.workload, scale=args.scale)
    alpha = args.alpha if args.alpha is not None else w.alphas[-1]
    d = args.d or w.d
    t_gen = time.perf_counter() - t0
    if args.probe:
        from cbm4gnn_amd.cbm import cbm_matrix
        mat = cbm_matrix(torch.from_numpy(w.edge_index), None, alpha=alpha, normalized=w.normalized,
                         builder=args.builder, max_levels=args.max_levels)
        xd = w.features(0, d).cuda()
        yd = torch.empty_like(xd)
        step = (lambda: mat.omp_mkl_csr_fused_spmm_update(xd, yd)) if w.normalized else (lambda: mat.omp_mkl_csr_spmm_update(xd, yd))
        for _ in range(3):
            step()
        torch.cuda.synchronize()
        for _ in range(3):
            yd.copy_(xd)                                   # reads and writes n*d*4 bytes each
        torch.cuda.synchronize()
        print(f"probe: 3 multiplies, then 3 device copies of {xd.numel() * 4} bytes (read) + the same written; "
              f"kernels_sha256={kernel_source_hash()}")
        return

    row, ex = measure_multiply(w, alpha, d, args, torch, vendor=not args.only_multiply,
                               cpu=None if args.no_cpu else 20.0)
    mat = ex["mat"]
    n, nnz, n_edges = w.n, mat.nnz, mat.nnz_a
    b_spmm, b_prop, b_csr = ex["b"]
    span_ms = ex["span_ms"]
    out = {
        "metric": "CBM SpMM ms at d=%d" % d,
        "value": span_ms, "unit": "ms", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": span_ms, "higher_is_better": False, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": f"{w.name}: {w.note}", "nodes": n, "nnz_A": n_edges, "nnz_delta": nnz, "d": d,
                   "alpha": alpha, "normalized": bool(w.normalized), "tree_levels": mat.n_levels,
                   "tree_edges": ex["tree_edges"], "scale": args.scale},
        "ms_per_step_wall": ex["wall_ms"], "ms_per_step_median": ex["med_ms"],
        "cbm_GBps": (b_spmm + b_prop) / (span_ms * 1e-3) / 1e9,
        "cbm_frac_of_8TBps": (b_spmm + b_prop) / (span_ms * 1e-3) / 1e9 / HBM_PEAK_GBPS,
        "edges_x_features_per_s": n_edges * d / (span_ms * 1e-3),
        "compression_ratio": mat.compression_ratio(),
        "kernel_ms": row["kernel_ms"], "launches_per_multiply": row["launches_per_multiply"],
        "gpu_csr_ms": ex["csr_ms"], "gpu_csr_GBps": b_csr / (ex["csr_ms"] * 1e-3) / 1e9,
        "speedup_vs_gpu_csr": ex["csr_ms"] / span_ms,
        "flat_binary_ms": row["flat_binary_ms"], "speedup_from_compression": row["speedup_from_compression"],
        "gpu_vendor_csr": row.get("gpu_vendor_csr"),
        "max_rel_err_vs_gpu_csr": row["max_rel_err_vs_gpu_csr"],
        "max_rel_err_vs_cpu_fp64_rows": row["max_rel_err_vs_cpu_fp64_rows"],
        "roofline": row["roofline"],
        "host_s": {"generate": t_gen, "build_format": ex["t_build"], "builder": mat.builder, "build_phases": mat.build_seconds},
    }
    if "cpu_baseline" in row:
        out["cpu_baseline"] = row["cpu_baseline"]
        out["max_rel_err_vs_cpu_cbm"] = row["max_rel_err_vs_cpu_cbm"]
    if not args.only_multiply and args.workload == "c3" and args.scale == 1.0:
        del ex, mat
        torch.cuda.empty_cache()
        others = []
        short = argparse.Namespace(**{**vars(args), "steps": min(args.steps, 20), "warmup": min(args.warmup, 3)})
        # (workload, alpha, seconds of CPU legs or None): the CPU legs run where the tree exists -- on the
        # headline graph at alpha = 0, on both readings of the duplication graph, on the dense-community graph
        # on the deep-and-wide tree and on the union of cliques -- so that the reference's OpenMP walk is timed
        # where it walks
        plan = (("c3", 0, 10.0), ("c1", 0, 4.0), ("c2", 0, 8.0), ("c2", 8, None), ("c2b", 0, 6.0),
                ("c5", 0, 40.0), ("c6", 0, 12.0), ("c7", 0, 8.0))
        wk = None
        for name, a, cpu_s in plan:
            if wk is None or wk.name != name:
                wk = w if name == w.name else graphs.workload(name)
            r, e = measure_multiply(wk, a, wk.d, short, torch, cpu=None if args.no_cpu else cpu_s)
            del e
            others.append(r)
            torch.cuda.empty_cache()
        del wk
        out["other_workloads"] = others
        out["gcn_epoch"] = gcn_epoch(short, torch, "c4")
    print(json.dumps(out))


if __name__ == "__main__":
    main()
