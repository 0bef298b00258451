#!/usr/bin/env python3
"""Benchmark of the CBM multiply on one MI355X.

    python bench.py [--gpus 1] [--steps 50] [--warmup 5] [--workload c3] [--alpha 16] [--d 256]

A "step" is one CBM multiply  Y = A_hat X  (delta SpMM + tree propagation through the C ABI)
on fixed device buffers; the format is built once, outside the timed region, as in the
reference's protocol (``benchmark/parallel/benchmark_spmm_cpu.py:119-151``: 50 timed calls on
fixed x, y).  Default workload: the 100k-node Chung-Lu + cliques graph, GCN-normalised, alpha=16,
feature width 256.  Prints ONE JSON line.

The ``cpu_baseline`` leg times the reference-style CPU path on the host cores of the same box:
MKL ``mkl_sparse_s_mm`` (reached through torch's libtorch_cpu.so, handle re-created per call
like the reference) followed by the OpenMP tree walk of the CPU oracle.
"""
from __future__ import annotations

import argparse
import json
import os
import statistics
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0

# HBM-side bytes per launch of the dominant kernel, from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE
# runs of `bench.py --probe` scaled by a plain copy of known size (FETCH_SIZE x 2.00, WRITE_SIZE
# x 1.00 on this part); keyed by (workload, alpha, d).  Counters cannot be read from inside this
# process, so a configuration that was not profiled reports null.
MEASURED_TRAFFIC_BYTES = {("c3", 16, 256): 2.32e9 + 0.1024e9}


def algorithmic_bytes(n, nnz, d, norm, tree_edges, levels, n_edges_a):
    """Bytes one multiply must move under the gather model (no reuse of X rows assumed)."""
    b_spmm = 4 * (n + 1) + 4 * nnz * (1 + norm) + 4 * d * nnz + 4 * d * n
    b_prop = (4 * (2 * n + levels + 1) + 4 * n * norm + 4 * d * 3 * tree_edges) if tree_edges else 0
    b_csr = 4 * (n + 1) + 4 * n_edges_a * (1 + norm) + 4 * d * n_edges_a + 4 * d * n
    return b_spmm, b_prop, b_csr


def time_gpu(fn, steps, warmup, torch):
    """(mean ms per step over the bracketed loop, median ms of per-call events)."""
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    starts = [torch.cuda.Event(enable_timing=True) for _ in range(steps)]
    ends = [torch.cuda.Event(enable_timing=True) for _ in range(steps)]
    t0 = time.perf_counter()
    for i in range(steps):
        starts[i].record()
        fn()
        ends[i].record()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3 / steps
    per_call = [s.elapsed_time(e) for s, e in zip(starts, ends)]
    span_ms = starts[0].elapsed_time(ends[-1]) / steps
    return wall_ms, span_ms, statistics.median(per_call)


def cpu_baseline(w, mat, x, budget_s=20.0, max_iters=50):
    """Reference-style CPU CBM and CPU CSR multiplies on this host (MKL SpMM + OpenMP walk)."""
    import numpy as np
    from oracle import cbm_oracle as orc

    n, d = x.shape
    threads = orc.max_threads()
    ei = w.edge_index
    m = orc.col_multiplier(ei, n) if w.normalized else None
    col, sign = mat.columns()
    col = col.numpy().astype(np.int32)
    val = (sign.numpy() * (m[col] if m is not None else 1.0)).astype(np.float32)
    rp = mat.rowptr.numpy()
    rb, re = np.ascontiguousarray(rp[:-1]), np.ascontiguousarray(rp[1:])
    mst_row, mst_col = mat.mst_row.numpy(), mat.mst_col.numpy()
    order = np.lexsort((ei[1], ei[0]))
    arp = np.concatenate([[0], np.cumsum(np.bincount(ei[0], minlength=n))]).astype(np.int32)
    arb, are = np.ascontiguousarray(arp[:-1]), np.ascontiguousarray(arp[1:])
    acol = np.ascontiguousarray(ei[1][order].astype(np.int32))
    aval = ((m[ei[0][order]] * m[acol]) if m is not None else np.ones(acol.shape[0])).astype(np.float32)
    y = np.empty((n, d), np.float32)
    use_mkl = orc.mkl() is not None

    def spmm(b, e, c, v):
        if use_mkl:
            orc.mkl_csr_spmm(b, e, c, v, x, y)
        else:
            y[:] = orc.csr_spmm(np.concatenate([b, e[-1:]]), c, v, x, threads)

    def cbm_call():
        spmm(rb, re, col, val)
        if m is None:
            orc.update_plain(mst_row, mst_col, y, threads)
        else:
            orc.update_fused(mst_row, mst_col, m, y, threads)

    def csr_call():
        spmm(arb, are, acol, aval)

    def run(fn):
        fn()                                              # 1 warm-up, as the reference
        ts = []
        t_end = time.perf_counter() + budget_s / 2
        while len(ts) < max_iters and time.perf_counter() < t_end:
            t = time.perf_counter(); fn(); ts.append((time.perf_counter() - t) * 1e3)
        return ts

    t_cbm = run(cbm_call)
    y_cbm = y.copy()
    t_csr = run(csr_call)
    return {
        "cbm_ms_mean": statistics.mean(t_cbm), "cbm_ms_median": statistics.median(t_cbm),
        "csr_ms_mean": statistics.mean(t_csr), "csr_ms_median": statistics.median(t_csr),
        "iters": [len(t_cbm), len(t_csr)], "threads": threads,
        "spmm": "mkl_sparse_s_mm via libtorch_cpu.so" if use_mkl else "hand OpenMP CSR SpMM (non-MKL stand-in)",
    }, y_cbm


def gcn_epoch_bench(args):
    """2-layer GCN forward + backward (cross-entropy) with CBM aggregation; prints one JSON line.
    Model and protocol follow benchmark/parallel/benchmark_gcn_cpu.py:70-103 (3 warm-up + 10 timed
    passes, one cbm_matrix shared by both layers), plus the backward pass the reference lacks."""
    import numpy as np
    import torch

    from cbm4gnn_amd import graphs
    from cbm4gnn_amd.gcn import CBMGCNLayer, CSRGCNLayer, TwoLayerGCN, build_operator, csr_operator

    t0 = time.perf_counter()
    w = graphs.workload(args.workload if args.workload != "c3" else "c4", scale=args.scale)
    t_gen = time.perf_counter() - t0
    alpha = args.alpha if args.alpha is not None else w.alphas[-1]
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
    torch.manual_seed(0)
    model = TwoLayerGCN(CBMGCNLayer(w.d, hidden, op), CBMGCNLayer(hidden, classes, op)).to(dev)
    m = op.col_multiplier
    vals = m[ei[0].long()] * m[ei[1].long()]
    fwd = csr_operator(torch.stack([ei[1], ei[0]]), n, vals, dev)       # rows = targets, as the CBM operator
    bwd = fwd if op.is_symmetric else csr_operator(ei, n, vals, dev)
    torch.manual_seed(0)
    base = TwoLayerGCN(CSRGCNLayer(w.d, hidden, fwd, bwd), CSRGCNLayer(hidden, classes, fwd, bwd)).to(dev)

    def epoch(net):
        net.zero_grad(set_to_none=True)
        loss = torch.nn.functional.cross_entropy(net(x), labels)
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
        return a.elapsed_time(b) / args.steps, float(loss)

    ms_cbm, loss_cbm = run(model)
    ms_csr, loss_csr = run(base)
    # aggregation alone: the 4 multiplies of an epoch (d = hidden and d = classes, forward and backward)
    agg = 0.0
    for dd in (hidden, classes):
        h = torch.randn((n, dd), device=dev)
        o = torch.empty_like(h)
        _, t, _ = time_gpu(lambda: op._run_spmm_update(h, o, use_m=True), args.steps, args.warmup, torch)
        agg += 2 * t
    grad_err = max(float((p.grad - q.grad).abs().max() / q.grad.abs().max())
                   for p, q in zip(model.parameters(), base.parameters()))
    print(json.dumps({
        "metric": "2-layer GCN epoch ms (forward + backward, CBM aggregation)", "value": ms_cbm, "unit": "ms",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": ms_cbm, "higher_is_better": False,
        "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": f"{w.name}: {w.note}", "nodes": n, "nnz_A": op.nnz_a, "nnz_delta": op.nnz,
                   "alpha": alpha, "in": w.d, "hidden": hidden, "classes": classes, "tree_levels": op.n_levels,
                   "scale": args.scale},
        "compression_ratio": op.compression_ratio(), "gcn_epoch_ms_gpu_csr": ms_csr, "speedup_vs_gpu_csr": ms_csr / ms_cbm,
        "aggregation_ms_per_epoch": agg, "aggregation_share": agg / ms_cbm,
        "loss": loss_cbm, "loss_gpu_csr": loss_csr, "max_rel_weight_grad_diff_vs_gpu_csr": grad_err,
        "host_s": {"generate": t_gen, "build_format": t_build, "build_phases": op.build_seconds},
    }))


def alpha_sweep_bench(args):
    """CBM multiply per alpha on one graph (default: the dense-community workload c5, d = 512):
    compression ratio, tree depth and runtime per alpha, as alpha_searcher/spmm_cpu_parallel.py:84-124
    does on the CPU.  Prints one JSON line with a row per alpha."""
    import numpy as np
    import torch

    from cbm4gnn_amd import graphs
    from cbm4gnn_amd.cbm import cbm_matrix, csr_spmm, schedule_rows

    w = graphs.workload(args.workload if args.workload != "c3" else "c5", scale=args.scale)
    d = args.d or w.d
    n = w.n
    ei = torch.from_numpy(w.edge_index)
    xd = w.features(0, d).cuda()
    yd = torch.empty_like(xd)
    order = np.lexsort((w.edge_index[1], w.edge_index[0]))
    rp = torch.from_numpy(np.concatenate([[0], np.cumsum(np.bincount(w.edge_index[0], minlength=n))]).astype(np.int32)).cuda()
    col = torch.from_numpy(w.edge_index[1][order].astype(np.int32)).cuda()
    val = None
    if w.normalized:
        m = torch.bincount(ei[0].long(), minlength=n).float().pow(-0.5)
        val = (m[torch.from_numpy(w.edge_index[0][order].astype(np.int64))] * m[torch.from_numpy(w.edge_index[1][order].astype(np.int64))]).cuda()
    ycsr = torch.empty_like(xd)
    sched = schedule_rows(rp).to(xd.device)
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
        rows.append({"alpha": alpha, "compression_ratio": mat.compression_ratio(), "nnz_delta": mat.nnz,
                     "tree_levels": mat.n_levels, "tree_edges": tree_edges,
                     "level_widths": {"first": np.diff(mat.level_off.numpy())[:12].tolist(),
                                      "histogram": {int(k): int(v) for k, v in zip(*np.unique(np.diff(mat.level_off.numpy()), return_counts=True))} if mat.n_levels <= 64 or True else None},
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
    ap.add_argument("--max-levels", type=int, default=None,
                    help="depth limit of the arborescence (default: none, as the reference)")
    ap.add_argument("--builder", choices=("auto", "host", "gpu"), default="auto",
                    help="where the format builder computes its row intersections (same format either way)")
    ap.add_argument("--probe", action="store_true",
                    help="counter run: 3 multiplies and 3 plain device copies of X (known size, for scaling "
                         "FETCH_SIZE / WRITE_SIZE), no timing, no JSON")
    ap.add_argument("--sweep", action="store_true",
                    help="alpha sweep (default workload c5): compression ratio and runtime per alpha")
    ap.add_argument("--gcn", action="store_true",
                    help="measure the 2-layer GCN forward+backward epoch (default workload c4) instead of the multiply")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: this build has no multi-GPU path (every box has one GPU); "
                 "run with --gpus 1")
    if args.gcn or args.sweep:
        import torch
        if not torch.cuda.is_available():
            sys.exit("bench.py needs a HIP device")
        return gcn_epoch_bench(args) if args.gcn else alpha_sweep_bench(args)

    import numpy as np
    import torch

    from cbm4gnn_amd import graphs
    from cbm4gnn_amd.cbm import cbm_matrix, csr_spmm, relayout_slabs, schedule_rows

    if not torch.cuda.is_available():
        sys.exit("bench.py needs a HIP device")
    t0 = time.perf_counter()
    w = graphs.workload(args.workload, scale=args.scale)
    alpha = args.alpha if args.alpha is not None else w.alphas[-1]
    d = args.d or w.d
    t_gen = time.perf_counter() - t0
    t0 = time.perf_counter()
    mat = cbm_matrix(torch.from_numpy(w.edge_index), None, alpha=alpha, normalized=w.normalized, builder=args.builder, max_levels=args.max_levels)
    t_build = time.perf_counter() - t0
    n, nnz, n_edges = w.n, mat.nnz, mat.nnz_a
    norm = int(w.normalized)
    tree_edges = n - int(mat.level_off[1])
    x = w.features(0, d)
    xd = x.cuda()
    yd = torch.empty_like(xd)
    mat.to(xd.device)

    step = (lambda: mat.omp_mkl_csr_fused_spmm_update(xd, yd)) if w.normalized else (lambda: mat.omp_mkl_csr_spmm_update(xd, yd))
    if args.probe:
        for _ in range(3):
            step()
        torch.cuda.synchronize()
        for _ in range(3):
            yd.copy_(xd)                                   # reads and writes n*d*4 bytes each
        torch.cuda.synchronize()
        print(f"probe: 3 multiplies, then 3 device copies of {xd.numel() * 4} bytes (read) + the same written")
        return
    wall_ms, span_ms, med_ms = time_gpu(step, args.steps, args.warmup, torch)

    # the dominant kernel alone (delta SpMM gather), same launch as inside the step; where the step
    # first copies X slab-major, that copy is made once here and timed on its own
    zd = torch.empty_like(xd)
    from cbm4gnn_amd.cbm import _wants_workspace
    ws = relayout_slabs(xd) if (mat.relayout and _wants_workspace(xd, zd, nnz)) else None
    relayout_ms = 0.0
    if ws is not None:
        _, relayout_ms, _ = time_gpu(lambda: relayout_slabs(xd), args.steps, args.warmup, torch)
    spmm_only = lambda: mat._run_spmm(xd, zd, use_m=w.normalized, scale_roots=w.normalized, workspace=ws,
                                      workspace_ready=ws is not None)
    _, spmm_ms, _ = time_gpu(spmm_only, args.steps, args.warmup, torch)
    prop_ms = 0.0
    if tree_edges:
        prop_only = lambda: mat._run_propagate(zd, use_m=w.normalized)
        _, prop_ms, _ = time_gpu(prop_only, args.steps, args.warmup, torch)

    # hand-written GPU CSR baseline on A_hat (explicit values when normalised)
    ei = w.edge_index
    order = np.lexsort((ei[1], ei[0]))
    rp = torch.from_numpy(np.concatenate([[0], np.cumsum(np.bincount(ei[0], minlength=n))]).astype(np.int32)).cuda()
    col = torch.from_numpy(ei[1][order].astype(np.int32)).cuda()
    val = None
    if w.normalized:
        m = mat.col_multiplier
        val = (m[torch.from_numpy(ei[0][order].astype(np.int64))] * m[torch.from_numpy(ei[1][order].astype(np.int64))]).cuda()
    ycsr = torch.empty_like(xd)
    csr_sched = schedule_rows(rp).to(xd.device)          # the baseline gets the same row scheduling
    _, csr_ms, _ = time_gpu(lambda: csr_spmm(rp, col, val, xd, ycsr, csr_sched), args.steps, args.warmup, torch)
    step()
    torch.cuda.synchronize()
    err_vs_csr = float((yd - ycsr).abs().max() / ycsr.abs().max())

    b_spmm, b_prop, b_csr = algorithmic_bytes(n, nnz, d, norm, tree_edges, mat.n_levels, n_edges)
    achieved = b_spmm / (spmm_ms * 1e-3) / 1e9
    out = {
        "metric": "CBM SpMM ms at d=%d" % d,
        "value": span_ms, "unit": "ms", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": span_ms, "higher_is_better": False, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": f"{w.name}: {w.note}", "nodes": n, "nnz_A": n_edges, "nnz_delta": nnz, "d": d,
                   "alpha": alpha, "normalized": bool(w.normalized), "tree_levels": mat.n_levels,
                   "tree_edges": tree_edges, "scale": args.scale},
        "ms_per_step_wall": wall_ms, "ms_per_step_median": med_ms,
        "cbm_GBps": (b_spmm + b_prop) / (span_ms * 1e-3) / 1e9,
        "cbm_frac_of_8TBps": (b_spmm + b_prop) / (span_ms * 1e-3) / 1e9 / HBM_PEAK_GBPS,
        "edges_x_features_per_s": n_edges * d / (span_ms * 1e-3),
        "compression_ratio": mat.compression_ratio(),
        "kernel_ms": {"relayout_slabs": relayout_ms, "delta_spmm": spmm_ms, "propagate": prop_ms},
        "gpu_csr_ms": csr_ms, "gpu_csr_GBps": b_csr / (csr_ms * 1e-3) / 1e9, "speedup_vs_gpu_csr": csr_ms / span_ms,
        "max_rel_err_vs_gpu_csr": err_vs_csr,
        "roofline": {"bound": "hbm", "kernel": "spmm_slab_per_xcd" if (ws is not None or d % 32 == 0) else "spmm_wave_per_row", "achieved": achieved, "peak": HBM_PEAK_GBPS,
                     "unit": "GB/s", "frac": achieved / HBM_PEAK_GBPS,
                     "traffic": MEASURED_TRAFFIC_BYTES.get((w.name, alpha, d)) if args.scale == 1.0 else None,
                     "algorithmic_bytes": b_spmm, "avg_launch_ms": spmm_ms},
        "host_s": {"generate": t_gen, "build_format": t_build, "builder": mat.builder, "build_phases": mat.build_seconds},
    }
    if not args.no_cpu:
        cpu, y_cpu = cpu_baseline(w, mat, x.numpy())
        out["cpu_baseline"] = {
            "value": cpu["cbm_ms_mean"], "unit": "ms", "cores": cpu["threads"], "kind": "port",
            "sample": f"{cpu['iters'][0]} full multiplies of the same workload after 1 warm-up ({cpu['spmm']} + OpenMP tree walk)",
            "cbm_ms_median": cpu["cbm_ms_median"], "csr_ms_mean": cpu["csr_ms_mean"], "csr_ms_median": cpu["csr_ms_median"],
        }
        got = yd.cpu().numpy()
        out["max_rel_err_vs_cpu_cbm"] = float(np.abs(got - y_cpu).max() / np.abs(y_cpu).max())
    print(json.dumps(out))


if __name__ == "__main__":
    main()
