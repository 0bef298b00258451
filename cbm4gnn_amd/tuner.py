"""Pick the CBM pruning parameter ``alpha`` by measurement on the GPU.

GPU analogue of the reference's alpha searcher (``alpha_searcher/spmm_cpu_parallel.py:84-124``):
for every candidate alpha build the format, time the multiply (median over per-call HIP events,
the reference takes the median of 50 ``perf_counter`` intervals) and check it against the plain
CSR product of the same matrix (the reference asserts ``atol=rtol=1e-2``, ``:120``; here the
tighter max-relative 1e-3 of this library's parity bar).  The trade-off differs from the CPU's: a
deeper tree costs extra kernel launches rather than idle threads, so small alphas win whenever
they compress at all.
"""
from __future__ import annotations

import statistics

import numpy as np
import torch

from .cbm import DEFAULT_BATCH_ROWS, cbm_matrix, csr_spmm, schedule_rows

__all__ = ["time_calls", "tune_alpha", "DEFAULT_ALPHAS"]

DEFAULT_ALPHAS = (0, 1, 2, 4, 8, 16, 32, 64, 128)          # spmm_cpu_parallel.py:18


def time_calls(fn, iters: int = 50, warmup: int = 5):
    """(median ms, mean ms over the whole loop) of ``fn`` on the current HIP stream."""
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    starts = [torch.cuda.Event(enable_timing=True) for _ in range(iters)]
    ends = [torch.cuda.Event(enable_timing=True) for _ in range(iters)]
    for s, e in zip(starts, ends):
        s.record()
        fn()
        e.record()
    torch.cuda.synchronize()
    return statistics.median(s.elapsed_time(e) for s, e in zip(starts, ends)), starts[0].elapsed_time(ends[-1]) / iters


def tune_alpha(edge_index, d: int, alphas=DEFAULT_ALPHAS, normalized: bool = False, iters: int = 50,
               warmup: int = 5, device="cuda", seed: int = 0, tolerance: float = 1e-3, max_levels=(None,),
               x=None, reference=None, reference_tolerance: float = 1e-4):
    """Returns ``(best_alpha, rows)``; ``rows`` has one dict per (alpha, depth limit) tried
    (compression ratio, tree depth, ms, speed-up over the GPU CSR baseline); the best row is marked
    ``"best": True``.  Ties go to the larger alpha (shallower tree).

    ``max_levels``: depth limits to try for every alpha (``None`` = no limit, the reference's
    trees).  On the GPU every tree level is a dependent launch, so cutting deep, thin levels can pay
    where alpha cannot reach them: 12 000-row duplication graph, d = 128: 99 us unlimited, 89 us at
    4 levels; 132 534-row clique graph with a 2 000-level chain, d = 512: 5.80 -> 5.54 ms at 8.

    ``x``: the [N, d] fp32 features to multiply (default: N(0,1) from ``seed``).  ``reference``: an
    independently computed product of the same matrix with ``x`` ([N, d] array, e.g. a dense fp64 one);
    every candidate is then also held against it, max-relative error at most ``reference_tolerance`` --
    the reference's searcher asserts each candidate against a product computed another way
    (``spmm_cpu_parallel.py:116-124``), and the GPU CSR baseline alone shares this library's kernels."""
    ei = torch.as_tensor(edge_index).to("cpu", torch.int32)
    n = int(ei.max()) + 1
    dev = torch.device(device)
    if x is None:
        x = torch.randn((n, d), generator=torch.Generator().manual_seed(seed))
    x = torch.as_tensor(x, dtype=torch.float32).to(dev).contiguous()
    if tuple(x.shape) != (n, d):
        raise ValueError(f"x must be [{n}, {d}], got {tuple(x.shape)}")
    want = None
    if reference is not None:
        want = torch.as_tensor(reference).to(dev, torch.float64)
        if tuple(want.shape) != (n, d):
            raise ValueError(f"reference must be [{n}, {d}], got {tuple(want.shape)}")
        want_scale = float(want.abs().max())
    y = torch.empty_like(x)
    key = ei[0].to(torch.int64) * n + ei[1].to(torch.int64)
    order = torch.argsort(key)
    rowptr = torch.zeros(n + 1, dtype=torch.int64)
    rowptr[1:] = torch.cumsum(torch.bincount(ei[0].to(torch.int64), minlength=n), 0)
    rowptr = rowptr.to(torch.int32)
    col = ei[1][order].contiguous()
    val = None
    if normalized:
        m = torch.bincount(ei[0].to(torch.int64), minlength=n).to(torch.float32).pow(-0.5)
        val = (m[ei[0][order].long()] * m[col.long()]).to(dev)
    rowptr_d, col_d, sched_d = rowptr.to(dev), col.to(dev), schedule_rows(rowptr, batch=DEFAULT_BATCH_ROWS).to(dev)
    y_csr = torch.empty_like(x)
    csr_ms, _ = time_calls(lambda: csr_spmm(rowptr_d, col_d, val, x, y_csr, sched_d), iters, warmup)
    scale = float(y_csr.abs().max())
    rows = []
    for alpha, limit in ((a, l) for a in alphas for l in max_levels):
        mat = cbm_matrix(ei, None, alpha=alpha, normalized=normalized, max_levels=limit)
        mat.to(dev)
        step = (lambda: mat.omp_mkl_csr_fused_spmm_update(x, y)) if normalized else (lambda: mat.omp_mkl_csr_spmm_update(x, y))
        ms, _ = time_calls(step, iters, warmup)
        err = float((y - y_csr).abs().max()) / scale if scale > 0 else 0.0
        if not err <= tolerance:
            raise AssertionError(f"alpha={alpha}: CBM product differs from the CSR product by {err:.2e}")
        err_ref = None
        if want is not None:
            err_ref = float((y.to(torch.float64) - want).abs().max()) / want_scale if want_scale > 0 else float(y.abs().max())
            if not err_ref <= reference_tolerance:
                raise AssertionError(f"alpha={alpha}: CBM product differs from the reference product by {err_ref:.2e}")
        rows.append({"alpha": int(alpha), "max_levels": limit, "compression_ratio": mat.compression_ratio(), "nnz_delta": mat.nnz,
                     "tree_levels": mat.n_levels, "cbm_ms": ms, "gpu_csr_ms": csr_ms, "speedup_vs_gpu_csr": csr_ms / ms,
                     "max_rel_err_vs_gpu_csr": err, "max_rel_err_vs_reference": err_ref, "n_candidates": mat.n_candidates,
                     "build_seconds": mat.build_seconds})
        del mat
    best = min(rows, key=lambda r: (round(r["cbm_ms"] / rows[0]["cbm_ms"], 2), -r["alpha"]))
    for r in rows:
        r["best"] = r is best
    return best["alpha"], rows
