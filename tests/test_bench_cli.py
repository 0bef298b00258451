"""bench.py's host-side pieces that need no GPU: the byte models behind the roofline figures, the
traffic records it reads from profiles/, and the command line's refusal of more than one GPU."""
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)

import bench  # noqa: E402


def test_gather_model_bytes_of_the_headline_workload():
    # 100,000 rows, 4,480,632 delta entries (= entries of A_hat: flat tree), d = 256, normalised:
    # row pointers + (index + coefficient) per entry + one 1024-byte row of X per entry + Y once
    n, nnz, d = 100_000, 4_480_632, 256
    b_spmm, b_prop, b_csr = bench.algorithmic_bytes(n, nnz, d, 1, 0, 1, nnz)
    assert b_spmm == 4 * 100_001 + 8 * nnz + 1024 * nnz + 1024 * n == 4_726_812_228
    assert b_prop == 0                      # no tree edge, no walk
    assert b_csr == b_spmm                  # delta = A_hat: the CSR baseline moves the same bytes
    # un-normalised: no coefficient word per entry
    assert bench.algorithmic_bytes(n, nnz, d, 0, 0, 1, nnz)[0] == b_spmm - 4 * nnz


def test_walk_bytes_count_three_rows_per_tree_edge():
    n, d, edges, levels = 1000, 64, 600, 5
    _, b_prop, _ = bench.algorithmic_bytes(n, 5000, d, 1, edges, levels, 9000)
    # parent + order per row, level offsets, m per row, and per tree edge: parent row read, row read, row written
    assert b_prop == 4 * (2 * n + levels + 1) + 4 * n + 4 * d * 3 * edges


def test_compulsory_bytes():
    assert bench.compulsory_bytes(100_000, 4_480_632, 256) == 223_922_528


def test_traffic_record_lookup():
    total, src, stale = bench.measured_traffic("c3", 16, 256)
    assert src is not None and src["file"].startswith("profiles/") and len(src["kernels_sha256"]) == 16
    if stale:                               # counters taken on another version of the kernels: no number
        assert total is None
    else:
        assert src["kernels_sha256"] == bench.kernel_source_hash()
        assert 1e9 < total < 1e10           # a gather launch of this workload moves about 2 GB
    assert bench.measured_traffic("no-such-workload", 0, 1) == (None, None, False)


def test_launch_count_follows_the_walk_plan():
    """Copy of X + SpMM, then the walk: one launch per wide level, one per run of narrow levels, one per
    chain of at least four single-row levels; one launch in all for a small product on a shallow tree; one
    more than the SpMM's two for a tree the path walk finishes in one launch."""
    import types
    import torch

    def fake(widths, tiled=False, cut=False, single=False, paths=False, subtrees=None, stream=False):
        lo = torch.tensor([0] + list(__import__("itertools").accumulate(widths)), dtype=torch.int32)
        return types.SimpleNamespace(level_off=lo, n_levels=len(widths), is_tiled=lambda: tiled, has_cut_rows=lambda: cut,
                                     _single_launch=lambda n, d: single, _walks_paths=lambda n, d: paths,
                                     walk_plan=lambda d: ({"cut": subtrees} if subtrees is not None else None),
                                     stream_plan=lambda d: ({"n_bins": 1} if stream else None))

    assert bench.launches_per_multiply(fake([500]), 500, 64) == 2                         # flat tree
    assert bench.launches_per_multiply(fake([500], cut=True), 500, 64) == 3               # + adding the pieces
    assert bench.launches_per_multiply(fake([500, 300, 200]), 1000, 64) == 4              # two wide levels
    assert bench.launches_per_multiply(fake([500, 300, 200], single=True), 1000, 64) == 1
    assert bench.launches_per_multiply(fake([500, 300, 200], paths=True), 1000, 64) == 3
    assert bench.launches_per_multiply(fake([500, 300, 200], paths=True, tiled=True), 1000, 64) == 4
    # wide, wide, narrow run of three, chain of five, narrow pair (a chain of two is not a chain)
    assert bench.launches_per_multiply(fake([900, 100, 70, 30, 20, 10, 1, 1, 1, 1, 1, 9, 1, 1]), 2000, 64) == 2 + 2 + 1 + 1 + 1
    # the walk by subtrees: the levels above its cut level by level, then one launch
    deep = [900, 100, 70, 30, 20, 10, 1, 1, 1, 1, 1, 9, 1, 1]
    assert bench.launches_per_multiply(fake(deep, subtrees=0), 2000, 64) == 2 + 1
    assert bench.launches_per_multiply(fake(deep, subtrees=2), 2000, 64) == 2 + 2 + 1
    assert bench.launches_per_multiply(fake(deep, subtrees=0, paths=True), 2000, 64) == 2 + 1      # the path walk asks first
    # the multiply by subtrees is one launch; small products and plan-based multiplies never ask for it
    assert bench.launches_per_multiply(fake(deep, subtrees=0, stream=True), 2000, 64) == 1
    assert bench.launches_per_multiply(fake(deep, subtrees=0, stream=True, tiled=True), 2000, 64) == 2 + 1
    assert bench.launches_per_multiply(fake([500], stream=True), 500, 64) == 2
    # short rows / a small X are gathered in place: no copy launch
    assert bench.launches_per_multiply(fake([500]), 500, 64, copies_x=False) == 1
    assert bench.launches_per_multiply(fake([500, 300, 200], paths=True), 1000, 64, copies_x=False) == 2
    assert bench.launches_per_multiply(fake(deep, subtrees=0), 2000, 64, copies_x=False) == 1 + 1
    assert bench.launches_per_multiply(fake([500], cut=True), 500, 64, copies_x=False) == 3       # pieces always go through the copy
    assert bench.walks_paths_in_multiply(fake([500, 300, 200], paths=True), 1000, 64)
    assert not bench.walks_paths_in_multiply(fake([500, 300, 200], paths=True, tiled=True), 1000, 64)
    assert not bench.walks_paths_in_multiply(fake([500], paths=True), 500, 64)
    # a lone narrow level between wide ones is a launch of its own
    assert bench.launches_per_multiply(fake([900, 100, 7, 100]), 2000, 64) == 2 + 3


def test_more_than_one_gpu_is_refused():
    p = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True,
                       timeout=120)
    assert p.returncode != 0
    assert "--gpus 1" in (p.stdout + p.stderr)
