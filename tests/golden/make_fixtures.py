"""Writes the small golden fixtures of this directory.

The reference ships no golden vectors: its tests draw a fresh unseeded Erdos-Renyi graph on
every run and compare the CBM product with ``sparse_coo_tensor(A) @ x``
(``tests/test_matmul_correctness.py:30-61``, n=25, p=0.5, d=10, integer features, alpha=3).
These fixtures freeze that same experiment for a few seeds: the edge list, the integer feature
matrix and the products computed here in dense fp64 NumPy -- nothing below imports this
repository's kernels or oracle, so the expected values are independent of both.

    python tests/golden/make_fixtures.py
"""
import json
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from cbm4gnn_amd import graphs  # noqa: E402  (generators only)


def er_case(n, p, d, seed, self_loops):
    ei = graphs.erdos_renyi(n, p, seed)
    if self_loops:
        ei = graphs.add_self_loops(ei, n)
    rng = np.random.default_rng(1000 + seed)
    x = rng.integers(0, 10, size=(n, d)).astype(np.float32)
    a = np.zeros((n, n), np.float64)
    a[ei[0], ei[1]] = 1.0
    deg = a.sum(axis=1)
    m = deg ** -0.5
    return {
        "edge_index": ei.astype(np.int32), "x": x,
        "ax": a @ x.astype(np.float64),
        "ax_normalized": (m[:, None] * a * m[None, :]) @ x.astype(np.float64),
        "row_degree": deg.astype(np.int64),
    }


def main():
    cases = {}
    for seed, (n, p, d, loops) in enumerate([(25, 0.5, 10, False), (25, 0.75, 10, False), (25, 0.5, 10, True),
                                             (40, 0.3, 41, True), (64, 0.9, 7, False)]):
        c = er_case(n, p, d, seed, loops)
        for k, v in c.items():
            cases[f"case{seed}_{k}"] = v
    np.savez_compressed(os.path.join(HERE, "er_products.npz"), **cases)
    hashes = {}
    for name in ("c1", "c2", "c2b", "c3", "c6", "c7"):
        w = graphs.workload(name)
        hashes[name] = {"n": int(w.n), "edges": int(w.edge_index.shape[1]), "sha256": graphs.edge_hash(w.edge_index)}
    with open(os.path.join(HERE, "graph_hashes.json"), "w") as f:
        json.dump(hashes, f, indent=1, sort_keys=True)
    print("wrote", len(cases), "arrays and", len(hashes), "graph hashes")


if __name__ == "__main__":
    main()
