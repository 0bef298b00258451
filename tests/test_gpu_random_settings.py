"""Random graphs, widths and settings through ``cbm_matrix`` on the GPU, bit for bit against the oracle
evaluated in the order the chosen kernels sum in (the helpers of test_gpu_parity compose that order)."""
import numpy as np
import pytest
import torch

import test_gpu_parity as parity
from cbm4gnn_amd import graphs
from cbm4gnn_amd.cbm import cbm_matrix

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("seed", [11, 12])
def test_random_settings_against_oracle(orc, seed, monkeypatch):
    """40 cases per seed: SBM / Erdos-Renyi / hub-row graphs of 7 .. 3,000 nodes, plain and normalised,
    alpha 0 .. huge, widths 1 .. 258, with and without the LDS tiling, the depth limit, rows cut by
    length and at column-block boundaries, the one-launch path walk and the one-launch product on and off, the
    walk by subtrees off / by estimate / forced (with a forced cut), the one-launch multiply by subtrees off / by
    estimate / forced, short rows in batches of every limit; also staircase graphs (deep and wide trees)."""
    if not torch.cuda.is_available():
        pytest.skip("no HIP device")
    rng = np.random.default_rng(seed)
    from cbm4gnn_amd import cbm as cbm_mod
    for case in range(40):
        monkeypatch.setattr(cbm_mod, "_SMALL_X_BYTES", int(rng.choice([0, 8 << 20])))     # both copy rules (the helpers read it too)
        n = int(rng.choice([7, 65, 300, 700, 1500, 3000]))
        kind = str(rng.choice(["sbm", "er", "hub", "stairs"]))
        if kind == "stairs":
            ei = graphs.staircases(int(rng.choice([3, 12])), int(rng.choice([5, 40])), 4, float(rng.choice([0.0, 2.0])), seed=case)
            n = int(ei.max()) + 1
        elif kind == "sbm":
            ei = graphs.sbm(n, max(1, n // 100), float(rng.choice([0.2, 0.6])), float(rng.choice([0.002, 0.02])), seed=case)
        elif kind == "er":
            ei = graphs.erdos_renyi(n, float(rng.choice([0.01, 0.05, 0.3])) if n <= 700 else 0.01, case)
        else:
            n = max(n, 300)
            ei = parity.hub_graph(n, 4, seed=case)
        ei = graphs.add_self_loops(ei, n)
        normalized = bool(rng.integers(2))
        alpha = int(rng.choice([0, 1, 4, 10 ** 6]))
        d = int(rng.choice([1, 5, 16, 33, 41, 64, 100, 128, 200, 258]))
        tiling = str(rng.choice(["off", "on"])) if n >= 1500 else "off"
        max_levels = None if rng.integers(2) else int(rng.choice([1, 2, 3, 16]))
        mat = cbm_matrix(torch.from_numpy(ei), None, alpha=alpha, normalized=normalized, tiling=tiling, max_levels=max_levels)
        mat.tile_min_block_entries = int(rng.choice([500, 2000]))
        mat.split_chunk = int(rng.choice([0, 64, 2048]))
        mat.column_blocks = int(rng.choice([1, 1, 2, 3]))
        mat.path_walk_max_bytes = int(rng.choice([0, 64 << 20]))
        mat.single_launch_max_bytes = int(rng.choice([0, 4 << 20]))
        mat.batch_rows = int(rng.choice([0, 8, 32, 64]))
        walk = ["off", "auto", "on", 0, 2][int(rng.integers(5))]
        mat.subtree_walk = walk
        mat.stream_multiply = ["off", "auto", "on"][int(rng.integers(3))]
        x = rng.standard_normal((n, d)).astype(np.float32)
        parity.say("random settings", seed, case, kind, n, mat.nnz, mat.n_levels, normalized, alpha, d, tiling, mat.is_tiled(),
                   mat.has_cut_rows(), mat.split_chunk, mat.column_blocks, max_levels, mat.path_walk_max_bytes,
                   mat.single_launch_max_bytes, "batch", mat.batch_rows, "walk", walk, "stream", mat.stream_multiply)
        got = parity.gpu_product(mat, x, normalized)
        assert np.array_equal(got, parity.oracle_product(orc, mat, ei, n, x, normalized)), (seed, case)
        assert orc.max_rel_err(got, orc.dense_product(ei, n, x, normalized)) <= parity.TOL_CBM, (seed, case)
