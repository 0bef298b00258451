"""Deterministic synthetic graphs for the CBM multiply workloads.

Every generator is pure NumPy on ``numpy.random.default_rng(seed)`` and returns a
directed, symmetric, coalesced edge list ``edge_index`` (int32, shape ``[2, E]``, sorted
by (row, col)) whose ids are contiguous from 0 and in which every node has at least one
edge -- the four preconditions the reference states in ``cbm/utility.py:4-29``.

The five named workloads (``workload("c1") .. workload("c5")``) are the graphs the
reference-style benchmarks of this repository run on (plus ``"c2b"``, the second workload held to
its configured size, and ``"c6"``, a deep and wide tree outside the five); the reference itself downloads
SNAP / DIMACS graphs (``benchmark/utility.py:23-42``), which is impossible offline.
"""
from __future__ import annotations

import hashlib
from dataclasses import dataclass

import numpy as np

__all__ = [
    "Workload", "workload", "coalesce_undirected", "add_self_loops", "edge_hash",
    "erdos_renyi", "sbm", "duplication", "chung_lu_cliques", "sbm_with_chain", "staircases",
]


# ----------------------------------------------------------------------------------------
# helpers
# ----------------------------------------------------------------------------------------
def _tri_decode(t: np.ndarray):
    """Map linear indices t in [0, n(n-1)/2) to pairs (i, j) with i > j >= 0."""
    t = t.astype(np.int64, copy=False)
    i = np.floor((1.0 + np.sqrt(1.0 + 8.0 * t.astype(np.float64))) * 0.5).astype(np.int64)
    # repair the float rounding at triangle boundaries
    base = i * (i - 1) // 2
    i = np.where(base > t, i - 1, i)
    base = i * (i - 1) // 2
    i = np.where(t - base >= i, i + 1, i)
    base = i * (i - 1) // 2
    return i, t - base


def _bernoulli_positions(rng, m: int, p: float) -> np.ndarray:
    """Sorted positions of the successes of m independent Bernoulli(p) trials."""
    if m <= 0 or p <= 0.0:
        return np.empty(0, np.int64)
    if p >= 1.0:
        return np.arange(m, dtype=np.int64)
    out = []
    pos = -1
    while True:
        want = int((m - pos) * p * 1.05) + 64
        gaps = rng.geometric(p, size=want).astype(np.int64)
        cs = pos + np.cumsum(gaps)
        if cs[-1] >= m:
            out.append(cs[cs < m])
            break
        out.append(cs)
        pos = int(cs[-1])
    return np.concatenate(out)


def coalesce_undirected(u: np.ndarray, v: np.ndarray, n: int, drop_loops: bool = True,
                        assume_unique: bool = False) -> np.ndarray:
    """Symmetrise, de-duplicate and sort an undirected pair list -> int32 [2, E].
    ``assume_unique``: the pairs are known to be distinct (only the sort is needed)."""
    u = np.asarray(u, np.int64)
    v = np.asarray(v, np.int64)
    if drop_loops:
        keep = u != v
        u, v = u[keep], v[keep]
    key = np.concatenate([u * n + v, v * n + u])
    if assume_unique:
        key.sort(kind="stable")                 # two long sorted-ish runs: timsort territory
    else:
        key = np.unique(key)
    out = np.empty((2, key.shape[0]), np.int32)
    np.floor_divide(key, n, out=out[0], casting="unsafe")
    np.remainder(key, n, out=out[1], casting="unsafe")
    return out


def add_self_loops(edge_index: np.ndarray, n: int | None = None) -> np.ndarray:
    """Remove existing self loops, append the identity, coalesce (``gnns/utility.py:36-43``)."""
    ei = np.asarray(edge_index, np.int64)
    if n is None:
        n = int(ei.max()) + 1
    keep = ei[0] != ei[1]
    key = np.concatenate([ei[0][keep] * n + ei[1][keep], np.arange(n, dtype=np.int64) * (n + 1)])
    key.sort(kind="stable")
    if key.size > 1:
        key = key[np.concatenate([[True], key[1:] != key[:-1]])]
    out = np.empty((2, key.shape[0]), np.int32)
    np.floor_divide(key, n, out=out[0], casting="unsafe")
    np.remainder(key, n, out=out[1], casting="unsafe")
    return out


def _patch_isolated(rng, edge_index: np.ndarray, n: int) -> np.ndarray:
    """Give every node without an edge one random neighbour, so ids stay contiguous."""
    deg = np.bincount(edge_index[0], minlength=n)
    iso = np.flatnonzero(deg == 0)
    if iso.size == 0:
        return edge_index
    other = rng.integers(0, n - 1, size=iso.size)
    other = np.where(other >= iso, other + 1, other)
    u = np.concatenate([edge_index[0].astype(np.int64), iso])
    v = np.concatenate([edge_index[1].astype(np.int64), other])
    return coalesce_undirected(u, v, n)


def edge_hash(edge_index: np.ndarray) -> str:
    """SHA-256 of the (row, col)-sorted int32 edge array; pins a generator against drift."""
    ei = np.ascontiguousarray(np.asarray(edge_index, np.int32))
    return hashlib.sha256(ei.tobytes()).hexdigest()


# ----------------------------------------------------------------------------------------
# generators
# ----------------------------------------------------------------------------------------
def erdos_renyi(n: int, p: float, seed: int = 0) -> np.ndarray:
    """G(n, p), undirected, no self loops -- the graph family of the reference's tests
    (``tests/test_matmul_correctness.py:11-23``: n=25, p=0.5)."""
    rng = np.random.default_rng(seed)
    pos = _bernoulli_positions(rng, n * (n - 1) // 2, p)
    i, j = _tri_decode(pos)
    return _patch_isolated(rng, coalesce_undirected(i, j, n), n)


def sbm(n: int, blocks: int, p_in: float, p_out: float, seed: int = 0, patch: bool = True) -> np.ndarray:
    """Stochastic block model with ``blocks`` contiguous, (almost) equal blocks."""
    rng = np.random.default_rng(seed)
    bounds = np.linspace(0, n, blocks + 1).astype(np.int64)
    us, vs = [], []
    for b in range(blocks):
        lo, hi = int(bounds[b]), int(bounds[b + 1])
        sz = hi - lo
        pos = _bernoulli_positions(rng, sz * (sz - 1) // 2, p_in)
        i, j = _tri_decode(pos)
        us.append(i + lo)
        vs.append(j + lo)
    # inter-block pairs: thin all pairs with p_out, drop those that fall inside a block
    pos = _bernoulli_positions(rng, n * (n - 1) // 2, p_out)
    i, j = _tri_decode(pos)
    blk = np.searchsorted(bounds, np.arange(n), side="right") - 1
    keep = blk[i] != blk[j]
    us.append(i[keep])
    vs.append(j[keep])
    # positions inside one triangle are distinct and inter-block pairs never fall inside a block
    ei = coalesce_undirected(np.concatenate(us), np.concatenate(vs), n, assume_unique=True)
    return _patch_isolated(rng, ei, n) if patch else ei


def duplication(n: int, keep: float = 0.7, extra: int = 3, seed_clique: int = 8, seed: int = 0,
                copy_cap: int | None = None) -> np.ndarray:
    """Duplication model: node t picks a uniform earlier node, copies that node's CURRENT
    neighbour list keeping each entry with probability ``keep``, and adds ``extra`` uniform
    random earlier nodes.  A node's row overlaps its template's by ~``keep``, which is what
    CBM compresses.  Copying current lists makes the edge count grow like t^(2*keep): with
    keep=0.7 and n=12000 the graph has ~1.8M undirected edges.  ``copy_cap``: copy from at most
    this many entries of the template's list (a uniform sample of it), which bounds a new node's
    degree and with it the growth: keep=0.7, n=12000, copy_cap=26 gives ~240k undirected edges.
    (``copy_cap=None`` draws exactly the random numbers it always drew.)"""
    rng = np.random.default_rng(seed)
    nb = [set(s for s in range(seed_clique) if s != t) for t in range(seed_clique)] + [None] * (n - seed_clique)
    for t in range(seed_clique, n):
        proto = int(rng.integers(0, t))
        src = np.fromiter(nb[proto], np.int64, len(nb[proto]))
        src.sort()
        if copy_cap is not None and src.size > copy_cap:
            src = np.sort(rng.choice(src, size=copy_cap, replace=False))
        kept = src[rng.random(src.size) < keep]
        mine = set(kept.tolist()) | set(rng.integers(0, t, size=extra).tolist())
        nb[t] = mine
        for s in mine:
            nb[s].add(t)
    u = np.concatenate([np.full(len(s), i, np.int64) for i, s in enumerate(nb)])
    v = np.concatenate([np.fromiter(s, np.int64, len(s)) for s in nb])
    return coalesce_undirected(u, v, n)


def chung_lu_cliques(n: int = 100_000, gamma: float = 2.1, mean_deg: float = 32.0,
                     n_cliques: int = 20_000, kmin: int = 4, kmax: int = 12, seed: int = 0) -> np.ndarray:
    """Chung-Lu power-law graph (expected degree sequence w_i ~ i^(-1/(gamma-1)), scaled to
    ``mean_deg`` and capped at sqrt(sum w) so that edge probabilities stay below 1) overlaid
    with ``n_cliques`` cliques on uniform random node sets of size U{kmin..kmax}."""
    rng = np.random.default_rng(seed)
    w = (np.arange(n, dtype=np.float64) + 1.0) ** (-1.0 / (gamma - 1.0))
    w *= mean_deg * n / w.sum()
    for _ in range(8):                                   # cap, then rescale the rest
        cap = np.sqrt(w.sum())
        over = w > cap
        if not over.any():
            break
        w[over] = cap
        w[~over] *= (mean_deg * n - w[over].sum()) / w[~over].sum()
    perm = rng.permutation(n)                            # hubs are not the low ids
    pr = w / w.sum()
    m = int(round(mean_deg * n / 2))
    a = perm[rng.choice(n, size=m, p=pr)]
    b = perm[rng.choice(n, size=m, p=pr)]
    us, vs = [a], [b]
    sizes = rng.integers(kmin, kmax + 1, size=n_cliques)
    for k in range(kmin, kmax + 1):
        cnt = int((sizes == k).sum())
        if cnt == 0:
            continue
        # k distinct members per clique: argpartition of random keys would be O(n) each;
        # draw k uniform ids and redraw the few cliques with a repeat
        mem = rng.integers(0, n, size=(cnt, k))
        for _ in range(64):
            srt = np.sort(mem, axis=1)
            bad = (srt[:, 1:] == srt[:, :-1]).any(axis=1)
            if not bad.any():
                break
            mem[bad] = rng.integers(0, n, size=(int(bad.sum()), k))
        iu, ju = np.triu_indices(k, 1)
        us.append(mem[:, iu].ravel())
        vs.append(mem[:, ju].ravel())
    ei = coalesce_undirected(np.concatenate(us), np.concatenate(vs), n)
    return _patch_isolated(rng, ei, n)


def sbm_with_chain(n: int = 132_534, blocks: int = 300, p_in: float = 1.0, mean_deg: float = 600.0,
                   chain: int = 2000, base: int = 48, seed: int = 0) -> np.ndarray:
    """Dense-community SBM on the first ``n - chain - 1`` ids plus a staircase that forces a
    ``chain + 1``-deep path into every minimum arborescence: chain node c_k (one of the last
    ``chain + 1`` ids) is adjacent to anchors a_1 .. a_{base+k}, so row(c_k) = row(c_{k-1}) +
    one column and the Hamming distance between consecutive chain rows is 1."""
    rng = np.random.default_rng(seed)
    n_chain = chain + 1
    n_sbm = n - n_chain
    blk = n_sbm / blocks
    intra = p_in * (blk - 1.0)
    p_out = max(0.0, (mean_deg - intra) / (n_sbm - blk))
    ei = sbm(n_sbm, blocks, p_in, p_out, seed=seed + 1, patch=True)
    anchors = rng.choice(n_sbm, size=base + chain, replace=False).astype(np.int64)
    cu, cv = [], []
    for k in range(n_chain):
        cu.append(np.full(base + k, n_sbm + k, np.int64))
        cv.append(anchors[: base + k])
    cu = np.concatenate(cu); cv = np.concatenate(cv)
    u = np.concatenate([ei[0].astype(np.int64), cu])
    v = np.concatenate([ei[1].astype(np.int64), cv])
    return coalesce_undirected(u, v, n)


def staircases(n_chains: int = 800, depth: int = 100, base: int = 28, noise_deg: float = 2.0, seed: int = 0) -> np.ndarray:
    """``n_chains`` disjoint half-graphs ("staircases") plus a sparse random background: a graph whose
    minimum arborescence is DEEP AND WIDE at once.  Staircase w has ``depth`` chain nodes c_0 .. c_{depth-1}
    and ``base + depth`` anchors; c_k is adjacent to the anchors a_0 .. a_{base+k}, so row(c_k) =
    row(c_{k-1}) + one column, and on the other side row(a_{base+j}) = row(a_{base+j+1}) + one column: both
    sides are chains of Hamming distance 1, ``depth`` levels deep, and every tree level holds about
    2 * n_chains rows.  On top, ``noise_deg * n / 2`` uniform random edges, so that consecutive rows
    differ in a handful of columns rather than one.  Node ids are shuffled: neither the kernels nor the
    builder get the chains as contiguous id ranges.  n = n_chains * (2 * depth + base)."""
    rng = np.random.default_rng(seed)
    per = 2 * depth + base
    n = n_chains * per
    k = np.repeat(np.arange(depth, dtype=np.int64), base + 1 + np.arange(depth))      # chain node of every stair edge
    j = np.concatenate([np.arange(base + 1 + q, dtype=np.int64) for q in range(depth)])  # its anchor
    off = (np.arange(n_chains, dtype=np.int64) * per)[:, None]
    u = (off + k[None, :]).ravel()                                                      # chain nodes: first `depth` ids of a staircase
    v = (off + depth + j[None, :]).ravel()                                              # anchors: the rest
    m = int(round(noise_deg * n / 2))
    nu, nv = rng.integers(0, n, size=m), rng.integers(0, n, size=m)
    perm = rng.permutation(n)
    u, v = perm[np.concatenate([u, nu])], perm[np.concatenate([v, nv])]
    return _patch_isolated(rng, coalesce_undirected(u, v, n), n)


def clique_union(n: int = 150_000, n_cliques: int = 12_000, lo: int = 15, hi: int = 40, strangers: int = 2,
                 seed: int = 0) -> np.ndarray:
    """Union of ``n_cliques`` cliques of ``lo`` .. ``hi`` nodes -- the shape of a co-authorship graph (every
    paper a clique of its authors), the family behind the reference's best compression ratios.  A clique is a
    run of consecutive ids (a "group") plus ``strangers`` uniform random nodes, so neighbouring cliques overlap
    and the rows of a clique's members differ in a handful of columns."""
    rng = np.random.default_rng(seed)
    us, vs = [], []
    for _ in range(n_cliques):
        k = int(rng.integers(lo, hi + 1))
        start = int(rng.integers(0, n - k))
        members = np.unique(np.concatenate([np.arange(start, start + k - strangers), rng.integers(0, n, strangers)]))
        a, b = np.meshgrid(members, members)
        keep = a < b
        us.append(a[keep]); vs.append(b[keep])
    return _patch_isolated(rng, coalesce_undirected(np.concatenate(us), np.concatenate(vs), n), n)


# ----------------------------------------------------------------------------------------
# the five named workloads (and two outside them)
# ----------------------------------------------------------------------------------------
@dataclass
class Workload:
    name: str
    edge_index: np.ndarray      # int32 [2, E], what the cbm_matrix constructor receives
    n: int
    d: int                      # feature width of X
    normalized: bool
    alphas: tuple
    x_dist: str                 # "normal" | "uniform"
    note: str = ""

    def features(self, seed: int = 0, d: int | None = None):
        """X (fp32, [n, d]) from ``torch.Generator().manual_seed(seed)`` on the CPU."""
        import torch
        g = torch.Generator().manual_seed(seed)
        d = self.d if d is None else d
        if self.x_dist == "uniform":
            return torch.rand((self.n, d), generator=g, dtype=torch.float32) * 2.0 - 1.0
        return torch.randn((self.n, d), generator=g, dtype=torch.float32)


def workload(name: str, seed: int = 0, scale: float = 1.0) -> Workload:
    """Build one of the named workloads.  ``scale`` < 1 shrinks the node count (same
    generator, same densities) for quick parity runs; the benchmark uses ``scale == 1``."""
    name = name.lower()
    if name == "c1":
        n = max(64, int(4096 * scale)); blocks = max(1, n // 64)
        ei = sbm(n, blocks, 0.2, 0.0005, seed)
        return Workload("c1", ei, n, 64, False, (0,), "normal",
                        "SBM 64 blocks x 64, p_in=0.2, p_out=0.0005, plain A")
    if name == "c2":
        n = max(64, int(12_000 * scale))
        ei = add_self_loops(duplication(n, 0.7, 3, 8, seed), n)
        return Workload("c2", ei, n, 128, True, (0, 8), "normal",
                        "duplication model keep=0.7 +3 random, A+I normalised [the stated process, taken literally, yields "
                        "1.82 M undirected edges at N = 12 000, not the ~240 k the configuration names; c2b is the same "
                        "process held to that size]")
    if name == "c2b":
        # the same process held to the SIZE the configuration names (~240k undirected edges at N = 12 000): a new
        # node copies from at most 26 entries of its template's list
        n = max(64, int(12_000 * scale))
        ei = add_self_loops(duplication(n, 0.7, 3, 8, seed, copy_cap=26), n)
        return Workload("c2b", ei, n, 128, True, (0, 8), "normal",
                        "duplication model keep=0.7 +3 random, copying from at most 26 entries of the template's list "
                        "(~240k undirected edges), A+I normalised")
    if name == "c3":
        n = max(256, int(100_000 * scale))
        ei = add_self_loops(chung_lu_cliques(n, 2.1, 32.0, max(1, int(20_000 * scale)), 4, 12, seed), n)
        return Workload("c3", ei, n, 256, True, (16,), "uniform",
                        "Chung-Lu gamma=2.1 mean degree 32 + 20k cliques of 4..12, A+I normalised")
    if name == "c4":
        n = max(500, int(232_965 * scale)); blocks = 50
        blk = n / blocks
        mean_deg = 490.0 * min(1.0, scale)                   # 90 % of it inside the block
        p_in = min(1.0, 0.9 * mean_deg / (blk - 1.0))
        p_out = 0.1 * mean_deg / (n - blk)
        ei = add_self_loops(sbm(n, blocks, p_in, p_out, seed), n)
        return Workload("c4", ei, n, 602, True, (2,), "normal",
                        "SBM 50 blocks, mean degree ~490 (90% intra), A+I normalised, GCN 602-128-41")
    if name == "c5":
        n = max(4000, int(132_534 * scale)); blocks = max(2, int(300 * scale))
        chain = max(8, int(2000 * min(1.0, scale)))
        ei = sbm_with_chain(n, blocks, 1.0, 600.0 * min(1.0, scale), chain, 48, seed)
        return Workload("c5", ei, n, 512, False, (0, 2, 4, 8, 16, 32), "normal",
                        "SBM 300 clique blocks (p_in=1) + p_out to mean degree ~600, + 2000-deep staircase chain, plain A")
    if name == "c6":
        # outside the five configured workloads: a deep AND wide arborescence with a high compression ratio, the
        # regime of the reference's best datasets (plot_results_alpha_vs_runtime.py:55,63: ratios 5.9 .. 9.8),
        # where its tree walk -- serial inside a subtree, cbm_extensions.cpp:1166-1218 -- is the bottleneck
        chains = max(4, int(800 * scale))
        ei = add_self_loops(staircases(chains, 100, 28, 2.0, seed))
        n = chains * 228
        return Workload("c6", ei, n, 256, True, (0,), "normal",
                        "800 disjoint staircases (half-graphs) of depth 100 + random edges of mean degree 2, ids shuffled, "
                        "A+I normalised: ~100 tree levels of ~1 600 rows each")
    if name == "c7":
        # outside the five as well: a union of cliques, the co-authorship shape of the reference's own datasets
        # (ca-AstroPh, ca-HepPh, COLLAB, coPapers*): compression ~5.8, 44 tree levels, subtrees of a few to a
        # few hundred rows -- what CBM gives on a graph nobody shaped for it
        n = max(2000, int(150_000 * scale))
        ei = add_self_loops(clique_union(n, max(20, int(12_000 * scale)), 15, 40, 2, seed), n)
        return Workload("c7", ei, n, 128, True, (0,), "normal",
                        "union of 12 000 cliques of 15..40 nodes (runs of consecutive ids + 2 random nodes each), "
                        "A+I normalised: the co-authorship shape")
    raise ValueError(f"unknown workload {name!r}")
