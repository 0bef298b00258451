"""Host side of the tiled multiply (no GPU): ``cbm_tile_rows`` splits the packed delta matrix into
local blocks and remote entries exactly as defined -- a (256-row panel, 1024-column tile) block is
local iff it holds at least ``min_block_entries`` entries -- and lays the local entries out as the
kernel reads them (segments per block and panel row, padded to 8 with the zero-row index)."""
import numpy as np
import pytest
import torch

from cbm4gnn_amd import graphs
from cbm4gnn_amd.cbm import cbm_matrix

P, T = 256, 1024


def split_by_definition(mat, min_block_entries):
    """(local mask per delta entry, row per entry, column per entry, sign bit per entry), NumPy."""
    n = mat.num_rows
    rp = mat.rowptr.numpy().astype(np.int64)
    idx = mat.idx.numpy().view(np.uint32)
    row = np.repeat(np.arange(n), np.diff(rp))
    col = (idx & 0x7FFFFFFF).astype(np.int64)
    n_tiles = (n + T - 1) // T
    key = (row // P) * n_tiles + col // T
    cnt = np.bincount(key, minlength=((n + P - 1) // P) * n_tiles)
    return cnt[key] >= min_block_entries, row, col, (idx >> 31).astype(np.int64), key, cnt, n_tiles


def decode(th, n):
    """Every local entry the tiling arrays hold, as sorted (row, col, negative) triples, checking
    the layout on the way."""
    pp, bt, seg, lidx = (th[k].numpy() for k in ("panel_ptr", "blk_tile", "seg", "lidx"))
    lidx = lidx.view(np.uint16).astype(np.int64)
    seg = seg.reshape(-1, P + 1).astype(np.int64)
    assert pp[0] == 0 and pp[-1] == seg.shape[0] == bt.shape[0] and (np.diff(pp) >= 0).all()
    flat = seg.ravel()
    assert (np.diff(flat) >= 0).all() and flat[0] == 0 and flat[-1] * 8 == lidx.shape[0]
    assert (seg[1:, 0] == seg[:-1, P]).all()                # blocks follow each other without a gap
    out = []
    pad = T * 8
    for p in range(pp.shape[0] - 1):
        assert (np.diff(bt[pp[p]:pp[p + 1]]) > 0).all()     # ascending tiles within a panel
        for b in range(pp[p], pp[p + 1]):
            for pr in range(P):
                ent = lidx[seg[b, pr] * 8:seg[b, pr + 1] * 8]
                real = ent[ent != pad]
                k = real.shape[0]
                assert (ent[:k] != pad).all() and (ent[k:] == pad).all() and ent.shape[0] - k < 8   # padding only at the end
                off = (real & 0x7FFF) // 8
                assert ((real & 0x7FFF) % 8 == 0).all() and (off < T).all()
                r = p * P + pr
                # by class (column - row) mod 4 in the order 0, 2, 1, 3 (so: own parity first), ascending inside a class
                cls = (off - r) % 4
                want = np.concatenate([np.sort(off[cls == q]) for q in (0, 2, 1, 3)])
                assert np.array_equal(off, want)
                assert k == 0 or r < n
                out += [(r, int(bt[b]) * T + int(o), int(v >> 15)) for o, v in zip(off, real)]
    return sorted(out)


@pytest.mark.parametrize("n,blocks,p_in,alpha,thr", [(3000, 30, 0.6, 0, 64), (2600, 5, 0.08, 1, 300), (1500, 2, 0.08, 0, 1)])
def test_tiling_is_the_defined_split(n, blocks, p_in, alpha, thr):
    ei = graphs.add_self_loops(graphs.sbm(n, blocks, p_in, 0.002, seed=n), n)
    mat = cbm_matrix(torch.from_numpy(ei), None, alpha=alpha, tiling="on")
    mat.tile_min_block_entries = thr
    th = mat._host_tiling()
    assert th and mat.is_tiled()
    local, row, col, neg, key, cnt, n_tiles = split_by_definition(mat, thr)
    assert mat.tiling_info["nnz_local"] == int(local.sum()) and mat.tiling_info["nnz_remote"] == int((~local).sum())
    assert th["has_negative"] == int(neg[local].any())
    if p_in > 0.5:
        assert neg.any() and mat.n_levels > 2               # the deltas really carry negative entries
    assert decode(th, n) == sorted(zip(row[local].tolist(), col[local].tolist(), neg[local].tolist()))
    # blocks = the (panel, tile) pairs at or above the threshold, in (panel, tile) order
    want_blocks = np.nonzero(cnt >= thr)[0]
    pp, bt = th["panel_ptr"].numpy(), th["blk_tile"].numpy()
    got_blocks = np.concatenate([np.full(pp[p + 1] - pp[p], p) for p in range(pp.shape[0] - 1)]) * n_tiles + bt
    assert np.array_equal(got_blocks, want_blocks)
    # remote part: an ordinary packed CSR of the other entries, columns ascending, signs kept
    rr, ir = th["rowptr_r"].numpy().astype(np.int64), th["idx_r"].numpy().view(np.uint32)
    assert np.array_equal(np.repeat(np.arange(n), np.diff(rr)), row[~local])
    assert np.array_equal(ir, mat.idx.numpy().view(np.uint32)[~local])
    if thr == 1:
        assert not (~local).any() and rr[-1] == 0           # everything is local


def test_tiling_policy():
    n = 3000
    ei = torch.from_numpy(graphs.add_self_loops(graphs.sbm(n, 3, 0.08, 0.002, seed=1), n))
    assert not cbm_matrix(ei, None, tiling="off").is_tiled()
    assert not cbm_matrix(ei, None, tiling="auto").is_tiled()        # far too small for "auto"
    forced = cbm_matrix(ei, None, tiling="on")
    forced.tile_min_block_entries = 10 ** 9                           # no block reaches it
    assert not forced.is_tiled() and forced.tiling_info["n_blocks"] == 0
    with pytest.raises(ValueError):
        cbm_matrix(ei, None, tiling="sometimes")
    # "auto" on a large matrix decides by the share of entries that fall into blocks
    big = graphs.add_self_loops(graphs.sbm(20_000, 8, 0.03, 0.0001, seed=2), 20_000)   # ~75 entries per row, 8 communities
    a = cbm_matrix(torch.from_numpy(big), None, alpha=10 ** 6, tiling="auto")
    assert a.is_tiled() and a.tiling_info["local_fraction"] > 0.8
    scattered = graphs.add_self_loops(graphs.erdos_renyi(20_000, 0.002, 3), 20_000)     # ~40 entries per row, no structure
    b = cbm_matrix(torch.from_numpy(scattered), None, alpha=10 ** 6, tiling="auto")
    assert not b.is_tiled() and b.tiling_info["local_fraction"] < 0.1


def test_split_schedule_covers_every_entry_once():
    """``cbm_schedule_rows_split``: rows above the chunk size become pieces of at most ``chunk``
    entries with consecutive slots, every other row keeps one descriptor with its left scale, and
    the descriptors are ordered by descending number of 64-entry gather rounds (stable)."""
    rng = np.random.default_rng(0)
    lens = rng.integers(0, 40, size=500)
    lens[[3, 77, 400]] = [10_000, 2049, 4096]              # three rows to cut at chunk = 2048; 4096 = exactly two pieces
    lens[5] = 2048                                          # exactly the chunk: not cut
    rowptr = torch.from_numpy(np.concatenate([[0], np.cumsum(lens)]).astype(np.int32))
    n = lens.shape[0]
    parent = torch.from_numpy(np.where(rng.random(n) < 0.5, -1, 0).astype(np.int32))
    m = torch.from_numpy(rng.random(n).astype(np.float32) + 0.5)
    mat = cbm_matrix.__new__(cbm_matrix)
    mat.split_chunk = 2048
    sched, long_rows, pieces = mat._split_schedule(rowptr, None, parent, m)
    assert long_rows[:, 0].tolist() == [3, 77, 400] and long_rows[:, 2].tolist() == [5, 2, 2] and pieces == 9
    assert long_rows[:, 1].tolist() == [0, 5, 7]
    assert sched.shape[0] == n - 3 + 9
    PIECE = 0x40000000
    covered = np.zeros(int(rowptr[-1]), np.int32)
    slots_seen = []
    rounds = []
    for s0, s1, row, w in sched.tolist():
        covered[s0:s1] += 1
        rounds.append((s1 - s0 + 63) // 64)
        scale = np.array([w], np.int32).view(np.float32)[0]
        if row & PIECE:
            slot = row & ~PIECE
            slots_seen.append(slot)
            owner = [r for r, f, k, _ in long_rows.tolist() if f <= slot < f + k][0]
            assert rowptr[owner] <= s0 < s1 <= rowptr[owner + 1] and s1 - s0 <= 2048 and scale == 1.0
            assert (s0 - int(rowptr[owner])) // 2048 == slot - [f for r, f, k, _ in long_rows.tolist() if r == owner][0]
        else:
            assert s0 == rowptr[row] and s1 == rowptr[row + 1] and s1 - s0 <= 2048
            assert scale == (float(m[row]) if parent[row] < 0 else 1.0)
    assert (covered == 1).all() and sorted(slots_seen) == list(range(9))
    assert rounds == sorted(rounds, reverse=True)
    for r, f, k, w in long_rows.tolist():                   # the left scale of a cut row travels with it
        assert np.array([w], np.int32).view(np.float32)[0] == (float(m[r]) if parent[r] < 0 else 1.0)
    # nothing to cut: the plain schedule
    mat.split_chunk = 1 << 20
    s2, l2, p2 = mat._split_schedule(rowptr, None, parent, m)
    from cbm4gnn_amd.cbm import schedule_rows
    assert l2.shape[0] == 0 and p2 == 0 and torch.equal(s2, schedule_rows(rowptr, parent, m))


def test_column_block_schedule():
    """``cbm_schedule_rows_blocks``: every row is cut where its columns pass from one block of
    ceil(n / B) columns to the next (and runs above the chunk size further), a row inside one block
    keeps one descriptor, every entry is covered once, slots of a row are consecutive in column
    order, and the descriptors are ordered by column block, longest first inside a block."""
    rng = np.random.default_rng(1)
    n, B, chunk = 1000, 4, 128
    block_cols = (n + B - 1) // B
    rows = []
    for r in range(n):
        k = int(rng.integers(0, 60))
        if r == 10:
            k = 900                                        # long row: cut by blocks and by chunk
        lo, hi = (0, n) if r % 3 else (300, 340)            # every third row lives inside block 1
        rows.append(np.sort(rng.choice(np.arange(lo, hi), size=min(k, hi - lo), replace=False)))
    rowptr = torch.from_numpy(np.concatenate([[0], np.cumsum([len(c) for c in rows])]).astype(np.int32))
    col = np.concatenate(rows).astype(np.uint32)
    idx = torch.from_numpy((col | (rng.random(col.shape[0]) < 0.3).astype(np.uint32) << 31).view(np.int32))
    parent = torch.from_numpy(np.where(rng.random(n) < 0.5, -1, 0).astype(np.int32))
    m = torch.from_numpy(rng.random(n).astype(np.float32) + 0.5)
    mat = cbm_matrix.__new__(cbm_matrix)
    mat.split_chunk = chunk
    sched, long_rows, pieces = mat._split_schedule(rowptr, idx, parent, m, B)
    PIECE = 0x40000000
    owner_of = {}
    for r, f, k, w in long_rows.tolist():
        for q in range(k):
            owner_of[f + q] = (r, q)
        assert np.array([w], np.int32).view(np.float32)[0] == (float(m[r]) if parent[r] < 0 else 1.0)
    assert sorted(owner_of) == list(range(pieces))
    covered = np.zeros(col.shape[0], np.int32)
    keys, starts_of = [], {}
    for s0, s1, row, w in sched.tolist():
        covered[s0:s1] += 1
        blocks = set((col[s0:s1] // block_cols).tolist())
        assert len(blocks) <= 1 and s1 - s0 <= chunk
        blk = blocks.pop() if blocks else 0
        keys.append((blk, -((s1 - s0 + 63) // 64)))
        if row & PIECE:
            r, q = owner_of[row & ~PIECE]
            starts_of.setdefault(r, []).append((q, s0, s1))
            assert np.array([w], np.int32).view(np.float32)[0] == 1.0
        else:
            assert s0 == rowptr[row] and s1 == rowptr[row + 1]
            assert np.array([w], np.int32).view(np.float32)[0] == (float(m[row]) if parent[row] < 0 else 1.0)
    assert (covered == 1).all() and keys == sorted(keys)
    for r, lst in starts_of.items():                       # the pieces of a row tile it in slot order
        lst.sort()
        assert lst[0][1] == rowptr[r] and lst[-1][2] == rowptr[r + 1] and len(lst) >= 2
        assert all(a[2] == b[1] for a, b in zip(lst, lst[1:]))
    assert 10 in starts_of and len(starts_of[10]) == sum(-(-int(((rows[10] // block_cols) == b).sum()) // chunk) for b in range(B))
    assert not any(r % 3 == 0 and r != 10 for r in starts_of)      # rows inside one block are not cut
    # one block, no chunk: the plain schedule
    mat.split_chunk = 0
    s1_, l1_, p1_ = mat._split_schedule(rowptr, idx, parent, m, 1)
    from cbm4gnn_amd.cbm import schedule_rows
    assert p1_ == 0 and torch.equal(s1_, schedule_rows(rowptr, parent, m))


def test_tiling_rejects_unsorted_and_out_of_range_columns():
    """The fill takes the entries of one row inside one block as a single ascending run; a row whose
    columns do not ascend strictly (or leave the matrix) is refused, not tiled wrongly."""
    import ctypes as C
    from cbm4gnn_amd import _lib
    host = _lib.host_lib()
    n = 2048
    rp = np.arange(0, 4 * (n + 1), 4, dtype=np.int32)
    # row r holds the columns r % 1000 + {0, 7, 14, 21}
    good = (np.arange(4, dtype=np.uint32)[None, :] * 7 + (np.arange(n, dtype=np.uint32)[:, None] % 1000)).ravel()

    def run(idx):
        t = _lib.CbmTiling()
        rc = host.cbm_tile_rows(C.c_void_p(rp.ctypes.data), C.c_void_p(idx.ctypes.data), n, 1024, 1, 0, C.byref(t))
        blocks = int(t.n_blocks)
        host.cbm_tiling_free(C.byref(t))
        return rc, blocks

    rc, blocks = run(good)
    assert rc == 0 and blocks > 0
    for damage in ("swap", "repeat", "range", "sign"):
        bad = good.copy()
        if damage == "swap":
            bad[[4 * 700, 4 * 700 + 1]] = bad[[4 * 700 + 1, 4 * 700]]
        elif damage == "repeat":
            bad[4 * 701 + 2] = bad[4 * 701 + 1]
        elif damage == "range":
            bad[4 * 702 + 3] = n
        else:
            bad[4 * 703 + 3] = np.uint32(0x80000000) | np.uint32(n + 5)      # out of range under the sign bit
        assert run(bad)[0] == _lib.CBM_ERR_SHAPE, damage
    signed = good.copy(); signed[4 * 9 + 1] |= np.uint32(0x80000000)         # a negative entry in range is fine
    assert run(signed)[0] == 0


def test_batched_schedule_layout():
    """cbm_schedule_rows_batched: rows above the limit first, in the order of cbm_schedule_rows; then the others by
    descending number of 8-entry chunks, natural order inside a chunk count; a trailer says where they start."""
    from cbm4gnn_amd.cbm import schedule_rows
    rng = np.random.default_rng(2)
    lens = rng.integers(0, 200, size=500)
    lens[rng.random(500) < 0.5] //= 12
    rp = torch.from_numpy(np.concatenate([[0], np.cumsum(lens)]).astype(np.int32))
    parent = torch.from_numpy(np.where(rng.random(500) < 0.3, -1, 0).astype(np.int32))
    m = torch.from_numpy((rng.random(500) + 0.5).astype(np.float32))
    plain = schedule_rows(rp, parent, m).numpy()
    for limit in (1, 8, 20, 64):
        s = schedule_rows(rp, parent, m, batch=limit).numpy()
        assert s.shape == (501, 4)
        n_wide, t, magic, zero = s[-1]
        assert t == limit and magic == 0x62617463 and zero == 0 and n_wide == int((lens > limit).sum())
        body = s[:-1]
        assert sorted(body[:, 2].tolist()) == list(range(500))                      # every row once
        assert np.array_equal(body[:, 0], rp.numpy()[body[:, 2]]) and np.array_equal(body[:, 1], rp.numpy()[body[:, 2] + 1])
        want_scale = np.where(parent.numpy()[body[:, 2]] < 0, m.numpy()[body[:, 2]], np.float32(1)).astype(np.float32)
        assert np.array_equal(body[:, 3].view(np.float32), want_scale)
        wide = body[:n_wide]
        assert np.array_equal(wide, plain[lens[plain[:, 2]] > limit])               # same relative order as the plain schedule
        short = body[n_wide:]
        sl = lens[short[:, 2]]
        assert (sl <= limit).all()
        chunks = (sl + 7) // 8
        assert (np.diff(chunks) <= 0).all()
        for c in np.unique(chunks):
            assert (np.diff(short[chunks == c, 2]) > 0).all()                       # stable
    import ctypes as C
    from cbm4gnn_amd import _lib
    out = np.empty(4 * 501, np.int32)
    ptr = lambda a: C.c_void_p(a.ctypes.data)
    assert _lib.host_lib().cbm_schedule_rows_batched(ptr(rp.numpy()), None, None, 500, 65, ptr(out)) == _lib.CBM_ERR_SHAPE
    assert _lib.host_lib().cbm_schedule_rows_batched(None, None, None, 500, 8, ptr(out)) == _lib.CBM_ERR_NULL
