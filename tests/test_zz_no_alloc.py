"""The entry point that allocates nothing, ``cbm_spmm_update_static_f32``, called through the C ABI:
its output must equal, bit for bit, that of ``cbm_spmm_update_f32`` with a caller-owned workspace,
on two calls in a row (the second with a smaller input, so the static scratch still holds the
first call's larger copy), and a shape beyond the static array must be refused before anything
is enqueued."""
import ctypes as C
import sys

import numpy as np
import pytest
import torch

from cbm4gnn_amd import _lib, graphs
from cbm4gnn_amd.cbm import cbm_matrix

pytestmark = pytest.mark.gpu


def say(*a):
    print("[gpu-case]", *a, flush=True)
    sys.stdout.flush()


@pytest.fixture(scope="module", autouse=True)
def _need_gpu():
    if not torch.cuda.is_available():
        pytest.skip("no HIP device")
    _lib.hip_lib()


def p(t):
    return C.c_void_p(t.data_ptr()) if t is not None else None


def both_entry_points(mat, x, normalized):
    """(output of cbm_spmm_update_f32 with a workspace, output of cbm_spmm_update_static_f32)."""
    lib = _lib.hip_lib()
    dev = x.device
    st = mat._device_arrays(dev)
    n, d = x.shape
    m = st["m"] if normalized else None
    coef = st["coef"] if normalized else None
    sched = st["sched_scaled"] if normalized else st["sched"]
    stream = C.c_void_p(torch.cuda.current_stream(dev).cuda_stream)
    y_ws = torch.full_like(x, float("nan"))
    y_st = torch.full_like(x, float("nan"))
    floats = lib.cbm_spmm_workspace_floats(n, d, d, d, p(x), p(y_ws))
    assert floats > 0
    ws = torch.empty(floats, dtype=torch.float32, device=dev)
    rc = lib.cbm_spmm_update_f32(p(st["rowptr"]), p(st["idx"]), mat.nnz, p(m), p(coef), p(st["parent"]), p(sched),
                                 p(st["order"]), p(st["level_off"]), p(mat.level_off), mat.n_levels, p(x), p(y_ws),
                                 p(ws), n, d, d, d, 0, stream)
    assert rc == 0
    torch.cuda.synchronize()
    before = torch.cuda.memory_allocated(dev)
    rc = lib.cbm_spmm_update_static_f32(p(st["rowptr"]), p(st["idx"]), mat.nnz, p(m), p(coef), p(st["parent"]),
                                        p(sched), p(st["order"]), p(st["level_off"]), p(mat.level_off), mat.n_levels,
                                        p(x), p(y_st), n, d, d, d, 0, stream)
    assert rc == 0
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated(dev) == before
    return y_ws.cpu().numpy(), y_st.cpu().numpy()


@pytest.mark.parametrize("normalized", [False, True])
def test_static_scratch_entry_point_matches_the_workspace_one(orc, normalized):
    dev = torch.device("cuda", 0)
    # first call: 3000 rows x 200 columns (7 slabs -> 8 padded); second: 900 rows x 41 columns
    for n, blocks, d, seed in ((3000, 30, 200, 1), (900, 10, 41, 2)):
        say("static scratch", normalized, n, d)
        ei = graphs.add_self_loops(graphs.sbm(n, blocks, 0.6, 0.002 * 3000 / n, seed=seed), n)
        mat = cbm_matrix(torch.from_numpy(ei), None, alpha=1, normalized=normalized)
        assert mat.n_levels >= 2
        x = torch.randn((n, d), generator=torch.Generator().manual_seed(seed)).to(dev)
        want, got = both_entry_points(mat, x, normalized)
        assert np.isfinite(want).all()
        assert np.array_equal(got, want)                    # bit for bit
        assert orc.max_rel_err(got, orc.dense_product(ei, n, x.cpu().numpy(), normalized)) <= 1e-3


def test_static_scratch_refuses_what_does_not_fit():
    lib = _lib.hip_lib()
    dev = torch.device("cuda", 0)
    n = 70_000
    d = 512                                                 # 70 000 x 512 floats = 35.8 M > 32 Mi
    assert n * d > _lib.CBM_STATIC_SCRATCH_FLOATS
    say("static scratch too large", n, d)
    x = torch.zeros((n, d), device=dev)
    y = torch.full((n, d), 7.0, device=dev)
    rp = torch.zeros(n + 1, dtype=torch.int32, device=dev)
    idx = torch.zeros(1, dtype=torch.int32, device=dev)
    par = torch.full((n,), -1, dtype=torch.int32, device=dev)
    order = torch.arange(n, dtype=torch.int32, device=dev)
    lo_host = torch.tensor([0, n], dtype=torch.int32)
    lo = lo_host.to(dev)
    rc = lib.cbm_spmm_update_static_f32(p(rp), p(idx), 0, None, None, p(par), None, p(order), p(lo), p(lo_host), 1,
                                        p(x), p(y), n, d, d, d, 0, None)
    assert rc == _lib.CBM_ERR_SCRATCH
    assert b"scratch" in lib.cbm_status_string(rc)
    torch.cuda.synchronize()
    assert bool((y == 7.0).all())                           # nothing was enqueued
    # the same rows at a width whose copy fits are accepted (empty rows: the product is zero)
    d2 = 256
    rc = lib.cbm_spmm_update_static_f32(p(rp), p(idx), 0, None, None, p(par), None, p(order), p(lo), p(lo_host), 1,
                                        p(x), p(y), n, d2, d, d, 0, None)
    assert rc == 0
    torch.cuda.synchronize()
    assert bool((y[:, :d2] == 0).all()) and bool((y[:, d2:] == 7.0).all())
