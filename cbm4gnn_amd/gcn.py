"""GCN layers over the CBM multiply, for the 2-layer forward+backward epoch measurement.

The reference's layer is ``x = Linear(x); x = aggregate(x)`` with a cached ``cbm_matrix`` built
on the transposed, self-looped edge list and ``normalize=True``
(``gnns/graph_convolutional_network/cbm_gcn.py:27-41``,
``gnns/message_passing/cbm_message_passing.py:40-60``); its benchmark model stacks two of them
with a ReLU in between and shares one ``cbm_matrix`` between the layers
(``benchmark/parallel/benchmark_gcn_cpu.py:62-89``).  The reference uses
``torch_geometric.nn.Linear(bias=False, weight_initializer='glorot')``; torch_geometric is not a
dependency here, ``torch.nn.Linear`` with Xavier-uniform weights is the same layer.

Unlike the reference's CBM layers, whose aggregation mutates a cached output behind autograd's
back (so they have no usable backward), aggregation here is differentiable: backward is the same
CBM multiply with the transposed operator.

``CBMGCNLayer(fused=True)`` (the default) runs the whole layer as one autograd function around
the multiply:

* with a plain (un-normalised) operator the Linear output is written by the GEMM straight into a
  buffer whose row stride is d + 32 floats (an odd number of 128-byte lines), which the SpMM
  gathers in place -- no slab-major copy of it is made (widths other than 32, 64, 128 or 256
  still take the copy).  A normalised operator keeps the copy: scaled by m on the way, it
  spares the multiply every per-entry coefficient, which is worth more than the copy costs;
* the ReLU is applied in the multiply's store epilogue (``CBM_UPDATE_RELU``) and its gradient is
  folded into the slab-major copy the backward multiply makes of the incoming gradient
  (``cbm_relayout_slabs_masked_f32``), with the layer's own output as the mask;
* the Linear output, the layer output, the workspace and the gradient buffer are allocated once
  per layer and reused by every call, as the reference caches its output
  (``cbm_message_passing.py:26-29``).  As there, the tensor a call returns is overwritten by the
  next call of the same layer.  A backward that would read an overwritten buffer raises: the layer
  counts its forward calls and bumps the buffer's autograd version, so ``forward, forward, backward
  of the first`` is an error, never a wrong gradient (``fused=False`` allocates per call instead).
"""
from __future__ import annotations

import contextlib
import os
import tempfile

import torch
from torch import nn

from . import _lib
from .cbm import DEFAULT_BATCH_ROWS, CBMMatmul, _ld, _ptr, _wants_workspace, cbm_matrix, csr_spmm, relayout_slabs, schedule_rows

__all__ = ["CBMGCNLayer", "CSRGCNLayer", "TwoLayerGCN", "build_operator", "csr_operator", "CSRMatmul", "tuned_gemms"]


@contextlib.contextmanager
def tuned_gemms(max_ms_per_solution: int = 10, filename: str | None = None):
    """Run the dense GEMMs inside the block on the library solution torch's TunableOp measures to be
    fastest for each shape (first call of a shape inside the block tunes it, later calls reuse the pick).

    The GEMMs around the aggregation are tall and skinny -- ``x W^T`` and the weight gradients
    ``g^T x`` over N = 10^5..10^6 rows against 41..602 columns -- and hipBLASLt's default heuristic
    serves the weight gradients badly (232,965 rows: 932 -> 484 us for 128 x N x 602, 435 -> 94 us for
    41 x N x 128).  This is plumbing around the CBM multiply, not part of it; outside the block torch's
    default choice is back.  The picks go to ``filename`` (default: a file in the temporary directory)."""
    import torch.cuda.tunable as tunable
    was_enabled, was_tuning = tunable.is_enabled(), tunable.tuning_is_enabled()
    tunable.set_filename(filename or os.path.join(tempfile.gettempdir(), f"cbm4gnn_tunableop_{os.getpid()}.csv"))
    tunable.set_max_tuning_duration(int(max_ms_per_solution))
    tunable.enable(True)
    tunable.tuning_enable(True)
    try:
        yield
    finally:
        tunable.tuning_enable(was_tuning)
        tunable.enable(was_enabled)


def build_operator(edge_index, alpha: int = 2, normalized: bool = True, builder: str = "auto") -> cbm_matrix:
    """``cbm_matrix`` of the TRANSPOSED edge list, as the reference's layers build it
    (``cbm_message_passing.py:48-49``; default alpha = 2, ``:8``)."""
    ei = torch.as_tensor(edge_index)
    ei_t = torch.stack([ei[1], ei[0]], dim=0).to(torch.int32)
    return cbm_matrix(ei_t, torch.ones(ei.size(1), dtype=torch.float32), normalized=normalized, alpha=alpha,
                      builder=builder)


class _FusedGCNLayer(torch.autograd.Function):
    """y = [relu](A_hat (x W^T)) on the layer's cached buffers; see the module docstring."""

    @staticmethod
    def forward(ctx, x, weight, layer):
        op = layer.cached_a_t
        xd = x.detach()
        if xd.dtype != torch.float32:
            raise RuntimeError("rhs tensor (NOT torch::kFloat32)")
        n, d = xd.size(0), weight.size(0)
        b = layer._layer_buffers(n, d, xd.device)
        torch.mm(xd, weight.detach().t(), out=b["h"])
        op._run_spmm_update(b["h"], b["y"], use_m=op.col_multiplier is not None,
                            workspace=b["ws"] if b["copy_h"] else None, relu=layer.relu)
        # The kernels wrote y through a raw pointer, which autograd cannot see: say so, so that a tensor
        # saved on this storage by an earlier call (the next layer keeps its input for its weight gradient)
        # fails its version check in backward instead of silently holding this call's values ...
        torch.autograd.graph.increment_version(b["y"])
        # ... and count the calls: this layer's own backward reads y as the ReLU mask and must see the
        # y of the forward it belongs to.
        layer._generation += 1
        ctx.generation = layer._generation
        ctx.layer = layer
        ctx.save_for_backward(xd, weight)
        return b["y"].detach()                              # a fresh tensor object on the cached storage

    @staticmethod
    def backward(ctx, g):
        layer = ctx.layer
        if layer._generation != ctx.generation:
            raise RuntimeError("CBMGCNLayer(fused=True) keeps one output buffer per layer: this layer ran forward again "
                               "before the backward of an earlier call, which overwrote the output that backward needs. "
                               "Run backward before the next forward, or build the layer with fused=False.")
        x, weight = ctx.saved_tensors
        op_t = layer.cached_a_t.transposed()
        n, d = g.shape
        b = layer._layer_buffers(n, d, g.device)
        if g.stride(1) != 1 or (n > 1 and g.stride(0) < d):
            g = g.contiguous()
        if layer.relu:
            # d relu: the copy the multiply gathers from holds g where the layer's output is positive
            # (and, like every copy a normalised multiply makes, g scaled by m row by row)
            scale = op_t._device_arrays(g.device)["m"]
            relayout_slabs(g, mask=b["y"], out=b["ws"], scale=scale)
            op_t._run_spmm_update(g, b["gh"], use_m=scale is not None, workspace=b["ws"], workspace_ready=True,
                                  workspace_prescaled=scale is not None)
        else:
            op_t._run_spmm_update(g, b["gh"], use_m=op_t.col_multiplier is not None,
                                  workspace=b["ws"] if b["copy_g"] else None)
        gh = b["gh"]
        gw = torch.mm(gh.t(), x) if ctx.needs_input_grad[1] else None
        gx = torch.mm(gh, weight) if ctx.needs_input_grad[0] else None
        return gx, gw, None


class CBMGCNLayer(nn.Module):
    """``x -> [relu](A_hat (x W^T))``: the reference's GCN layer (``cbm_gcn.py:27-41``) with the
    activation that follows it in the benchmark model optionally folded in (``relu=True``).
    ``fused=False`` is the plain composition Linear -> ``CBMMatmul`` (-> ``relu``)."""

    def __init__(self, in_channels: int, out_channels: int, operator: cbm_matrix, fused: bool = True, relu: bool = False):
        super().__init__()
        self.lin = nn.Linear(in_channels, out_channels, bias=False)
        nn.init.xavier_uniform_(self.lin.weight)            # 'glorot'
        self.cached_a_t = operator
        self.fused, self.relu = bool(fused), bool(relu)
        self._cache = None
        self._generation = 0                                # forward calls of the fused path so far

    def _layer_buffers(self, n, d, device):
        """Device buffers of the layer for n rows of width d, allocated at the first call."""
        key = (n, d, device)
        if self._cache is not None and self._cache["key"] == key:
            return self._cache
        op = self.cached_a_t
        lib = _lib.hip_lib()
        y = torch.empty((n, d), dtype=torch.float32, device=device)
        gh = torch.empty((n, d), dtype=torch.float32, device=device)
        # Linear output with rows d + 32 floats apart when the library then gathers it in place
        # (plain matrices only: a normalised multiply gains more from scaling its slab-major copy by
        # m -- the entries then carry no coefficient -- than the copy costs: 233k rows x 128, 491
        # entries per row: 2.81 ms with the scaled copy, 3.08 ms gathered in place)
        in_place = False
        tiled = op._device_arrays(device)["tiled"] is not None or op.transposed()._device_arrays(device)["tiled"] is not None
        if d % 32 == 0 and op.col_multiplier is None and not tiled:     # (the plan-based multiply always copies)
            padded = torch.empty((n, d + 32), dtype=torch.float32, device=device)[:, :d]
            in_place = lib.cbm_spmm_workspace_floats(n, d, _ld(padded), _ld(y), _ptr(padded), _ptr(y)) == 0
        h = padded if in_place else torch.empty((n, d), dtype=torch.float32, device=device)
        copy_h = (not in_place) and op.relayout and _wants_workspace(h, y, op.nnz)
        copy_g = op.relayout and _wants_workspace(gh, y, op.transposed().nnz)
        floats = max(op.workspace_floats(n, d, device), op.transposed().workspace_floats(n, d, device))
        copy_h, copy_g = copy_h or tiled, copy_g or tiled
        ws = torch.empty(floats, dtype=torch.float32, device=device) if (copy_h or copy_g or self.relu) else None
        self._cache = {"key": key, "h": h, "y": y, "gh": gh, "ws": ws, "copy_h": copy_h, "copy_g": copy_g,
                       "h_in_place": in_place}
        return self._cache

    def forward(self, x, edge_index=None):
        if self.fused and x.is_cuda:
            return _FusedGCNLayer.apply(x, self.lin.weight, self)
        y = CBMMatmul.apply(self.lin(x), self.cached_a_t, self.cached_a_t.col_multiplier is not None)
        return y.relu() if self.relu else y


class CSRMatmul(torch.autograd.Function):
    """y = A x on the hand-written GPU CSR kernel; backward uses the CSR of A^T."""

    @staticmethod
    def forward(ctx, x, fwd, bwd):
        ctx.bwd = bwd
        x = x.detach().contiguous()
        y = torch.empty_like(x)
        csr_spmm(*fwd[:3], x, y, fwd[3])
        return y

    @staticmethod
    def backward(ctx, g):
        g = g.contiguous()
        gx = torch.empty_like(g)
        csr_spmm(*ctx.bwd[:3], g, gx, ctx.bwd[3])
        return gx, None, None


def csr_operator(edge_index, n: int, values, device):
    """(rowptr, col, val, sched) device tensors of the CSR of a COO list sorted or not."""
    ei = torch.as_tensor(edge_index).to(torch.int64)
    key = ei[0] * n + ei[1]
    order = torch.argsort(key)
    rowptr = torch.zeros(n + 1, dtype=torch.int64)
    rowptr[1:] = torch.cumsum(torch.bincount(ei[0], minlength=n), 0)
    rowptr = rowptr.to(torch.int32)
    col = ei[1][order].to(torch.int32)
    val = None if values is None else values[order].to(torch.float32)
    return (rowptr.to(device), col.to(device), None if val is None else val.to(device),
            schedule_rows(rowptr, batch=DEFAULT_BATCH_ROWS).to(device))


class CSRGCNLayer(nn.Module):
    """Same layer on the plain CSR of the normalised adjacency (the baseline)."""

    def __init__(self, in_channels: int, out_channels: int, fwd, bwd):
        super().__init__()
        self.lin = nn.Linear(in_channels, out_channels, bias=False)
        nn.init.xavier_uniform_(self.lin.weight)
        self.fwd, self.bwd = fwd, bwd

    def forward(self, x, edge_index=None):
        return CSRMatmul.apply(self.lin(x), self.fwd, self.bwd)


class TwoLayerGCN(nn.Module):
    """first layer -> ReLU -> last layer (``benchmark_gcn_cpu.py:70-89`` with num_layers = 2).
    ``relu_between=False`` when the first layer applies the ReLU itself."""

    def __init__(self, first: nn.Module, last: nn.Module, relu_between: bool = True):
        super().__init__()
        self.first_layer, self.last_layer = first, last
        self.relu_between = bool(relu_between)

    def forward(self, x, edge_index=None):
        h = self.first_layer(x, edge_index)
        return self.last_layer(h.relu() if self.relu_between else h, edge_index)
