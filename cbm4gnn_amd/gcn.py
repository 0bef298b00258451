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
back (so they have no usable backward), aggregation here is ``CBMMatmul``: backward is the same
CBM multiply with the transposed operator.
"""
from __future__ import annotations

import torch
from torch import nn

from .cbm import CBMMatmul, cbm_matrix, csr_spmm, schedule_rows

__all__ = ["CBMGCNLayer", "CSRGCNLayer", "TwoLayerGCN", "build_operator", "csr_operator", "CSRMatmul"]


def build_operator(edge_index, alpha: int = 2, normalized: bool = True, builder: str = "auto") -> cbm_matrix:
    """``cbm_matrix`` of the TRANSPOSED edge list, as the reference's layers build it
    (``cbm_message_passing.py:48-49``; default alpha = 2, ``:8``)."""
    ei = torch.as_tensor(edge_index)
    ei_t = torch.stack([ei[1], ei[0]], dim=0).to(torch.int32)
    return cbm_matrix(ei_t, torch.ones(ei.size(1), dtype=torch.float32), normalized=normalized, alpha=alpha,
                      builder=builder)


class CBMGCNLayer(nn.Module):
    def __init__(self, in_channels: int, out_channels: int, operator: cbm_matrix):
        super().__init__()
        self.lin = nn.Linear(in_channels, out_channels, bias=False)
        nn.init.xavier_uniform_(self.lin.weight)            # 'glorot'
        self.cached_a_t = operator

    def forward(self, x, edge_index=None):
        x = self.lin(x)
        return CBMMatmul.apply(x, self.cached_a_t, self.cached_a_t.col_multiplier is not None)


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
            schedule_rows(rowptr).to(device))


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
    """first layer -> ReLU -> last layer (``benchmark_gcn_cpu.py:70-89`` with num_layers = 2)."""

    def __init__(self, first: nn.Module, last: nn.Module):
        super().__init__()
        self.first_layer, self.last_layer = first, last

    def forward(self, x, edge_index=None):
        return self.last_layer(self.first_layer(x, edge_index).relu(), edge_index)
