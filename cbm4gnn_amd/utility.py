"""Input contract of the CBM builder, restated from the reference's validators
(``/root/reference/cbm/utility.py:4-29``): shape (2, E), ids start at 0 and are contiguous,
no duplicate edges."""
from torch import Tensor

__all__ = ["check_edge_index", "check_edge_index_contiguous", "check_edge_index_coalesced",
           "check_edge_index_indices", "check_edge_index_shape"]


def check_edge_index_shape(edge_index: Tensor) -> None:
    if edge_index.dim() != 2 or edge_index.shape[0] != 2:
        raise ValueError("Edge index should have shape (2, num_edges)")


def check_edge_index_indices(edge_index: Tensor) -> None:
    if edge_index.min() != 0:
        raise ValueError("Edge index should start from 0")


def check_edge_index_contiguous(edge_index: Tensor) -> None:
    if edge_index.unique().size(0) != edge_index.max() + 1:
        raise ValueError("Edge index is not contiguous")


def check_edge_index_coalesced(edge_index: Tensor) -> None:
    if edge_index.shape[1] != edge_index.unique(dim=1).shape[1]:
        raise ValueError("Edge index is not coalesced")


def check_edge_index(edge_index: Tensor) -> None:
    check_edge_index_shape(edge_index)
    check_edge_index_indices(edge_index)
    check_edge_index_contiguous(edge_index)
    check_edge_index_coalesced(edge_index)
