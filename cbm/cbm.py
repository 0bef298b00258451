"""``from cbm.cbm import cbm_matrix`` -> the MI355X implementation."""
from cbm4gnn_amd.cbm import cbm_matrix, CBMMatmul, csr_spmm  # noqa: F401
