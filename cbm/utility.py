"""``from cbm.utility import check_edge_index`` -> the input contract of the builder."""
from cbm4gnn_amd.utility import *  # noqa: F401,F403
