"""``from cbm import cbm_mkl_cpp`` -> the shim with the reference extension's 13 functions."""
from cbm4gnn_amd.cbm_mkl_cpp import *  # noqa: F401,F403
