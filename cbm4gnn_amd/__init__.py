"""MI355X-native compressed-binary-matrix (CBM) multiply.

``cbm4gnn_amd.cbm.cbm_matrix`` mirrors the reference's ``cbm.cbm.cbm_matrix``; the top-level
``cbm`` package of this repository re-exports it under the reference's import path.
"""
__version__ = "0.1.0"
