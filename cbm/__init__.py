"""Import-path compatibility: the reference's callers do ``from cbm.cbm import cbm_matrix`` and
``from cbm import cbm_mkl_cpp`` (``gnns/message_passing/cbm_message_passing.py:3``,
``gnns/message_passing/mkl_message_passing.py:3``).  Both resolve to ``cbm4gnn_amd``."""
