"""Sparse-format flags (reference src/graph_storage.h:32-36, python/gs/format.py)."""
_DCSR = 16
_DCSC = 8
_CSR = 4
_CSC = 2
_COO = 1
