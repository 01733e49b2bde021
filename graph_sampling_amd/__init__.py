"""MI355X-native graph-sampling engine: hand-written HIP kernels behind a C ABI,
with a host layer mirroring the `gs` Graph / Matrix surface of
czkkkkkk/graph_sampling."""
from .format import _COO, _CSC, _CSR, _DCSC, _DCSR  # noqa: F401
