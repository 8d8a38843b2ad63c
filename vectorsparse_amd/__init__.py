"""MI355X (gfx950) column-vector-sparse SpMM / SDDMM: hand-written HIP kernels behind a C ABI.

`colvec_csr` is pure numpy (format, .smtx I/O, synthetic patterns); `ops` needs
torch-ROCm for device memory and the built `libvsparse.so` for everything else.
"""
from . import colvec_csr  # noqa: F401

__all__ = ["colvec_csr"]
