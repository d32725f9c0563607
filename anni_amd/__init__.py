"""anni_amd -- MI355X (gfx950) backend of AnnI's optimizer step.

The product is the C-ABI shared library ``libanni_gpu_hip.so`` (headers under
``include/``).  This package is the thin Python host side used by the tests and
the benchmark: a ctypes loader (``anni_amd.lib``), a mirror of the reference's
``lm_adam`` interface over the device arena (``anni_amd.lm_adam``) and the
tensor lists of the reference's model sizes (``anni_amd.layout``).
"""
from .lib import load, LibraryMissing  # noqa: F401
