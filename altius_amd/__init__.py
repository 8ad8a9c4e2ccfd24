"""altius_amd: an MI355X (gfx950) backend for the altius interpreter's tensor kernels.

Everything computes in libaltius_hip.so (hand-written HIP kernels behind a C ABI,
include/altius_hip.h).  This package is the Python view of that ABI used by the
tests and the benchmark; it contains no arithmetic and has no CPU fallback.
"""
from ._lib import AltiusHipError, LIB_PATH  # noqa: F401
