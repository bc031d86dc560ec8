"""MI355X-native Prioritized DCI k-nearest-neighbour search.

Drop-in for the Python API of niopeng/dciknn_cuda (`DCI`, `MDCI`), backed by
hand-written gfx950 HIP kernels behind a C-ABI shared library.
"""
__version__ = "0.1.0"

from .core import DCI, MDCI  # noqa: F401
