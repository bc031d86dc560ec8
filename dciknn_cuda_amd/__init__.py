"""MI355X-native Prioritized DCI k-nearest-neighbour search.

Drop-in for the Python API of niopeng/dciknn_cuda (`DCI`, `MDCI`), backed by
hand-written gfx950 HIP kernels behind a C-ABI shared library.
"""
__version__ = "0.1.0"

__all__ = ["DCI", "MDCI"]


def __getattr__(name):
    # DCI and MDCI need the compiled libraries (there is no fallback: without them this
    # raises ImportError); the build script and the workload generators of this package
    # must be importable before anything is compiled, hence the late import.
    if name in __all__:
        from . import core
        globals().update(DCI=core.DCI, MDCI=core.MDCI)
        return globals()[name]
    raise AttributeError("module %r has no attribute %r" % (__name__, name))
