"""Import-name compatibility: `from dciknn_cuda import DCI, MDCI` keeps working."""
from dciknn_cuda_amd import DCI, MDCI, __version__  # noqa: F401
