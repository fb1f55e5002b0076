"""MI355X-native PagedAttention decode + ReshapeAndCache behind the ATB operator API.

The product is the two shared libraries under lib/ (see build.py):
libatbmi_kernels.so (HIP kernels, C ABI in include/atbmi_kernels.h) and
libatb.so (atb::Operation layer, C++ headers in include/atb/). This package
is the Python driver used by the tests and the benchmark: `binding` (ctypes),
`workloads` (seeded synthetic decode steps) and `torch_atb`, the reference's
torch binding surface (Operation(param).forward) over `binding`.

The directory name is not a Python identifier; import it with
importlib.import_module("ascend-transformer-boost_amd").
"""
from . import binding  # noqa: F401
from . import workloads  # noqa: F401
from . import torch_atb  # noqa: F401
