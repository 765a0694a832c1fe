"""MI355X-native compact-counter update (MotifCL's CounterStateLinear optimizer step).

The computation lives in libmotifcl_amd.so (HIP kernels behind the C ABI of
include/motifcl_amd.h).  `motifcl_amd.ops` is a thin ctypes front for device
tensors; it raises if the library has not been built.
"""
from .lib import LIB_PATH, LibraryMissing, MccError, load  # noqa: F401
