"""MI355X (gfx950) device backend for CTorch's operator set.

csrc/      hand-written HIP kernels and the extern "C" launch layer (include/ctorch_amd.h)
host/      C++ Tensor / Storage / Ctorch_Scheduler / AutoDiff front-end over that layer
capi.py    ctypes binding of the C ABI, used by the tests and the benchmark
"""
from . import capi  # noqa: F401
