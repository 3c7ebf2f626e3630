"""coconet_amd: MI355X (gfx950) backend for CoCoNet's fused reduce + optimizer-update kernels.

The product is the C-ABI shared library `coconet_amd/lib/libcoconet_hip.so` (sources in
`coconet_amd/csrc`, interface in `include/coconet_hip.h`) and the C++ DSL front end in `coconet_amd/dsl`.
`coconet_amd.capi` is the ctypes binding used by the tests and the benchmark.
"""
__version__ = "0.1.0"
