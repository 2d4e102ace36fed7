"""gfx950 (MI355X) compute backend for OriginDL's hot path.

csrc/   hand-written HIP kernels and the C ABI declared in include/odl_hip.h
lib/    the built shared library (python -m origindl_amd.build)
_lib    ctypes binding generated from the header
capi    torch-tensor convenience over the C ABI for tests and the benchmark
"""
__all__ = ["build", "capi"]
