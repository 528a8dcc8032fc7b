"""mshadow_amd - MI355X (gfx950) device layer behind mshadow's Tensor<gpu> API.

The product is native: C++ headers under mshadow_amd/mshadow/ (the expression API), HIP
kernels and the C ABI in mshadow_amd/csrc/ (include/mshadow_hip.h). This Python package
only *loads* the built shared libraries with ctypes so that tests and the benchmark can
drive them; it contains no compute path and no fallback: if the library is missing or
no GPU is present, calls raise.
"""
from .capi import (  # noqa: F401
    CASES_SO, HIP_SO, DeviceBuffer, HipError, Library, cases, lib, load_cases, load_lib, load_probe,
)

__all__ = ["lib", "cases", "load_lib", "load_cases", "load_probe", "Library", "DeviceBuffer", "HipError",
           "HIP_SO", "CASES_SO"]
