"""MI355X-native FP32 CSR SpMM behind the entry points of fan1997/HP-SpMM-SDDMM.

  capi    ctypes binding of libhpspmm.so (include/hpspmm.h): the HIP path
  graphs  seeded synthetic inputs of the benchmark configurations
  build   in-tree build of the native libraries

The directory name carries a hyphen, so load the package with
importlib.import_module("hp-spmm-sddmm_amd").
"""
from . import capi, graphs  # noqa: F401

__all__ = ["capi", "graphs"]
