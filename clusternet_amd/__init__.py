"""clusternet_amd: MI355X (gfx950) implementation of clusterNet's matrix-multiply and 8-bit codec
path.  The product is the C-ABI library libcnhip.so (see include/cnhip.h) and the C++
ClusterNet / Matrix facade over it; this package is the thin Python host binding used by the
tests and the benchmark.  PyTorch appears only as the owner of device memory and streams.
"""
from ._lib import (CnError, absmax, absmax_compression_8bit, compression_8bit, compression_8bit_axpy, decompression_8bit, decompression_8bit_axpy, dot, dotT,
                   Tdot, gemm, gemm_w8, init, lib, lib_path, num_compute_units, rmsprop_update, table)

__all__ = ["CnError", "absmax", "absmax_compression_8bit", "compression_8bit", "compression_8bit_axpy", "decompression_8bit", "decompression_8bit_axpy", "dot",
           "dotT", "Tdot", "gemm", "gemm_w8", "init", "lib", "lib_path", "num_compute_units", "rmsprop_update",
           "table"]
