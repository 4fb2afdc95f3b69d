"""thrust_amd — Python harness over the gfx950 device system for Thrust.

The product is the C-ABI library `thrust_amd/lib/libthrust_cdna4.so` (sources in
`thrust_amd/csrc/`, declarations in `include/thrust_cdna4.h`) and the C++ dispatch headers in
`include/thrust/`.  This package is the thin harness the tests and the benchmark use to call
the C ABI on torch-owned device memory; torch supplies allocations and streams only.
"""
from . import capi  # noqa: F401
from .api import (exclusive_scan, exclusive_scan_by_key, histogram_even,  # noqa: F401
                  inclusive_scan, inclusive_scan_by_key, reduce_by_key, sort, sort_by_key)
