"""cudadma_amd: Python side of the hipDMA host drivers (libcudadma_amd.so, libcudadma_amd_harness.so).

The device library itself is header-only C++ (include/hipDMA.h).  This package
only loads the C ABI declared in include/cudadma_amd.h and include/cudadma_amd_harness.h with ctypes and wraps it
for tests and benchmarks; PyTorch is used by callers for device memory and
streams, never for compute.  Loading fails loudly when the shared library has
not been built: there is no CPU fallback.
"""
from ._lib import (  # noqa: F401
    CALL_GLOBAL,
    CALL_INDEX_AHEAD,
    CALL_LDS_DIRECT_NT,
    CALL_LDS_DIRECT_SC1,
    CALL_MATRIX_GENERIC,
    CALL_MATRIX_GLOBAL,
    CALL_LDS_DIRECT,
    CALL_LDS_DIRECT_SWIZZLE,
    CALL_LDS_SWIZZLE,
    CALL_QUALIFIED,
    CALL_UNQUALIFIED,
    PATTERN_GATHER,
    PATTERN_HALO,
    PATTERN_SCATTER,
    PATTERN_SEQUENTIAL,
    PATTERN_STRIDED,
    Case,
    CudaDMAError,
    PlanQuery,
    RunArgs,
    STATUS_WAIT_GAVE_UP,
    V1Case,
    device_status,
    harness_lib,
    harness_lib_path,
    lib,
    lib_path,
)
from . import examples, harness, plan, workloads  # noqa: F401
