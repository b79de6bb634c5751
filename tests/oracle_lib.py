"""ctypes binding of oracle/liboracle.so (the CPU checker; test infrastructure only)."""
import ctypes
import os
import subprocess

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
ORACLE_DIR = os.path.join(ROOT, "oracle")
_vp, _ci, _cs, _u64 = ctypes.c_void_p, ctypes.c_int, ctypes.c_size_t, ctypes.c_uint64

_SIGS = {
    "oracle_num_threads": (_ci, []),
    "oracle_splitmix64": (_u64, [_u64]),
    "oracle_hash32": (ctypes.c_uint32, [_u64, _u64]),
    "oracle_fill_uniform": (None, [_vp, _cs, _u64]),
    "oracle_fill_ramp": (None, [_vp, _cs]),
    "oracle_fill_indices": (None, [_vp, _cs, ctypes.c_uint32, _u64]),
    "oracle_fill_permutation": (None, [_vp, _ci, _u64]),
    "oracle_fill_normal_bf16": (None, [_vp, _cs, _u64]),
    "oracle_f32_to_bf16": (ctypes.c_uint16, [ctypes.c_float]),
    "oracle_bf16_to_f32": (ctypes.c_float, [ctypes.c_uint16]),
    "oracle_sequential": (None, [_vp, _vp, _cs]),
    "oracle_strided": (None, [_vp, _vp, _ci, _ci, _ci, _ci]),
    "oracle_strided_swizzled": (None, [_vp, _vp, _ci, _ci, _ci, _ci, _ci]),
    "oracle_gather": (None, [_vp, _vp, _vp, _ci, _ci, _ci]),
    "oracle_scatter": (None, [_vp, _vp, _vp, _ci, _ci, _ci]),
    "oracle_halo": (None, [_vp, _vp, _ci, _ci, _ci, _ci, _ci, _ci]),
    "oracle_halo_pitched": (None, [_vp, _vp, _ci, _ci, _ci, _ci, _ci, _ci, _ci]),
    "oracle_halo_check": (_ci, [_vp, _vp, _ci, _ci, _ci, _ci, _ci, _ci]),
    "oracle_copy": (None, [_vp, _vp, _cs]),
    "oracle_transpose": (None, [_vp, _vp, _ci]),
    "oracle_gather_copy": (None, [_vp, _vp, _vp, _cs, _ci]),
    "oracle_gather_rowsum": (None, [_vp, _vp, _vp, _cs, _ci, _ci]),
    "oracle_scatter_copy": (None, [_vp, _vp, _vp, _cs, _ci]),
    "oracle_stencil25": (None, [_vp, _vp, _ci, _ci, _ci, _ci]),
    "oracle_gemm_bf16": (None, [_vp, _vp, _vp, _ci, _ci, _ci]),
    "oracle_gemm_bf16_entry": (ctypes.c_float, [_vp, _vp, _ci, _ci, _ci, _ci]),
    "oracle_saxpy": (None, [ctypes.c_float, _vp, _vp, _cs]),
    "oracle_sgemv": (None, [_ci, _ci, ctypes.c_float, _vp, _ci, _vp, _vp]),
    "oracle_stencil2d": (None, [_vp, _vp, _ci, _ci, _ci, _ci, _ci]),
}

_lib = None


def load():
    global _lib
    if _lib is not None:
        return _lib
    path = os.path.join(ORACLE_DIR, "liboracle.so")
    if not os.path.exists(path):
        subprocess.check_call(["make", "-C", ORACLE_DIR], stdout=subprocess.DEVNULL)
    L = ctypes.CDLL(path)
    for name, (res, args) in _SIGS.items():
        fn = getattr(L, name)
        fn.restype = res
        fn.argtypes = args
    _lib = L
    return L


def ptr(a, byte_offset=0):
    """Address of a numpy array's data (plus an offset) as c_void_p."""
    return ctypes.c_void_p(a.ctypes.data + byte_offset)


def uniform(n, seed):
    out = np.empty(n, dtype=np.float32)
    load().oracle_fill_uniform(ptr(out), n, seed)
    return out


def ramp(n):
    out = np.empty(n, dtype=np.float32)
    load().oracle_fill_ramp(ptr(out), n)
    return out


def permutation(log2_n, seed):
    out = np.empty(1 << log2_n, dtype=np.int32)
    load().oracle_fill_permutation(ptr(out), log2_n, seed)
    return out


def indices(n, n_records, seed):
    out = np.empty(n, dtype=np.int32)
    load().oracle_fill_indices(ptr(out), n, n_records, seed)
    return out
