"""ctypes binding of include/cudadma_amd.h (lib()) and include/cudadma_amd_harness.h (harness_lib())."""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))

PATTERN_SEQUENTIAL, PATTERN_STRIDED, PATTERN_GATHER, PATTERN_SCATTER, PATTERN_HALO = range(5)
(CALL_UNQUALIFIED, CALL_GLOBAL, CALL_QUALIFIED, CALL_LDS_DIRECT, CALL_LDS_SWIZZLE, CALL_LDS_DIRECT_SWIZZLE,
 CALL_Q_GLOBAL_CG, CALL_Q_LASTUSE_CS, CALL_Q_VOLATILE_WT, CALL_Q_STREAMING_WB,
 CALL_QG_GLOBAL_CS, CALL_QG_STREAMING_WT, CALL_QG_LASTUSE_CG, CALL_QG_VOLATILE_WB,
 CALL_LDS_DIRECT_SC1, CALL_LDS_DIRECT_NT, CALL_INDEX_AHEAD) = range(17)
# the qualifier matrix: source known to be global / generic source (the latter also run LDS -> global)
STATUS_WAIT_GAVE_UP = 1
NOALLOC_MAX_PHASES = 1 << 20
CALL_MATRIX_GLOBAL = (CALL_Q_GLOBAL_CG, CALL_Q_LASTUSE_CS, CALL_Q_VOLATILE_WT, CALL_Q_STREAMING_WB)
CALL_MATRIX_GENERIC = (CALL_QG_GLOBAL_CS, CALL_QG_STREAMING_WT, CALL_QG_LASTUSE_CG, CALL_QG_VOLATILE_WB)

PATTERN_NAMES = {
    PATTERN_SEQUENTIAL: "sequential",
    PATTERN_STRIDED: "strided",
    PATTERN_GATHER: "gather",
    PATTERN_SCATTER: "scatter",
    PATTERN_HALO: "halo",
}


class CudaDMAError(RuntimeError):
    pass


class Case(ctypes.Structure):
    """struct cudadma_case"""
    _fields_ = [(n, ctypes.c_int) for n in (
        "pattern", "warp_specialized", "level", "alignment", "bytes_per_thread", "bytes_per_elmt",
        "dma_threads", "num_elmts", "radius", "corners", "dimx", "dimy")]

    def __repr__(self):
        return "Case(" + ", ".join(f"{n}={getattr(self, n)}" for n, _ in self._fields_) + ")"


class V1Case(ctypes.Structure):
    """struct cudadma_v1_case_t"""
    _fields_ = [(n, ctypes.c_int) for n in (
        "pattern", "warp_specialized", "bytes_per_elmt", "num_elmts", "src_stride", "dst_stride",
        "dma_threads", "block_threads", "window_bytes")]


class PlanQuery(ctypes.Structure):
    """struct cudadma_plan_query"""
    _fields_ = [(n, ctypes.c_int) for n in (
        "pattern", "alignment", "bytes_per_thread", "bytes_per_elmt", "dma_threads", "num_elmts",
        "src_stride", "dst_stride", "radius", "corners", "dimx", "dimy", "pitch")] + [("index", ctypes.c_void_p),
                                                                                       ("dst_pitch", ctypes.c_int)]


class RunArgs(ctypes.Structure):
    """struct cudadma_run"""
    _fields_ = [
        ("d_in", ctypes.c_void_p), ("d_out", ctypes.c_void_p), ("d_index", ctypes.c_void_p),
        ("lds_bytes", ctypes.c_int), ("src_offset_bytes", ctypes.c_int), ("dst_offset_bytes", ctypes.c_int),
        ("src_stride", ctypes.c_int), ("dst_stride", ctypes.c_int), ("pitch", ctypes.c_int),
        ("call_style", ctypes.c_int), ("two_phase", ctypes.c_int), ("reps", ctypes.c_int),
        ("rep_src_bytes", ctypes.c_int), ("rep_index_elmts", ctypes.c_int),
        ("reverse", ctypes.c_int), ("out_bytes", ctypes.c_int),
        ("rt_bytes_per_elmt", ctypes.c_int), ("rt_dma_threads", ctypes.c_int), ("rt_num_elmts", ctypes.c_int),
        ("rt_dimx", ctypes.c_int), ("rt_dimy", ctypes.c_int),
        ("dst_pitch", ctypes.c_int),
        ("in_bytes", ctypes.c_size_t), ("out_capacity", ctypes.c_size_t), ("index_elmts", ctypes.c_int),
    ]


def lib_path():
    return os.path.join(_HERE, "libcudadma_amd.so")


def harness_lib_path():
    return os.path.join(_HERE, "libcudadma_amd_harness.so")


_lib = None
_harness_lib = None


def _load(path):
    if not os.path.exists(path):
        raise CudaDMAError(
            f"{path} is missing: build it with `make -C cudadma_amd/csrc` "
            "(or python -c 'import __graft_entry__ as g; g.build()'); there is no fallback path")
    return ctypes.CDLL(path, mode=ctypes.RTLD_GLOBAL)


def _declare(L, signatures):
    for name, argtypes in signatures.items():
        fn = getattr(L, name)
        fn.restype = ctypes.c_int
        fn.argtypes = argtypes


def lib():
    """The workloads, probes, examples and planner; raises when the library has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    L = _load(lib_path())
    vp, ci, cs = ctypes.c_void_p, ctypes.c_int, ctypes.c_size_t
    L.cudadma_last_error.restype = ctypes.c_char_p
    L.cudadma_last_error.argtypes = []
    L.cudadma_device_cus.restype = ci
    _declare(L, _WORKLOAD_SIGNATURES)
    L.cudadma_plan_map.restype = ci
    L.cudadma_plan_map.argtypes = [ctypes.POINTER(PlanQuery), ctypes.c_longlong, ctypes.c_longlong, vp, cs,
                                   ctypes.POINTER(ci)]
    L.cudadma_plan_extents.restype = ci
    L.cudadma_plan_extents.argtypes = [ctypes.POINTER(PlanQuery), ctypes.POINTER(ctypes.c_longlong * 4)]
    L.cudadma_diagnose.restype = ci
    L.cudadma_diagnose.argtypes = [ci] * 8
    L.cudadma_set_tuning.restype = ci
    L.cudadma_set_tuning.argtypes = [ctypes.c_char_p, ci]
    L.cudadma_variant_name.restype = ctypes.c_char_p
    L.cudadma_variant_name.argtypes = [ci, ci]
    L.cudadma_perf_sequential.restype = ctypes.c_longlong
    L.cudadma_perf_sequential.argtypes = [vp, cs, vp, ci, ci, ci, ci, ci, ci, ci, vp]
    L.cudadma_probe_memory.restype = ctypes.c_longlong
    L.cudadma_probe_memory.argtypes = [ci, vp, vp, cs, ci, vp]
    L.cudadma_probe_pattern.restype = ctypes.c_longlong
    L.cudadma_probe_pattern.argtypes = [ci, vp, vp, vp, cs, cs, ci, vp]
    L.cudadma_transpose_splits.restype = ci
    L.cudadma_transpose_splits.argtypes = [ctypes.POINTER(ci), ci]
    L.cudadma_example_variant_name.restype = ctypes.c_char_p
    L.cudadma_example_variant_name.argtypes = [ci, ci]
    _lib = L
    return L


def harness_lib():
    """The known-answer cases and self-tests of the DMA objects: a library of its own that needs the main one
    (error text, failure record), which is therefore loaded first; raises when either has not been built."""
    global _harness_lib
    if _harness_lib is not None:
        return _harness_lib
    lib()
    L = _load(harness_lib_path())
    ci = ctypes.c_int
    L.cudadma_num_cases.restype = ci
    L.cudadma_get_case.restype = ci
    L.cudadma_get_case.argtypes = [ci, ctypes.POINTER(Case)]
    L.cudadma_run_case.restype = ci
    L.cudadma_run_case.argtypes = [ci, ctypes.POINTER(RunArgs), ctypes.c_void_p]
    _declare(L, _HARNESS_SIGNATURES)
    L.cudadma_v1_get_case.restype = ci
    L.cudadma_v1_get_case.argtypes = [ci, ctypes.POINTER(V1Case)]
    L.cudadma_v1_case_text.restype = ctypes.c_char_p
    L.cudadma_v1_case_text.argtypes = [ci]
    _harness_lib = L
    return L


_vp, _ci, _cs, _u64 = ctypes.c_void_p, ctypes.c_int, ctypes.c_size_t, ctypes.c_uint64

# name -> argtypes of the workload entry points (all return int)
_WORKLOAD_SIGNATURES = {
    "cudadma_fill_uniform": [_vp, _cs, _u64, _vp],
    "cudadma_fill_indices": [_vp, _cs, ctypes.c_uint32, _u64, _vp],
    "cudadma_fill_normal_bf16": [_vp, _cs, _u64, _vp],
    "cudadma_plain_copy": [_vp, _vp, _cs, _vp],
    "cudadma_num_variants": [_ci],
    "cudadma_set_workgroups_per_cu": [_ci],
    "cudadma_sequential_copy": [_vp, _vp, _cs, _ci, _vp],
    "cudadma_strided_transpose": [_vp, _vp, _ci, _ci, _vp],
    "cudadma_fill_permutation": [_vp, _ci, _u64, _vp],
    "cudadma_scatter_copy": [_vp, _vp, _vp, _cs, _cs, _ci, _vp],
    "cudadma_gather_copy": [_vp, _vp, _vp, _cs, _cs, _ci, _vp],
    "cudadma_gather_rowsum": [_vp, _vp, _vp, _cs, _cs, _ci, _vp],
    "cudadma_halo_stencil": [_vp, _vp, _ci, _ci, _ci, _ci, _vp],
    "cudadma_gemm_bf16": [_vp, _vp, _vp, _ci, _ci, _ci, _ci, _vp],
    "cudadma_probe_clock": [_vp, _ci, _vp],
    "cudadma_device_status": [ctypes.POINTER(ctypes.c_uint), ctypes.POINTER(ctypes.c_uint), _ci, _vp],
    "cudadma_device_status_sources": [],
    "cudadma_example_num_variants": [_ci],
    "cudadma_example_saxpy": [_ci, ctypes.c_float, _vp, _vp, ctypes.c_longlong, _vp],
    "cudadma_example_sgemv": [_ci, _ci, _ci, ctypes.c_float, _vp, _ci, _vp, _vp, _vp],
    "cudadma_example_stencil2d": [_ci, _vp, _vp, _ci, _ci, _ci, _ci, _vp],
}

# name -> argtypes of the harness library's entry points that return int and take only plain words
_HARNESS_SIGNATURES = {
    "cudadma_selftest_bounded_wait": [_vp, _vp],
    "cudadma_selftest_split_wait": [_vp, _ci, _vp],
    "cudadma_selftest_global_handoff": [_vp, _vp, _ci, _vp],
    "cudadma_selftest_global_handoff_lds_only": [_vp, _vp, _ci, _vp],
    "cudadma_selftest_global_handoff_noalloc": [_vp, _ci, _vp],
    "cudadma_selftest_all_ids": [_vp, _ci, _vp],
    "cudadma_v1_num_cases": [],
    "cudadma_v1_run_case": [_ci, _vp, _vp, _vp, _vp],
}


def check(rc):
    if rc != 0:
        raise CudaDMAError(f"libcudadma_amd error {rc}: {lib().cudadma_last_error().decode()}")


def device_status(clear=True, stream=None):
    """(status bits, wavefronts whose wait gave up) summed over the library's kernels since the last clear."""
    bits, count = ctypes.c_uint(0), ctypes.c_uint(0)
    check(lib().cudadma_device_status(ctypes.byref(bits), ctypes.byref(count), int(bool(clear)), ctypes.c_void_p(stream or 0)))
    return bits.value, count.value


def exported_symbols():
    """Every extern "C" symbol include/cudadma_amd.h declares."""
    return ["cudadma_last_error", "cudadma_device_cus", "cudadma_variant_name", "cudadma_example_variant_name",
            "cudadma_perf_sequential", "cudadma_probe_memory", "cudadma_probe_pattern", "cudadma_transpose_splits",
            "cudadma_plan_map", "cudadma_plan_extents", "cudadma_diagnose", "cudadma_set_tuning"] + list(_WORKLOAD_SIGNATURES)


def harness_exported_symbols():
    """Every extern "C" symbol include/cudadma_amd_harness.h declares."""
    return ["cudadma_num_cases", "cudadma_get_case", "cudadma_run_case", "cudadma_v1_get_case",
            "cudadma_v1_case_text"] + list(_HARNESS_SIGNATURES)
