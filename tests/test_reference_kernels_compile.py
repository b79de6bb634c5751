"""The drop-in boundary on the reference's own text: the device kernels of the reference's v2 test programs
(src/tests/test_sequential/cudaDMA_test_sequential_v2.cu:53-391, src/tests/test_strided/cudaDMA_test_strided_v2.cu,
src/tests/test_indirect/cudaDMA_test_indirect_v2.cu: the special_xfer_* kernels, 22 in all) and of its halo test
(src/tests/test_halo/cudaDMA_test_halo.cu:52-232) are read from the reference tree when the test runs, written
unchanged into a scratch file behind `#include "cudaDMAv2.h"` (or "cudaDMA.h") of this repository and the macros
their Makefiles pass (-DALIGNMENT ... with thread counts in multiples of 64), and compiled for gfx950.  Nothing of
the reference is kept in this repository; where the reference tree is absent the test is skipped.  Device pass
only, no GPU needed: this checks names, template parameters, constructor forms and call forms, not results (the
known-answer harness does that)."""
import os
import re
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
REFERENCE_TESTS = "/root/reference/src/tests"
_V2_PROGRAMS = {
    "sequential": "test_sequential/cudaDMA_test_sequential_v2.cu",
    "strided": "test_strided/cudaDMA_test_strided_v2.cu",
    "indirect": "test_indirect/cudaDMA_test_indirect_v2.cu",
}
# values for the macros the reference's param_sweep_v2.py passes on the compiler's command line
_MACRO_SETS = [
    dict(ALIGNMENT=16, BYTES_PER_THREAD=64, BYTES_PER_ELMT=1024, DMA_THREADS=128, NUM_ELMTS=8, ALIGN_OFFSET=0),
    dict(ALIGNMENT=4, BYTES_PER_THREAD=16, BYTES_PER_ELMT=132, DMA_THREADS=64, NUM_ELMTS=5, ALIGN_OFFSET=1),
    dict(ALIGNMENT=8, BYTES_PER_THREAD=24, BYTES_PER_ELMT=40, DMA_THREADS=192, NUM_ELMTS=33, ALIGN_OFFSET=2),
]
_END_OF_FUNCTION = re.compile(r"^\}[ \t]*$", re.M)


def _hipcc():
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(hipcc):
        pytest.skip("no hipcc")
    return hipcc


def _compile(tmp_path, source):
    src = tmp_path / "reference_kernels.hip"
    src.write_text(source)
    cmd = [_hipcc(), "-std=c++17", "-O1", "--offload-arch=gfx950", "--cuda-device-only", "-c", str(src), "-o",
           str(tmp_path / "k.o"), "-I", os.path.join(ROOT, "include"), "-Xclang", "-target-feature", "-Xclang",
           "-packed-fp32-ops"]
    res = subprocess.run(cmd, capture_output=True, text=True, timeout=600)
    assert res.returncode == 0, "\n".join(l for l in res.stderr.splitlines() if "error" in l)[:4000]


def _kernels(text):
    """Every function of `text` that starts with __global__ in column 0, up to its closing brace in column 0."""
    out = []
    for m in re.finditer(r"^__global__", text, re.M):
        out.append(text[m.start():_END_OF_FUNCTION.search(text, m.start()).end()])
    return out


@pytest.mark.parametrize("macros", _MACRO_SETS, ids=lambda m: f"A{m['ALIGNMENT']}-E{m['BYTES_PER_ELMT']}-T{m['DMA_THREADS']}")
@pytest.mark.parametrize("program", sorted(_V2_PROGRAMS))
def test_reference_v2_test_kernels_compile_with_the_changed_include(tmp_path, program, macros):
    path = os.path.join(REFERENCE_TESTS, _V2_PROGRAMS[program])
    if not os.path.exists(path):
        pytest.skip("the reference tree is not present")
    kernels = _kernels(open(path).read())
    assert len(kernels) >= 6, f"expected the special_xfer_* kernels of {path}"
    defines = "".join(f"#define {k} {v}\n" for k, v in macros.items())
    _compile(tmp_path, '#include "cudaDMAv2.h"\n' + defines + "\n".join(kernels) + "\n")


def test_reference_halo_test_kernel_compiles_with_the_changed_include(tmp_path):
    path = os.path.join(REFERENCE_TESTS, "test_halo/cudaDMA_test_halo.cu")
    if not os.path.exists(path):
        pytest.skip("the reference tree is not present")
    text = open(path).read()
    start = text.index("template<typename TYPE>")                    # its element helpers (initialize, get_val) come first
    end = _END_OF_FUNCTION.search(text, text.index("dma_ld_test")).end()
    instantiations = "".join(
        f"template __global__ void dma_ld_test<{a}, 0, {t}, {r}, {c}>({t}*, {t}*, int, int, int, int, int, int);\n"
        for a, t, r, c in ((16, "float", 4, "false"), (8, "float2", 2, "true"), (4, "float", 1, "false"), (16, "float4", 3, "true")))
    _compile(tmp_path, '#include <stdio.h>\n#include <stdlib.h>\n#include <assert.h>\n#include <math.h>\n#include "cudaDMA.h"\n'
             + text[start:end] + "\n" + instantiations)


REFERENCE_EXAMPLES = "/root/reference/src/examples"


def test_reference_saxpy_kernels_compile_with_the_changed_include(tmp_path):
    """src/examples/saxpy/saxpy_cudaDMA_kernel.cu:54-400, the eight kernels (two of them on cudaDMASequential), with the
    parameters of its params_directed.h restated in multiples of 64 threads."""
    path = os.path.join(REFERENCE_EXAMPLES, "saxpy/saxpy_cudaDMA_kernel.cu")
    if not os.path.exists(path):
        pytest.skip("the reference tree is not present")
    kernels = _kernels(open(path).read())
    assert len(kernels) == 8
    params = ("#define CTA_COUNT 256\n#define COMPUTE_THREADS_PER_CTA (64 * 4)\n#define NUM_ITERS 64\n"
              "#define DMA_THREADS_PER_LD (64 * 1)\n#define BYTES_PER_DMA_THREAD 32\n"
              "#define DMA_SZ (4 * COMPUTE_THREADS_PER_CTA)\n#define DMA_THREADS_PER_CTA (4 * DMA_THREADS_PER_LD)\n")
    _compile(tmp_path, '#include <stdio.h>\n#include <stdlib.h>\n#include "cudaDMA.h"\n' + params + "\n".join(kernels) + "\n")


@pytest.mark.parametrize("config", ["VEC_SINGLE", "VEC_DOUBLE", "VEC_MANUAL", "BOTH_SINGLE", "BOTH_DOUBLE", "BOTH_MANUAL", "MAT_SINGLE"])
def test_reference_sgemv_kernels_compile_with_the_changed_include(tmp_path, config):
    """src/examples/sgemv/sgemv_dma.cu:72-620: its seven configurations (cudaDMASequential for the vector,
    cudaDMAStrided for the matrix panel), each compiled under its own -D switch as its Makefile does, with
    DMA_THREADS_PER_LD 64 instead of 32.  BOTH_DOUBLE carries a typing slip in the reference
    (`blockIdx.x**COMPUTE_THREADS_PER_CTA`, :468,:479) that no compiler accepts; it is read as one `*`."""
    path = os.path.join(REFERENCE_EXAMPLES, "sgemv/sgemv_dma.cu")
    if not os.path.exists(path):
        pytest.skip("the reference tree is not present")
    text = open(path).read()
    last = "#endif // MAT_SINGLE"
    body = text[text.index("#define SIZE_N"):text.index(last) + len(last)]
    body = re.sub(r"(#define DMA_THREADS_PER_LD\s+)32", r"\g<1>64", body).replace("blockIdx.x**COMPUTE", "blockIdx.x*COMPUTE")
    _compile(tmp_path, f"#define {config} 1\n" + '#include <cstdio>\n#include "cudaDMA.h"\n' + body + "\n")


@pytest.mark.parametrize("header", ["warp_specialized_single_buffer", "warp_specialized_double_buffer",
                                    "warp_specialized_manual_buffer", "non_warp_specialized_single_buffer",
                                    "non_warp_specialized_double_buffer"])
def test_reference_stencil_kernels_compile_with_the_changed_include(tmp_path, header):
    """src/examples/stencil/*_buffer.h with stencil_math.h: the five buffering styles on CudaDMAStrided, instantiated
    with the directed parameters of params_directed.h:17-24 (32 x 4 tiles, radius 4, 12 x 16 bytes per thread) and
    one DMA wavefront per load.  non_warp_specialized_double_buffer.h calls member templates of a dependent type
    without the `template` keyword, which nvcc lets pass and clang does not: the keyword is put in here."""
    base = os.path.join(REFERENCE_EXAMPLES, "stencil")
    if not os.path.exists(os.path.join(base, header + ".h")):
        pytest.skip("the reference tree is not present")

    def without_includes(path):
        return "\n".join(l for l in open(path).read().splitlines() if not l.strip().startswith("#include"))
    kernel = without_includes(os.path.join(base, header + ".h"))
    kernel = re.sub(r"(\w)\.(start_xfer_async|wait_xfer_finish|execute_dma)<", r"\1.template \2<", kernel)
    args = "16, 12 * 16, 32, 4, 4" + ("" if header.startswith("non") else ", 64")
    _compile(tmp_path, '#include "cudaDMAv2.h"\n' + without_includes(os.path.join(base, "stencil_math.h")) + "\n" + kernel +
             f"\ntemplate __global__ void stencil_2D_{header}<{args}>(const float2*, float2*, const int, const int, const int, const int);\n")


def test_reference_perf_kernels_compile_with_the_changed_include(tmp_path):
    """src/perf/sequential/perf_sequential.cu:52-224: the four kernel shapes of the read-bandwidth probe
    (non_specialized, single_buffer, double_buffer, manual_buffer on cudaDMASequential), instantiated with the
    directed parameters of its params_directed.h (float, ALIGNMENT 16, 4096-byte elements, 32 loops) and two DMA
    wavefronts of 64 in place of two warps of 32."""
    path = "/root/reference/src/perf/sequential/perf_sequential.cu"
    if not os.path.exists(path):
        pytest.skip("the reference tree is not present")
    text = open(path).read()
    start = text.index("template<typename T, int ALIGNMENT, int BYTES_PER_ELMT, int TOTAL_THREADS, int NUM_LOOPS>")
    end = _END_OF_FUNCTION.search(text, text.index("void manual_buffer")).end()
    instantiations = ("template __global__ void non_specialized<float, 16, 4096, 256, 32>(const float*, float*, bool);\n" +
                      "".join(f"template __global__ void {k}<float, 16, 4096, 128, 32>(const float*, float*, int, bool);\n"
                              for k in ("single_buffer", "double_buffer", "manual_buffer")))
    _compile(tmp_path, '#include "cudaDMA.h"\n' + text[start:end] + "\n" + instantiations)
