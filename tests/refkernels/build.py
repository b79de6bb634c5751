"""Builds tests/refkernels/_build/libref_kernels.so: the device kernels of the reference's own v2 test programs, compiled from the
reference tree where it lies (never copied into this repository) against this repository's cudaDMAv2.h, each behind
a small launcher that does what the reference's run_experiment() does (one workgroup; for the warp-specialised kernels
one compute wavefront of 64 threads plus DMA_THREADS DMA threads; dynamic LDS of the buffer size):

    src/tests/test_sequential/cudaDMA_test_sequential_v2.cu   kernels :52-391, launch :432-480
    src/tests/test_strided/cudaDMA_test_strided_v2.cu         kernels :52-535, launch :586-650
    src/tests/test_indirect/cudaDMA_test_indirect_v2.cu       kernels :55-536, launch :590-652
    src/tests/test_halo/cudaDMA_test_halo.cu                  kernel :180-232 with its element helpers :52-90
                                                              (first-generation cudaDMAHalo, "cudaDMA.h"), launch :261-268
    src/examples/saxpy/saxpy_cudaDMA_kernel.cu                the eight saxpy kernels :54-420 (two of them on
                                                              cudaDMASequential), launch saxpy_cudaDMA.cu:138
    src/examples/stencil/*_buffer.h + stencil_math.h          the five buffering styles of the 2-D stencil on
                                                              CudaDMAStrided, launch cudaDMA_stencil2D.cu:118-185
    src/perf/sequential/perf_sequential.cu                    the four kernel shapes of the read-bandwidth probe
    src/examples/sgemv/sgemv_dma.cu                           its seven DMA kernels :141-620 (cudaDMASequential for the
                                                              vector, cudaDMAStrided for the matrix panel), each under
                                                              its own -D switch with its own sizes :79-133, launch :845-856

The kernels take their parameters as template arguments named like the macros the reference's Makefiles pass
(-DALIGNMENT=... and so on); here the template heads are left out and the macros of one parameter set are defined in
front of the text, one translation unit per (program, parameter set).  Test infrastructure only: the GPU tests run
these kernels (the code under test is this repository's header; the reference supplies the callers) and compare their
output with the oracle's closed forms.

    python tests/refkernels/build.py          # needs /root/reference and hipcc; writes only into tests/refkernels/_build/
    CUDADMA_REFKERNEL_DRAWS=84 python tests/refkernels/build.py      # plus 84 seeded draws from the reference's random sweep
"""
import concurrent.futures
import os
import re
import shutil
import subprocess
import sys
import tempfile

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
REFERENCE_TESTS = "/root/reference/src/tests"
OUT_DIR = os.path.join(HERE, "_build")
OUT = os.path.join(OUT_DIR, "libref_kernels.so")

PROGRAMS = {
    "sequential": "test_sequential/cudaDMA_test_sequential_v2.cu",
    "strided": "test_strided/cudaDMA_test_strided_v2.cu",
    "indirect": "test_indirect/cudaDMA_test_indirect_v2.cu",
}
# Parameter sets (the macros of the reference's param_sweep_v2.py); thread counts in multiples of 64.  ALIGN_OFFSET is
# in floats and keeps the ALIGNMENT; sizes are chosen to hit whole chunks, 4/8/12-byte tails and several steps.
PARAMETER_SETS = {
    "a16_e1024_t128_n8": dict(ALIGNMENT=16, ALIGN_OFFSET=0, BYTES_PER_THREAD=64, BYTES_PER_ELMT=1024, DMA_THREADS=128, NUM_ELMTS=8),
    "a4_e132_t64_n5": dict(ALIGNMENT=4, ALIGN_OFFSET=1, BYTES_PER_THREAD=16, BYTES_PER_ELMT=132, DMA_THREADS=64, NUM_ELMTS=5),
    "a8_e40_t192_n33": dict(ALIGNMENT=8, ALIGN_OFFSET=2, BYTES_PER_THREAD=24, BYTES_PER_ELMT=40, DMA_THREADS=192, NUM_ELMTS=33),
    "a16_e1004_t256_n3": dict(ALIGNMENT=16, ALIGN_OFFSET=4, BYTES_PER_THREAD=32, BYTES_PER_ELMT=1004, DMA_THREADS=256, NUM_ELMTS=3),
    "a16_e6000_t64_n2": dict(ALIGNMENT=16, ALIGN_OFFSET=0, BYTES_PER_THREAD=16, BYTES_PER_ELMT=6000, DMA_THREADS=64, NUM_ELMTS=2),
}
COMPUTE_THREADS = 64          # one compute wavefront, where the reference launches one warp
MANIFEST = os.path.join(OUT_DIR, "parameter_sets.json")       # the sets the library on disk was built with
LDS_BUDGET = 60 * 1024        # bytes of dynamic LDS a drawn set may ask for (64 KB is what a launch gets without more ado)


def drawn_parameter_sets(count, seed=20240517):
    """`count` further parameter sets drawn the way the reference's own random sweep draws them
    (src/tests/test_strided/param_sweep_v2.py:50-71): ALIGNMENT from {4, 8, 16}, an offset in floats that keeps it,
    BYTES_PER_THREAD = ALIGNMENT x 1..8, an element of |N(256, 256)| floats, 1..32 elements, DMA thread groups of 1..8
    wavefronts of 64 (the reference: 1..16 warps of 32).  Draws whose buffer would not fit the LDS budget are drawn
    again.  Seeded: the same count gives the same sets."""
    import math
    import random
    rng = random.Random(seed)
    sets = {}
    while len(sets) < count:
        alignment = rng.choice([4, 8, 16])
        offset = {4: rng.choice([0, 1, 2, 3]), 8: rng.choice([0, 2]), 16: 0}[alignment]
        bpt = alignment * rng.randint(1, 8)
        floats = abs(int(math.ceil(rng.gauss(256, 256))))
        elmts = rng.randint(1, 32)
        waves = rng.randint(1, 8)
        if floats == 0:
            continue
        per = alignment // 4
        padded = (floats + per - 1) // per * per
        if (elmts * padded + offset) * 4 > LDS_BUDGET:
            continue
        name = f"draw_a{alignment}_o{offset}_b{bpt}_e{floats * 4}_t{waves * 64}_n{elmts}"
        sets[name] = dict(ALIGNMENT=alignment, ALIGN_OFFSET=offset, BYTES_PER_THREAD=bpt, BYTES_PER_ELMT=floats * 4,
                          DMA_THREADS=waves * 64, NUM_ELMTS=elmts)
    return sets


def built_parameter_sets():
    """The parameter sets of the library on disk (its manifest), or the standard ones when there is none."""
    import json
    try:
        with open(MANIFEST) as f:
            return json.load(f)
    except (OSError, ValueError):
        return dict(PARAMETER_SETS)

# kernel numbers of a launcher: 0-3 warp-specialised with four / three / two / one compile-time parameters (the
# sequential program has no "four"), 4-7 the same not warp-specialised
_LAUNCHERS = {
    "sequential": r'''
extern "C" int refk_sequential_@SET@(int which, float* d_in, float* d_out, int* /*unused*/, int single, int qualified, void* stream)
{
  const int buffer_size = BYTES_PER_ELMT / 4 + ALIGN_OFFSET;
  const size_t lds = (size_t)buffer_size * 4;
  hipStream_t s = (hipStream_t)stream;
  const bool one = single != 0, q = qualified != 0;
  switch (which) {
    case 1: hipLaunchKernelGGL(special_xfer_three, dim3(1), dim3(@C@ + DMA_THREADS), lds, s, d_in, d_out, buffer_size, @C@, one, q); break;
    case 2: hipLaunchKernelGGL(special_xfer_two, dim3(1), dim3(@C@ + DMA_THREADS), lds, s, d_in, d_out, buffer_size, @C@, DMA_THREADS, one, q); break;
    case 3: hipLaunchKernelGGL(special_xfer_one, dim3(1), dim3(@C@ + DMA_THREADS), lds, s, d_in, d_out, buffer_size, @C@, DMA_THREADS, BYTES_PER_ELMT, one, q); break;
    case 5: hipLaunchKernelGGL(nonspec_xfer_three, dim3(1), dim3(DMA_THREADS), lds, s, d_in, d_out, buffer_size, one, q); break;
    case 6: hipLaunchKernelGGL(nonspec_xfer_two, dim3(1), dim3(DMA_THREADS), lds, s, d_in, d_out, buffer_size, one, q); break;
    case 7: hipLaunchKernelGGL(nonspec_xfer_one, dim3(1), dim3(DMA_THREADS), lds, s, d_in, d_out, buffer_size, BYTES_PER_ELMT, one, q); break;
    default: return -1;
  }
  return hipGetLastError() == hipSuccess ? 0 : -2;
}
''',
    "strided": r'''
extern "C" int refk_strided_@SET@(int which, float* d_in, float* d_out, int* /*unused*/, int single, int qualified, void* stream)
{
  // the strides of the reference's run_experiment: the element rounded up to the alignment, both sides
  const int element = BYTES_PER_ELMT / 4, per = ALIGNMENT / 4;
  const int stride_floats = element + ((element % per) ? per - element % per : 0);
  const int stride = stride_floats * 4;
  const int buffer_size = NUM_ELMTS * stride_floats + ALIGN_OFFSET;
  const size_t lds = (size_t)buffer_size * 4;
  hipStream_t s = (hipStream_t)stream;
  const bool one = single != 0, q = qualified != 0;
  switch (which) {
    case 0: hipLaunchKernelGGL(special_xfer_four, dim3(1), dim3(@C@ + DMA_THREADS), lds, s, d_in, d_out, stride, stride, @C@, buffer_size, one, q); break;
    case 1: hipLaunchKernelGGL(special_xfer_three, dim3(1), dim3(@C@ + DMA_THREADS), lds, s, d_in, d_out, stride, stride, @C@, NUM_ELMTS, buffer_size, one, q); break;
    case 2: hipLaunchKernelGGL(special_xfer_two, dim3(1), dim3(@C@ + DMA_THREADS), lds, s, d_in, d_out, stride, stride, @C@, DMA_THREADS, NUM_ELMTS, buffer_size, one, q); break;
    case 3: hipLaunchKernelGGL(special_xfer_one, dim3(1), dim3(@C@ + DMA_THREADS), lds, s, d_in, d_out, stride, stride, @C@, DMA_THREADS, BYTES_PER_ELMT, NUM_ELMTS, buffer_size, one, q); break;
    case 4: hipLaunchKernelGGL(nonspec_xfer_four, dim3(1), dim3(DMA_THREADS), lds, s, d_in, d_out, stride, stride, buffer_size, one, q); break;
    case 5: hipLaunchKernelGGL(nonspec_xfer_three, dim3(1), dim3(DMA_THREADS), lds, s, d_in, d_out, stride, stride, NUM_ELMTS, buffer_size, one, q); break;
    case 6: hipLaunchKernelGGL(nonspec_xfer_two, dim3(1), dim3(DMA_THREADS), lds, s, d_in, d_out, stride, stride, NUM_ELMTS, buffer_size, one, q); break;
    case 7: hipLaunchKernelGGL(nonspec_xfer_one, dim3(1), dim3(DMA_THREADS), lds, s, d_in, d_out, stride, stride, BYTES_PER_ELMT, NUM_ELMTS, buffer_size, one, q); break;
    default: return -1;
  }
  return hipGetLastError() == hipSuccess ? 0 : -2;
}
''',
    "indirect": r'''
extern "C" int refk_indirect_@SET@(int which, float* d_in, float* d_out, int* d_offsets, int single, int qualified, void* stream)
{
  const int buffer_size = NUM_ELMTS * BYTES_PER_ELMT / 4 + ALIGN_OFFSET;
  const size_t lds = (size_t)buffer_size * 4;
  hipStream_t s = (hipStream_t)stream;
  const bool one = single != 0, q = qualified != 0;
  switch (which) {
    case 0: hipLaunchKernelGGL(special_xfer_four, dim3(1), dim3(@C@ + DMA_THREADS), lds, s, d_in, d_out, d_offsets, @C@, buffer_size, one, q); break;
    case 1: hipLaunchKernelGGL(special_xfer_three, dim3(1), dim3(@C@ + DMA_THREADS), lds, s, d_in, d_out, d_offsets, @C@, NUM_ELMTS, buffer_size, one, q); break;
    case 2: hipLaunchKernelGGL(special_xfer_two, dim3(1), dim3(@C@ + DMA_THREADS), lds, s, d_in, d_out, d_offsets, @C@, DMA_THREADS, NUM_ELMTS, buffer_size, one, q); break;
    case 3: hipLaunchKernelGGL(special_xfer_one, dim3(1), dim3(@C@ + DMA_THREADS), lds, s, d_in, d_out, d_offsets, @C@, DMA_THREADS, BYTES_PER_ELMT, NUM_ELMTS, buffer_size, one, q); break;
    case 4: hipLaunchKernelGGL(nonspec_xfer_four, dim3(1), dim3(DMA_THREADS), lds, s, d_in, d_out, d_offsets, buffer_size, one, q); break;
    case 5: hipLaunchKernelGGL(nonspec_xfer_three, dim3(1), dim3(DMA_THREADS), lds, s, d_in, d_out, d_offsets, NUM_ELMTS, buffer_size, one, q); break;
    case 6: hipLaunchKernelGGL(nonspec_xfer_two, dim3(1), dim3(DMA_THREADS), lds, s, d_in, d_out, d_offsets, NUM_ELMTS, buffer_size, one, q); break;
    case 7: hipLaunchKernelGGL(nonspec_xfer_one, dim3(1), dim3(DMA_THREADS), lds, s, d_in, d_out, d_offsets, BYTES_PER_ELMT, NUM_ELMTS, buffer_size, one, q); break;
    default: return -1;
  }
  return hipGetLastError() == hipSuccess ? 0 : -2;
}
''',
}
# Instantiations of the halo test kernel dma_ld_test<ALIGNMENT, ALIGN_OFFSET, ELMT_TYPE, RADIUS, CORNERS>, taken from the
# combinations run_all_experiments() of the reference allows (RADIUS * sizeof(ELMT_TYPE) keeps the ALIGNMENT)
HALO_INSTANCES = [
    dict(ALIGNMENT=4, ELMT="float", ELMT_BYTES=4, RADIUS=1, CORNERS=False),
    dict(ALIGNMENT=4, ELMT="float", ELMT_BYTES=4, RADIUS=3, CORNERS=True),
    dict(ALIGNMENT=8, ELMT="float", ELMT_BYTES=4, RADIUS=2, CORNERS=True),
    dict(ALIGNMENT=8, ELMT="float2", ELMT_BYTES=8, RADIUS=1, CORNERS=False),
    dict(ALIGNMENT=16, ELMT="float", ELMT_BYTES=4, RADIUS=4, CORNERS=False),
    dict(ALIGNMENT=16, ELMT="float", ELMT_BYTES=4, RADIUS=4, CORNERS=True),
    dict(ALIGNMENT=16, ELMT="float2", ELMT_BYTES=8, RADIUS=2, CORNERS=True),
    dict(ALIGNMENT=16, ELMT="float4", ELMT_BYTES=16, RADIUS=1, CORNERS=False),
]


def _halo_launcher():
    cases = "".join(
        f"    case {i}: hipLaunchKernelGGL((dma_ld_test<{h['ALIGNMENT']}, 0, {h['ELMT']}, {h['RADIUS']}, {'true' if h['CORNERS'] else 'false'}>), "
        f"dim3(1), dim3(@C@ + dma_threads), (size_t)((dimx + 2 * {h['RADIUS']}) * (dimy + 2 * {h['RADIUS']})) * {h['ELMT_BYTES']}, s, "
        f"({h['ELMT']}*)d_in, ({h['ELMT']}*)d_out, dimx, dimy, pitch, (dimx + 2 * {h['RADIUS']}) * (dimy + 2 * {h['RADIUS']}), @C@, dma_threads); break;\n"
        for i, h in enumerate(HALO_INSTANCES))
    return ('''
extern "C" int refk_halo(int instance, void* d_in, void* d_out, int dimx, int dimy, int pitch, int dma_threads, void* stream)
{
  hipStream_t s = (hipStream_t)stream;
  switch (instance) {
''' + cases + '''    default: return -1;
  }
  return hipGetLastError() == hipSuccess ? 0 : -2;
}
''').replace("@C@", str(COMPUTE_THREADS))


# saxpy example: the parameters of its params_directed.h in multiples of 64 threads
SAXPY = dict(CTA_COUNT=96, COMPUTE_THREADS_PER_CTA=256, NUM_ITERS=16, DMA_THREADS_PER_LD=64, BYTES_PER_DMA_THREAD=32)
SAXPY_KERNELS = ["saxpy_baseline", "saxpy_float4s", "saxpy_shmem", "saxpy_shmem_doublebuffer", "saxpy_float4s_shmem",
                 "saxpy_float4s_shmem_doublebuffer", "saxpy_cudaDMA", "saxpy_cudaDMA_doublebuffer"]


def _compile_saxpy_unit(hipcc, scratch):
    text = open("/root/reference/src/examples/saxpy/saxpy_cudaDMA_kernel.cu").read()
    kernels = [text[m.start():_END_OF_FUNCTION.search(text, m.start()).end()] for m in re.finditer(r"^__global__", text, re.M)]
    defines = "".join(f"#define {k} {v}\n" for k, v in SAXPY.items()) + "#define DMA_SZ (4 * COMPUTE_THREADS_PER_CTA)\n"
    # threads per workgroup as the reference's THREADS_PER_CTA macro has them: the compute threads, plus two DMA
    # groups for saxpy_cudaDMA and four for saxpy_cudaDMA_doublebuffer
    cases = "".join(
        f"    case {i}: hipLaunchKernelGGL({k}, dim3(CTA_COUNT), dim3(COMPUTE_THREADS_PER_CTA + "
        f"{ {'saxpy_cudaDMA': 2, 'saxpy_cudaDMA_doublebuffer': 4}.get(k, 0) } * DMA_THREADS_PER_LD), 0, s, d_y, d_x, a, (clock_t*)d_timers); break;\n"
        for i, k in enumerate(SAXPY_KERNELS))
    launcher = ('''
extern "C" int refk_saxpy(int which, float* d_y, float* d_x, float a, void* d_timers, void* stream)
{
  hipStream_t s = (hipStream_t)stream;
  switch (which) {
''' + cases + '''    default: return -1;
  }
  return hipGetLastError() == hipSuccess ? 0 : -2;
}
''')
    source = ('#include <hip/hip_runtime.h>\n#include <stdio.h>\n#include <stdlib.h>\n#include <time.h>\n#include "cudaDMA.h"\n' + defines +
              "namespace {\n" + "\n".join(kernels) + "\n}\n" + launcher)
    src, obj = os.path.join(scratch, "saxpy.hip"), os.path.join(scratch, "saxpy.o")
    with open(src, "w") as f:
        f.write(source)
    cmd = [hipcc, "-O3", "-std=c++17", "-fPIC", "--offload-arch=gfx950", "-Xclang", "-target-feature", "-Xclang",
           "-packed-fp32-ops", "-Wno-unused-command-line-argument", "-I", os.path.join(ROOT, "include"), "-c", src, "-o", obj]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError("saxpy:\n" + "\n".join(l for l in res.stderr.splitlines() if "error" in l)[:3000])
    return obj


# sgemv example: the seven configurations of sgemv_dma.cu:79-133; the matrix is SGEMV_N x SGEMV_N (the reference's 896
# does not divide by the 1024 vector elements of its own VEC_DOUBLE configuration)
SGEMV_CONFIGS = ["VEC_SINGLE", "VEC_DOUBLE", "VEC_MANUAL", "BOTH_SINGLE", "BOTH_DOUBLE", "BOTH_MANUAL", "MAT_SINGLE"]
SGEMV_N = 1024


def _compile_sgemv_unit(hipcc, scratch, config):
    text = open("/root/reference/src/examples/sgemv/sgemv_dma.cu").read()
    last = "#endif // MAT_SINGLE"
    body = text[text.index("#define num_threads"):text.index(last) + len(last)]
    # thread groups in wavefronts of 64; `blockIdx.x**COMPUTE_THREADS_PER_CTA` (:468, :479) is a typing slip for one `*`
    body = re.sub(r"(#define DMA_THREADS_PER_LD\s+)32", r"\g<1>64", body).replace("blockIdx.x**COMPUTE", "blockIdx.x*COMPUTE")
    launcher = '''
extern "C" int refk_sgemv_@CFG@(int n, int m, float alpha, float* d_A, float* d_x, float* d_y, void* stream)
{
  const int n1 = (m / COMPUTE_THREADS_PER_CTA) * COMPUTE_THREADS_PER_CTA;
  const int blocks = (n + COMPUTE_THREADS_PER_CTA - 1) / COMPUTE_THREADS_PER_CTA;
  hipLaunchKernelGGL(DMA_KERNEL, dim3(blocks), dim3(COMPUTE_THREADS_PER_CTA + DMA_LDS * DMA_THREADS_PER_LD), 0,
                     (hipStream_t)stream, n, m, n1, alpha, d_A, n, d_x, d_y);
  return hipGetLastError() == hipSuccess ? 0 : -2;
}
'''.replace("@CFG@", config)
    source = (f"#define {config} 1\n#define SIZE_N {SGEMV_N}\n#define SIZE_M SIZE_N\n"
              '#include <hip/hip_runtime.h>\n#include <cstdio>\n#include "cudaDMA.h"\nnamespace {\n' + body + "\n}\n" + launcher)
    src, obj = os.path.join(scratch, f"sgemv_{config}.hip"), os.path.join(scratch, f"sgemv_{config}.o")
    with open(src, "w") as f:
        f.write(source)
    cmd = [hipcc, "-O3", "-std=c++17", "-fPIC", "--offload-arch=gfx950", "-Xclang", "-target-feature", "-Xclang",
           "-packed-fp32-ops", "-Wno-unused-command-line-argument", "-I", os.path.join(ROOT, "include"), "-c", src, "-o", obj]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"sgemv {config}:\n" + "\n".join(l for l in res.stderr.splitlines() if "error" in l)[:3000])
    return obj


# stencil example: the directed parameters of params_directed.h:20-24 (tiles of 32 x 4 float2 cells, radius 4, 12 x 16
# bytes per DMA thread), one DMA wavefront of 64 per load in place of one warp
STENCIL_HEADERS = ["warp_specialized_single_buffer", "warp_specialized_double_buffer", "warp_specialized_manual_buffer",
                   "non_warp_specialized_single_buffer", "non_warp_specialized_double_buffer"]
STENCIL = dict(TILE_X=32, TILE_Y=4, RADIUS=4, DMA_THREADS_PER_LD=64)


def _compile_stencil_unit(hipcc, scratch):
    base = "/root/reference/src/examples/stencil"

    def without_includes(path):
        return "\n".join(l for l in open(path).read().splitlines() if not l.strip().startswith("#include"))
    body = without_includes(os.path.join(base, "stencil_math.h")) + "\n"
    for h in STENCIL_HEADERS:
        # non_warp_specialized_double_buffer.h calls member templates of a dependent type without the `template`
        # keyword, which nvcc lets pass and clang does not
        body += re.sub(r"(\w)\.(start_xfer_async|wait_xfer_finish|execute_dma)<", r"\1.template \2<",
                       without_includes(os.path.join(base, h + ".h"))) + "\n"
    t = STENCIL
    ws = f"16, 12 * 16, {t['TILE_X']}, {t['TILE_Y']}, {t['RADIUS']}, {t['DMA_THREADS_PER_LD']}"
    nws = f"16, 12 * 16, {t['TILE_X']}, {t['TILE_Y']}, {t['RADIUS']}"
    compute = t["TILE_X"] * t["TILE_Y"]
    dma_groups = [1, 2, 1, 0, 0]                       # total_warps of cudaDMA_stencil2D.cu:122,135,149,163,176
    cases = "".join(
        f"    case {i}: hipLaunchKernelGGL((stencil_2D_{h}<{ws if d else nws}>), grid, dim3({compute} + {d} * {t['DMA_THREADS_PER_LD']}), 0, s, "
        f"(const float2*)d_src, (float2*)d_dst, offset, row_stride, slice_stride, dimz); break;\n"
        for i, (h, d) in enumerate(zip(STENCIL_HEADERS, dma_groups)))
    launcher = ('''
extern "C" int refk_stencil2d(int which, const void* d_src, void* d_dst, int dimx, int dimy, int dimz, void* stream)
{
  const int row_stride = dimx + 2 * @R@, slice_stride = (dimy + 2 * @R@) * row_stride;
  const int offset = @R@ * slice_stride + @R@ * row_stride + @R@;
  const dim3 grid(dimx / @TX@, dimy / @TY@);
  hipStream_t s = (hipStream_t)stream;
  switch (which) {
''' + cases + '''    default: return -1;
  }
  return hipGetLastError() == hipSuccess ? 0 : -2;
}
''').replace("@R@", str(t["RADIUS"])).replace("@TX@", str(t["TILE_X"])).replace("@TY@", str(t["TILE_Y"]))
    source = '#include <hip/hip_runtime.h>\n#include "cudaDMAv2.h"\nnamespace {\n' + body + "\n}\n" + launcher
    src, obj = os.path.join(scratch, "stencil2d.hip"), os.path.join(scratch, "stencil2d.o")
    with open(src, "w") as f:
        f.write(source)
    cmd = [hipcc, "-O3", "-std=c++17", "-fPIC", "--offload-arch=gfx950", "-Xclang", "-target-feature", "-Xclang",
           "-packed-fp32-ops", "-Wno-unused-command-line-argument", "-I", os.path.join(ROOT, "include"), "-c", src, "-o", obj]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError("stencil2d:\n" + "\n".join(l for l in res.stderr.splitlines() if "error" in l)[:3000])
    return obj


# read-bandwidth probe: the directed parameters of src/perf/sequential/params_directed.h (float, ALIGNMENT 16, elements
# of 4096 bytes, 32 loops), two DMA wavefronts of 64 in place of two warps, one compute wavefront
PERF_KERNELS = ["non_specialized", "single_buffer", "double_buffer", "manual_buffer"]
PERF = dict(ALIGNMENT=16, ELMT_SIZE=4096, DMA_THREADS=128, LOOP_ITERS=32, COMPUTE_THREADS=64)


def _compile_perf_unit(hipcc, scratch):
    text = open("/root/reference/src/perf/sequential/perf_sequential.cu").read()
    start = text.index("template<typename T, int ALIGNMENT, int BYTES_PER_ELMT, int TOTAL_THREADS, int NUM_LOOPS>")
    end = _END_OF_FUNCTION.search(text, text.index("void manual_buffer")).end()
    t = PERF
    args = f"float, {t['ALIGNMENT']}, {t['ELMT_SIZE']}, {t['DMA_THREADS']}, {t['LOOP_ITERS']}"
    # threads per workgroup as performance_test() counts them (perf_sequential.cu:229-241): the DMA groups alone when not
    # specialised, plus one compute group, plus a second set of DMA groups when double-buffered
    launcher = f'''
extern "C" int refk_perf_sequential(int which, const float* d_src, float* d_dst, int ctas, int always_false, void* stream)
{{
  hipStream_t s = (hipStream_t)stream;
  const int dma = {t['DMA_THREADS']}, compute = {t['COMPUTE_THREADS']};
  switch (which) {{
    case 0: hipLaunchKernelGGL((non_specialized<{args}>), dim3(ctas), dim3(dma), 0, s, d_src, d_dst, always_false != 0); break;
    case 1: hipLaunchKernelGGL((single_buffer<{args}>), dim3(ctas), dim3(dma + compute), 0, s, d_src, d_dst, compute, always_false != 0); break;
    case 2: hipLaunchKernelGGL((double_buffer<{args}>), dim3(ctas), dim3(2 * dma + compute), 0, s, d_src, d_dst, compute, always_false != 0); break;
    case 3: hipLaunchKernelGGL((manual_buffer<{args}>), dim3(ctas), dim3(dma + compute), 0, s, d_src, d_dst, compute, always_false != 0); break;
    default: return -1;
  }}
  return hipGetLastError() == hipSuccess ? 0 : -2;
}}
'''
    source = '#include <hip/hip_runtime.h>\n#include "cudaDMA.h"\nnamespace {\n' + text[start:end] + "\n}\n" + launcher
    src, obj = os.path.join(scratch, "perf.hip"), os.path.join(scratch, "perf.o")
    with open(src, "w") as f:
        f.write(source)
    cmd = [hipcc, "-O3", "-std=c++17", "-fPIC", "--offload-arch=gfx950", "-Xclang", "-target-feature", "-Xclang",
           "-packed-fp32-ops", "-Wno-unused-command-line-argument", "-I", os.path.join(ROOT, "include"), "-c", src, "-o", obj]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError("perf_sequential:\n" + "\n".join(l for l in res.stderr.splitlines() if "error" in l)[:3000])
    return obj


def _compile_halo_unit(hipcc, scratch):
    text = open(os.path.join(REFERENCE_TESTS, "test_halo/cudaDMA_test_halo.cu")).read()
    start = text.index("template<typename TYPE>")                    # initialize<> / get_val<> come before the kernel
    end = _END_OF_FUNCTION.search(text, text.index("dma_ld_test")).end()
    source = ('#include <hip/hip_runtime.h>\n#include <stdio.h>\n#include <stdlib.h>\n#include <assert.h>\n#include <math.h>\n'
              '#include "cudaDMA.h"\nnamespace {\n' + text[start:end] + "\n}\n" + _halo_launcher())
    src, obj = os.path.join(scratch, "halo.hip"), os.path.join(scratch, "halo.o")
    with open(src, "w") as f:
        f.write(source)
    cmd = [hipcc, "-O3", "-std=c++17", "-fPIC", "--offload-arch=gfx950", "-Xclang", "-target-feature", "-Xclang",
           "-packed-fp32-ops", "-Wno-unused-command-line-argument", "-Wno-unused-function", "-I", os.path.join(ROOT, "include"),
           "-c", src, "-o", obj]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError("halo:\n" + "\n".join(l for l in res.stderr.splitlines() if "error" in l)[:3000])
    return obj


_END_OF_FUNCTION = re.compile(r"^\}[ \t]*$", re.M)


def reference_kernels(program):
    """The text of every __global__ function of the program, template heads left out."""
    text = open(os.path.join(REFERENCE_TESTS, PROGRAMS[program])).read()
    return [text[m.start():_END_OF_FUNCTION.search(text, m.start()).end()] for m in re.finditer(r"^__global__", text, re.M)]


def _compile_unit(hipcc, scratch, program, set_name, macros):
    # each unit in a namespace of its own would hide the extern "C" launcher; static kernels would not launch: the
    # kernels of different units carry the same names, so every unit becomes a code object of its own (-fgpu-rdc off)
    # and the kernels are given internal linkage through an unnamed namespace around the reference's text
    source = ('#include <hip/hip_runtime.h>\n#include "cudaDMAv2.h"\n' +
              "".join(f"#define {k} {v}\n" for k, v in macros.items()) +
              "namespace {\n" + "\n".join(reference_kernels(program)) + "\n}\n" +
              _LAUNCHERS[program].replace("@SET@", set_name).replace("@C@", str(COMPUTE_THREADS)))
    src = os.path.join(scratch, f"{program}_{set_name}.hip")
    obj = os.path.join(scratch, f"{program}_{set_name}.o")
    with open(src, "w") as f:
        f.write(source)
    cmd = [hipcc, "-O3", "-std=c++17", "-fPIC", "--offload-arch=gfx950", "-Xclang", "-target-feature", "-Xclang",
           "-packed-fp32-ops", "-Wno-unused-command-line-argument", "-I", os.path.join(ROOT, "include"), "-c", src, "-o", obj]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"{program} {set_name}:\n" + "\n".join(l for l in res.stderr.splitlines() if "error" in l)[:3000])
    return obj


def has_unit(program, macros):
    """An indexed transfer puts element i at i * BYTES_PER_ELMT: its element size has to keep the ALIGNMENT."""
    return program != "indirect" or macros["BYTES_PER_ELMT"] % macros["ALIGNMENT"] == 0


def build(jobs=None):
    if not os.path.isdir(REFERENCE_TESTS):
        print(f"{REFERENCE_TESTS} is not present: nothing to build")
        return None
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    os.makedirs(OUT_DIR, exist_ok=True)
    # CUDADMA_REFKERNEL_DRAWS=N adds N seeded draws from the distribution of the reference's random sweep to the five
    # directed sets (about 40 s of one core per program and set); the manifest tells the tests what was built
    sets = dict(PARAMETER_SETS)
    sets.update(drawn_parameter_sets(int(os.environ.get("CUDADMA_REFKERNEL_DRAWS", "0") or 0)))
    units = [(p, s, m) for p in PROGRAMS for s, m in sets.items() if has_unit(p, m)]
    with tempfile.TemporaryDirectory() as scratch:        # the reference's text exists only here, and only for the build
        with concurrent.futures.ThreadPoolExecutor(max_workers=jobs or min(16, os.cpu_count() or 8)) as pool:
            extra = [pool.submit(_compile_halo_unit, hipcc, scratch), pool.submit(_compile_saxpy_unit, hipcc, scratch)]
            extra += [pool.submit(_compile_sgemv_unit, hipcc, scratch, c) for c in SGEMV_CONFIGS]
            extra.append(pool.submit(_compile_stencil_unit, hipcc, scratch))
            extra.append(pool.submit(_compile_perf_unit, hipcc, scratch))
            objs = list(pool.map(lambda u: _compile_unit(hipcc, scratch, *u), units)) + [e.result() for e in extra]
        subprocess.check_call([hipcc, "-shared", "-fPIC", "--offload-arch=gfx950"] + objs + ["-o", OUT])
    import json
    with open(MANIFEST, "w") as f:
        json.dump(sets, f, indent=1)
    print(f"built {OUT}: {len(units)} units ({len(PROGRAMS)} programs, {len(sets)} parameter sets) + the halo "
          f"test kernel in {len(HALO_INSTANCES)} instantiations + the {len(SAXPY_KERNELS)} saxpy kernels + "
          f"the {len(SGEMV_CONFIGS)} sgemv configurations + the {len(STENCIL_HEADERS)} stencil kernels + the {len(PERF_KERNELS)} probe kernels")
    return OUT


if __name__ == "__main__":
    sys.exit(0 if build() or not os.path.isdir(REFERENCE_TESTS) else 1)
