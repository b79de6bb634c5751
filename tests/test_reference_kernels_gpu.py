"""The reference's own device kernels on the GPU.  tests/refkernels/build.py compiles them from the reference tree against
this repository's cudaDMAv2.h / cudaDMA.h into tests/refkernels/_build/libref_kernels.so (not kept in the repository; it travels with
the built libraries): the special_xfer_* / nonspec_xfer_* kernels of the v2 test programs
(src/tests/test_{sequential,strided,indirect}/cudaDMA_test_*_v2.cu), the halo test kernel, the saxpy, sgemv and stencil
examples and the read-bandwidth probe.  The test kernels run as the reference's run_experiment() runs them: input float(i)
(cudaDMA_test_sequential_v2.cu:416-418), one workgroup, the LDS buffer zeroed by the compute threads, filled by the DMA
threads, copied out; every kernel in its one-phase and two-phase form, with and without the cache qualifiers the kernel
text names.  The output is compared with the oracle's closed form over the whole buffer (the reference compares the
moved elements only, :501-512), bit for bit.  The examples and the probe run as their own main()s launch them."""
import ctypes
import os

import numpy as np
import pytest
import torch

from tests.refkernels import build as ref
from tests import oracle_lib as ol
from tests.oracle_lib import ptr

pytestmark = pytest.mark.gpu

_SETS = ref.built_parameter_sets()        # the directed sets, plus the seeded draws the library on disk was built with
_UNITS = [(p, s) for p in ref.PROGRAMS for s, m in _SETS.items() if ref.has_unit(p, m)]


@pytest.fixture(scope="module")
def kernels():
    if not os.path.exists(ref.OUT):
        pytest.skip(f"{ref.OUT} has not been built (python tests/refkernels/build.py, where the reference tree is present)")
    return ctypes.CDLL(ref.OUT)


def _expected(program, m, floats_in, index):
    """The LDS buffer after the transfer, as floats: zero where nothing lands."""
    e, off, n = m["BYTES_PER_ELMT"], m["ALIGN_OFFSET"], m["NUM_ELMTS"]
    O = ol.load()
    if program == "sequential":
        out = np.zeros(e // 4 + off, dtype=np.float32)
        O.oracle_sequential(ptr(floats_in[off:]), ptr(out[off:]), e)
    elif program == "strided":
        per = m["ALIGNMENT"] // 4
        stride = (e // 4 + per - 1) // per * per
        out = np.zeros(n * stride + off, dtype=np.float32)
        O.oracle_strided(ptr(floats_in[off:]), ptr(out[off:]), e, n, stride * 4, stride * 4)
    else:
        out = np.zeros(n * e // 4 + off, dtype=np.float32)
        O.oracle_gather(ptr(index), ptr(floats_in[off:]), ptr(out[off:]), e, n, 0)
    return out


@pytest.mark.parametrize("program,set_name", _UNITS, ids=[f"{p}-{s}" for p, s in _UNITS])
def test_reference_test_kernels_match_the_oracle(kernels, device, program, set_name):
    m = _SETS[set_name]
    e, off, n = m["BYTES_PER_ELMT"], m["ALIGN_OFFSET"], m["NUM_ELMTS"]
    rng = np.random.default_rng(e * 131 + n)
    index = None
    if program == "sequential":
        floats = e // 4 + off
    elif program == "strided":
        per = m["ALIGNMENT"] // 4
        floats = n * ((e // 4 + per - 1) // per * per) + off
    else:
        index = rng.integers(0, 3 * n, size=n, dtype=np.int32)          # with repeats now and then, in no order
        index[-1] = index[0]
        floats = (int(index.max()) + 1) * e // 4 + off
    host_in = np.arange(floats, dtype=np.float32)                         # input float(i), as the reference fills it
    want = _expected(program, m, host_in, index)
    fn = getattr(kernels, f"refk_{program}_{set_name}")
    fn.restype = ctypes.c_int
    fn.argtypes = [ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_void_p]
    d_in = torch.from_numpy(host_in).to(device)
    d_idx = torch.from_numpy(index).to(device) if index is not None else None
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    ran = 0
    for which in range(8):
        for single in (1, 0):
            for qualified in (0, 1):
                d_out = torch.full((want.size,), float("nan"), dtype=torch.float32, device=device)
                print(f"{program} {set_name} kernel {which} single {single} qualified {qualified}", flush=True)
                rc = fn(which, ctypes.c_void_p(d_in.data_ptr()), ctypes.c_void_p(d_out.data_ptr()),
                        ctypes.c_void_p(d_idx.data_ptr()) if d_idx is not None else None, single, qualified, stream)
                if rc == -1:
                    continue                                              # the program has no kernel of this number
                assert rc == 0
                torch.cuda.synchronize()
                got = d_out.cpu().numpy()
                assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), \
                    f"kernel {which} single {single} qualified {qualified}: first difference at float {int(np.argmax(got.view(np.uint32) != want.view(np.uint32)))}"
                ran += 1
    assert ran == (24 if program == "sequential" else 32)


@pytest.mark.parametrize("instance", range(len(ref.HALO_INSTANCES)),
                         ids=[f"A{h['ALIGNMENT']}-{h['ELMT']}-R{h['RADIUS']}-{'corners' if h['CORNERS'] else 'star'}" for h in ref.HALO_INSTANCES])
def test_reference_halo_test_kernel_matches_the_oracle(kernels, device, instance):
    """dma_ld_test of src/tests/test_halo/cudaDMA_test_halo.cu:180-232 (first-generation cudaDMAHalo) as its
    run_experiment() launches it (:261-268): pitch = 4 * dimx, one compute wavefront, 1-3 DMA wavefronts; input
    rand() % 10 (:245); checked with the reference's own checker restated (oracle_halo_check, :91-164) and, over the
    whole buffer, against the oracle's closed form."""
    h = ref.HALO_INSTANCES[instance]
    es, r, corners = h["ELMT_BYTES"], h["RADIUS"], int(h["CORNERS"])
    unit = max(1, h["ALIGNMENT"] // es)                      # dimx keeps the ALIGNMENT, as in run_subset_experiments (:290)
    fn = kernels.refk_halo
    fn.restype = ctypes.c_int
    fn.argtypes = [ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_void_p]
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    rng = np.random.default_rng(500 + instance)
    O = ol.load()
    ran = 0
    for dimx in (2 * unit, 8, 16, 24, 32):
        if dimx % unit:
            continue
        for dimy in (8, 9, 13, 32):
            for dma_threads in (64, 128, 192):
                pitch = 4 * dimx
                opitch = dimx + 2 * r
                n_in, n_out = pitch * (dimy + 2 * r), opitch * (dimy + 2 * r)
                if n_out * es > 49152:
                    continue
                host_in = rng.integers(0, 10, size=n_in * es // 4).astype(np.float32)
                want = np.zeros(n_out * es // 4, dtype=np.float32)
                src_origin = host_in.view(np.uint8)[(r * pitch + r) * es:]
                dst_origin = want.view(np.uint8)[(r * opitch + r) * es:]
                O.oracle_halo(ptr(src_origin), ptr(dst_origin), es, r, corners, dimx, dimy, pitch)
                d_in = torch.from_numpy(host_in).to(device)
                d_out = torch.full((want.size,), float("nan"), dtype=torch.float32, device=device)
                print(f"halo instance {instance} dimx {dimx} dimy {dimy} dma threads {dma_threads}", flush=True)
                assert fn(instance, ctypes.c_void_p(d_in.data_ptr()), ctypes.c_void_p(d_out.data_ptr()), dimx, dimy, pitch,
                          dma_threads, stream) == 0
                torch.cuda.synchronize()
                got = d_out.cpu().numpy()
                assert O.oracle_halo_check(ptr(host_in), ptr(got), es, r, corners, dimx, dimy, pitch) == 1
                assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
                ran += 1
    assert ran >= 30

@pytest.mark.parametrize("which", range(len(ref.SAXPY_KERNELS)), ids=ref.SAXPY_KERNELS)
def test_reference_saxpy_kernels_match_the_oracle(kernels, device, which):
    """The eight kernels of src/examples/saxpy/saxpy_cudaDMA_kernel.cu:54-420 (saxpy_cudaDMA and
    saxpy_cudaDMA_doublebuffer stage x and y through cudaDMASequential objects) launched as saxpy_cudaDMA.cu:138 does,
    on CTA_COUNT x NUM_ITERS x COMPUTE_THREADS_PER_CTA elements.  The reference accepts |host - device| <= 1e-6
    (saxpy_cudaDMA.cu:167-178); here the result is compared bit for bit with one fused multiply-add per element,
    which is what the device code does after contraction."""
    p = ref.SAXPY
    n = p["CTA_COUNT"] * p["NUM_ITERS"] * p["COMPUTE_THREADS_PER_CTA"]
    x = ol.uniform(n, 11)
    y0 = ol.uniform(n, 12)
    a = np.float32(0.37)
    want = y0.copy()
    ol.load().oracle_saxpy(ctypes.c_float(float(a)), ptr(x), ptr(want), n)
    fn = kernels.refk_saxpy
    fn.restype = ctypes.c_int
    fn.argtypes = [ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_float, ctypes.c_void_p, ctypes.c_void_p]
    d_x = torch.from_numpy(x).to(device)
    d_y = torch.from_numpy(y0).to(device)
    d_timers = torch.zeros(1024, dtype=torch.int64, device=device)
    print(f"saxpy kernel {ref.SAXPY_KERNELS[which]}", flush=True)
    assert fn(which, ctypes.c_void_p(d_y.data_ptr()), ctypes.c_void_p(d_x.data_ptr()), ctypes.c_float(float(a)),
              ctypes.c_void_p(d_timers.data_ptr()), ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)) == 0
    torch.cuda.synchronize()
    got = d_y.cpu().numpy()
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), float(np.abs(got - want).max())

@pytest.mark.parametrize("config", ref.SGEMV_CONFIGS)
def test_reference_sgemv_kernels_match_their_own_expectation(kernels, device, config):
    """The seven DMA kernels of src/examples/sgemv/sgemv_dma.cu:141-620 launched as its main() launches them (:845-856)
    on the reference's own data (initialize_host, :735-749: A[j][i] = (i * j) % 11, x[i] = i % 11, alpha = 2), whose
    products and sums are whole numbers below 2^24: the result is exact in any order of summation, and verify()
    (:752-771) is restated with integers.  The matrix is 1024 x 1024 instead of 896 x 896 so that every
    configuration's vector length divides it; the buffers carry a margin of zeros."""
    n = m = ref.SGEMV_N
    i = np.arange(n, dtype=np.int64)
    j = np.arange(m, dtype=np.int64)
    a_int = (j[:, None] * i[None, :]) % 11                              # matA[j * n + i]
    x_int = j % 11
    alpha = 2.0
    want = (alpha * (a_int * x_int[:, None]).sum(axis=0)).astype(np.float32)
    assert want.max() < 2 ** 24
    margin = 64
    d_a = torch.zeros((m + margin) * n, dtype=torch.float32, device=device)
    d_a[:m * n] = torch.from_numpy(a_int.astype(np.float32).reshape(-1)).to(device)
    d_x = torch.zeros(m + 2048, dtype=torch.float32, device=device)
    d_x[:m] = torch.from_numpy(x_int.astype(np.float32)).to(device)
    d_y = torch.full((n + 256,), float("nan"), dtype=torch.float32, device=device)
    fn = getattr(kernels, f"refk_sgemv_{config}")
    fn.restype = ctypes.c_int
    fn.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_float, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p]
    print(f"sgemv {config}", flush=True)
    assert fn(n, m, ctypes.c_float(alpha), ctypes.c_void_p(d_a.data_ptr()), ctypes.c_void_p(d_x.data_ptr()),
              ctypes.c_void_p(d_y.data_ptr()), ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)) == 0
    torch.cuda.synchronize()
    got = d_y.cpu().numpy()
    assert np.array_equal(got[:n], want), int(np.argmax(got[:n] != want))
    assert np.isnan(got[n:]).all()                                     # nothing written past the vector


@pytest.mark.parametrize("which", range(len(ref.STENCIL_HEADERS)), ids=ref.STENCIL_HEADERS)
@pytest.mark.parametrize("dims", [(32, 4, 2), (96, 20, 6), (960, 160, 8)], ids=lambda d: "x".join(map(str, d)))
def test_reference_stencil_kernels_match_the_oracle(kernels, device, which, dims):
    """The five kernels of src/examples/stencil/*_buffer.h launched as cudaDMA_stencil2D.cu:118-185 launches them
    (grid DIM_X/TILE_X x DIM_Y/TILE_Y, TILE_X * TILE_Y compute threads plus one or two DMA groups, the offset and
    strides of :94-97) on float2 cells in a (dimz + 2R, dimy + 2R, dimx + 2R) volume.  The reference checks nothing
    here; the oracle's cross (arms of R - 1 cells, as stencil_math.h sums them) is compared bit for bit over the whole
    destination, the cells no kernel may touch included."""
    O = ol.load()
    dimx, dimy, dimz = dims
    r = ref.STENCIL["RADIUS"]
    shape = (dimz + 2 * r, dimy + 2 * r, dimx + 2 * r, 2)
    cells = int(np.prod(shape))
    src = ol.uniform(cells, 31)
    want = np.full(cells, -7.0, dtype=np.float32)
    O.oracle_stencil2d(ptr(src), ptr(want), dimx, dimy, dimz, r, r - 1)
    margin = 4 * shape[1] * shape[2] * 2                                # four planes beyond either buffer
    d_src = torch.zeros(cells + margin, dtype=torch.float32, device=device)
    d_src[:cells] = torch.from_numpy(src).to(device)
    d_dst = torch.full((cells + margin,), -7.0, dtype=torch.float32, device=device)
    fn = kernels.refk_stencil2d
    fn.restype = ctypes.c_int
    fn.argtypes = [ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_void_p]
    print(f"stencil2d {ref.STENCIL_HEADERS[which]} {dims}", flush=True)
    assert fn(which, ctypes.c_void_p(d_src.data_ptr()), ctypes.c_void_p(d_dst.data_ptr()), dimx, dimy, dimz,
              ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)) == 0
    torch.cuda.synchronize()
    got = d_dst.cpu().numpy()
    assert np.array_equal(got[:cells].view(np.uint32), want.view(np.uint32)), int(np.argmax(got[:cells] != want))
    assert (got[cells:] == -7.0).all()


@pytest.mark.parametrize("which", range(len(ref.PERF_KERNELS)), ids=ref.PERF_KERNELS)
def test_reference_probe_kernels_move_what_they_should(kernels, device, which):
    """The four kernel shapes of src/perf/sequential/perf_sequential.cu:52-224 (not specialised; single, double and manual
    buffering on cudaDMASequential) launched as its performance_test() launches them (:229-241, :311-345).  The probe
    only times them: its `always_false` argument keeps the buffers from being read.  Here they also run with the
    argument true, which makes every compute thread add its word of each of the 32 buffers to the output
    (out[first + t] += buffer[t], :67-70), a sum that pins which bytes reached the LDS buffer in which loop."""
    t = ref.PERF
    ctas, loops, per = 96, t["LOOP_ITERS"], t["ELMT_SIZE"] // 4
    readers = t["DMA_THREADS"] if which == 0 else t["COMPUTE_THREADS"]       # threads that reach the addition
    rng = np.random.default_rng(12 + which)
    src = rng.integers(0, 10, size=ctas * loops * per).astype(np.float32)
    want = np.full(src.size, -3.0, dtype=np.float32)
    for i in range(loops):                                                    # float32 additions in the kernel's order
        want.reshape(ctas, loops * per)[:, :readers] += src.reshape(ctas, loops, per)[:, i, :readers]
    d_src = torch.from_numpy(src).to(device)
    fn = kernels.refk_perf_sequential
    fn.restype = ctypes.c_int
    fn.argtypes = [ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_void_p]
    for always_false in (0, 1):
        d_dst = torch.full((src.size,), -3.0, dtype=torch.float32, device=device)
        print(f"perf_sequential {ref.PERF_KERNELS[which]} always_false={always_false}", flush=True)
        assert fn(which, ctypes.c_void_p(d_src.data_ptr()), ctypes.c_void_p(d_dst.data_ptr()), ctas, always_false,
                  ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)) == 0
        torch.cuda.synchronize()
        got = d_dst.cpu().numpy()
        if always_false:
            assert np.array_equal(got, want), int(np.argmax(got != want))
        else:
            assert (got == -3.0).all()                                        # as timed: nothing is written
