"""The reference's own test kernels on the GPU.  oracle/build_ref_kernels.py compiles the special_xfer_* / nonspec_xfer_*
kernels of the reference's v2 test programs (src/tests/test_{sequential,strided,indirect}/cudaDMA_test_*_v2.cu) from the
reference tree against this repository's cudaDMAv2.h into oracle/_ref/libref_kernels.so (not kept in the repository;
it travels with the built libraries).  Here they run as the reference's run_experiment() runs them: input float(i)
(cudaDMA_test_sequential_v2.cu:416-418), one workgroup, the LDS buffer zeroed by the compute threads, filled by the DMA
threads, copied out; every kernel in its one-phase and two-phase form, with and without the cache qualifiers the kernel
text names.  The output is compared with the oracle's closed form over the whole buffer (the reference compares the
moved elements only, :501-512), bit for bit."""
import ctypes
import os

import numpy as np
import pytest
import torch

from oracle import build_ref_kernels as ref
from tests import oracle_lib as ol
from tests.oracle_lib import ptr

pytestmark = pytest.mark.gpu

_UNITS = [(p, s) for p in ref.PROGRAMS for s, m in ref.PARAMETER_SETS.items() if ref.has_unit(p, m)]


@pytest.fixture(scope="module")
def kernels():
    if not os.path.exists(ref.OUT):
        pytest.skip(f"{ref.OUT} has not been built (python oracle/build_ref_kernels.py, where the reference tree is present)")
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
    m = ref.PARAMETER_SETS[set_name]
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
