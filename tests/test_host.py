"""CPU-side tests of libcudadma_amd.so and libcudadma_amd_harness.so: they load, export what their headers declare,
validates arguments before touching a GPU, and its host replay of the device objects' index
arithmetic agrees with the oracle's closed forms for every compiled case."""
import ctypes
import os
import re
import subprocess

import numpy as np
import pytest

import cudadma_amd as cd
from tests.cases import CaseIO, case_id_str

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.mark.parametrize("header_name, load, path, bound", [
    ("cudadma_amd.h", cd.lib, cd.lib_path, cd._lib.exported_symbols),
    ("cudadma_amd_harness.h", cd.harness_lib, cd.harness_lib_path, cd._lib.harness_exported_symbols)])
def test_library_exports_every_declared_symbol(header_name, load, path, bound):
    header = open(os.path.join(ROOT, "include", header_name)).read()
    declared = set(re.findall(r"^(?:const\s+)?[a-z_][a-z_ ]*\**\s+(cudadma_[a-z0-9_]+)\s*\(", header, flags=re.M))
    assert declared, "no declarations found"
    load()
    # the symbol is looked up in this library's own file: its table of dynamic symbols, not what the loader
    # would also find in a library it depends on
    own = subprocess.run(["nm", "-D", "--defined-only", path()], capture_output=True, text=True, check=True).stdout
    exported = {line.split()[-1] for line in own.splitlines() if line.strip()}
    for name in sorted(declared):
        assert name in exported, f"{name} is declared in {header_name} but not exported by {os.path.basename(path())}"
    assert declared == set(bound())


def test_the_harness_stays_out_of_the_product_library():
    """The several hundred instantiations of the known-answer cases are test equipment: the library a user
    links holds the workloads, probes, examples and the planner and stays an order of magnitude smaller."""
    assert os.path.getsize(cd.lib_path()) < 4 << 20
    assert os.path.getsize(cd.harness_lib_path()) > os.path.getsize(cd.lib_path())


def test_missing_library_fails_loudly(monkeypatch):
    monkeypatch.setattr(cd._lib, "_lib", None)
    monkeypatch.setattr(cd._lib, "lib_path", lambda: "/nonexistent/libcudadma_amd.so")
    with pytest.raises(cd.CudaDMAError, match="no fallback"):
        cd._lib.lib()


def test_case_table_is_sane():
    cases = cd.harness.all_cases()
    assert len(cases) >= 150
    patterns = [c.pattern for c in cases]
    assert patterns == sorted(patterns)
    for p in range(5):
        assert patterns.count(p) >= 10
    for c in cases:
        assert c.alignment in (4, 8, 16)
        assert c.bytes_per_thread % c.alignment == 0 and c.bytes_per_thread > 0
        assert c.dma_threads % 64 == 0 and 64 <= c.dma_threads <= 960
        assert c.bytes_per_elmt % 4 == 0 and c.bytes_per_elmt >= 0
    # every constructor form is compiled: each (pattern, warp_specialized, level) combination exists
    seen = {(c.pattern, c.warp_specialized, c.level) for c in cases}
    for p, levels in ((0, (1, 2, 3)), (1, (1, 2, 3, 4)), (2, (1, 2, 3, 4)), (4, (1, 2, 3))):
        for ws in (0, 1):
            for lv in levels:
                assert (p, ws, lv) in seen, (p, ws, lv)
    assert (cd.PATTERN_HALO, 1, 0) in seen          # the older cudaDMAHalo class
    with pytest.raises(cd.CudaDMAError):
        cd.harness.get_case(len(cases))


def test_run_case_validates_before_launching():
    r = cd.RunArgs(d_in=0, d_out=0, lds_bytes=1024, reps=1)
    L = cd.harness_lib()
    assert L.cudadma_run_case(0, ctypes.byref(r), None) == -1
    assert b"d_in" in cd.lib().cudadma_last_error()
    r = cd.RunArgs(d_in=4096, d_out=8192, lds_bytes=1000, reps=1)
    assert L.cudadma_run_case(0, ctypes.byref(r), None) == -1
    assert b"lds_bytes" in cd.lib().cudadma_last_error()
    r = cd.RunArgs(d_in=4096, d_out=8192, lds_bytes=1024, reps=1, src_offset_bytes=2)
    assert L.cudadma_run_case(0, ctypes.byref(r), None) == -1
    assert L.cudadma_run_case(10 ** 6, ctypes.byref(r), None) == -3
    # run-time values are only taken for parameters the case's level leaves to its constructor
    cases = cd.harness.all_cases()
    full = next(i for i, c in enumerate(cases) if c.pattern == cd.PATTERN_STRIDED and c.level == 4)
    for field in ("rt_bytes_per_elmt", "rt_dma_threads", "rt_num_elmts", "rt_dimx"):
        r = cd.RunArgs(d_in=4096, d_out=8192, lds_bytes=1024, reps=1, **{field: 64})
        assert L.cudadma_run_case(full, ctypes.byref(r), None) == -1, field
        assert b"case" in cd.lib().cudadma_last_error()
    loose = next(i for i, c in enumerate(cases) if c.pattern == cd.PATTERN_STRIDED and c.level == 1)
    for field, value in (("rt_bytes_per_elmt", 6), ("rt_dma_threads", 100), ("rt_dma_threads", 2048), ("rt_num_elmts", -1)):
        r = cd.RunArgs(d_in=4096, d_out=8192, lds_bytes=1024, reps=1, **{field: value})
        assert L.cudadma_run_case(loose, ctypes.byref(r), None) == -1, (field, value)
    assert cd.lib().cudadma_scatter_copy(4096, 4096, 8192, 16, 33, 0, None) == -1
    assert cd.lib().cudadma_probe_memory(3, 4096, 8192, 100, 8, None) == -1           # bytes not a multiple of 16
    assert L.cudadma_probe_memory(99, 4096, 8192, 1024, 8, None) == -3
    assert L.cudadma_fill_permutation(4096, 0, 1, None) == -1
    # workloads: sizes and variants are checked first
    assert L.cudadma_sequential_copy(4096, 8192, 1000, 0, None) == -1
    assert L.cudadma_sequential_copy(4096, 8192, 16384, 99, None) == -3
    assert L.cudadma_strided_transpose(4096, 8192, 100, 0, None) == -1
    assert L.cudadma_gather_copy(4096, 4096, 8192, 16, 33, 0, None) == -1
    assert L.cudadma_halo_stencil(4096, 8192, 33, 32, 8, 0, None) == -1
    assert L.cudadma_plain_copy(4096, 8192, 10, None) == -1


def test_workload_kernels_use_no_scratch_memory():
    """An object that is not inlined into its kernel lives in scratch memory and a spilled register travels through
    the same counter as the tile loads: either one costs a workload most of its speed without breaking any result.
    The build keeps the compiler's per-kernel resource report; every kernel outside the known-answer harness
    (whose 1024-thread launch bound leaves 64 registers and may spill) must show no scratch and no spill."""
    import glob
    reports = [p for p in glob.glob(os.path.join(ROOT, "cudadma_amd", "csrc", "build", "*.resources"))
               if not os.path.basename(p).startswith(("harness", "v1_cases", "selftest"))]
    if not reports:
        pytest.skip("no resource reports: the library was not built with this Makefile")
    kernels = 0
    for path in reports:
        name = None
        for line in open(path):
            m = re.search(r"remark:\s+Function Name: (\S+)", line)
            if m:
                name = m.group(1)
                kernels += 1
            m = re.search(r"remark:\s+(ScratchSize \[bytes/lane\]|VGPRs Spill|SGPRs Spill): (\d+)", line)
            if m:
                assert int(m.group(2)) == 0, f"{os.path.basename(path)}: {name}: {m.group(1)} = {m.group(2)}"
    assert kernels >= 40


def test_variants_are_described():
    for w, least in ((cd.workloads.SEQUENTIAL, 4), (cd.workloads.STRIDED, 2), (cd.workloads.GATHER, 2), (cd.workloads.SCATTER, 4),
                     (cd.workloads.HALO, 2)):
        n = cd.workloads.num_variants(w)
        held = cd.workloads.variants(w)                  # sweep-only variants have an empty name unless the library was built for the sweeps
        assert len(held) >= least and 0 in held
        assert cd.workloads.variant_name(w, n) == ""
    assert cd.workloads.num_variants(99) == 0


def test_diagnose_prints_the_plan(capfd):
    cd.plan.diagnose(cd.PATTERN_SEQUENTIAL, 16, 128, 16384, 128, 0, True, True)
    cd.plan.diagnose(cd.PATTERN_SEQUENTIAL, 16, 64, 16384, 64)
    cd.plan.diagnose(cd.PATTERN_STRIDED, 16, 128, 256, 128, 64, True, True)
    cd.plan.diagnose(cd.PATTERN_GATHER, 16, 32, 128, 128, 32)
    out = capfd.readouterr().out
    assert "steps needed: 1 (1 full + 0 partial)" in out
    assert "steps needed: 4 (4 full + 0 partial)" in out and "DMA_THREADS >= 256" in out
    assert "16 lanes per element, 4 elements per wavefront load" in out
    assert "gather" in out
    with pytest.raises(cd.CudaDMAError):
        cd.plan.diagnose(cd.PATTERN_HALO, 16, 32, 128, 128, 32)


_CASES = cd.harness.all_cases()


@pytest.mark.parametrize("case_id", range(len(_CASES)), ids=[case_id_str(i, c) for i, c in enumerate(_CASES)])
def test_replay_of_every_compiled_case_matches_the_oracle(case_id):
    """Every destination byte is written exactly once and with the byte the closed form names."""
    case = _CASES[case_id]
    for flavour in (0, 1):
        io = CaseIO(case, flavour=flavour, reps=1)
        got, steps, doubles = io.replay_map()
        want = io.expected_map()
        if case.pattern == cd.PATTERN_GATHER:
            assert doubles == 0
        else:
            assert doubles == 0, f"{doubles} bytes written twice"
        assert np.array_equal(got, want)
        assert steps >= (1 if want.size and (want >= 0).any() else 0)


def test_replay_on_random_parameters():
    """The reference fuzz distribution (src/tests/test_strided/param_sweep_v2.py:51-75) on the host replay."""
    rng = np.random.default_rng(99)
    O = __import__("tests.oracle_lib", fromlist=["x"]).load()
    from tests.oracle_lib import ptr
    for _ in range(300):
        a = int(rng.choice([4, 8, 16]))
        bpt = a * int(rng.integers(1, 9))
        e = 4 * max(1, abs(int(np.ceil(rng.normal(256, 256)))))
        n = int(rng.integers(1, 33))
        t = 64 * int(rng.integers(1, 17))
        ss = (e + a - 1) // a * a + a * int(rng.integers(0, 3))
        ds = (e + a - 1) // a * a + a * int(rng.integers(0, 3))
        ids = np.arange(n * ss + 64, dtype=np.int32)
        want = np.full(n * ds + 64, -1, dtype=np.int32)
        O.oracle_strided(ptr(ids), ptr(want), 4 * e, n, 4 * ss, 4 * ds)
        got, steps, doubles = cd.plan.plan_map(cd.PATTERN_STRIDED, alignment=a, bytes_per_thread=bpt,
                                               bytes_per_elmt=e, dma_threads=t, num_elmts=n, src_stride=ss,
                                               dst_stride=ds, map_len=want.size)
        assert doubles == 0 and np.array_equal(got, want), (a, bpt, e, n, t)
        # sequential with the same numbers
        want = np.full(e + 32, -1, dtype=np.int32)
        O.oracle_sequential(ptr(ids), ptr(want), 4 * e)
        got, steps, doubles = cd.plan.plan_map(cd.PATTERN_SEQUENTIAL, alignment=a, bytes_per_thread=bpt,
                                               bytes_per_elmt=e, dma_threads=t, map_len=want.size)
        assert doubles == 0 and np.array_equal(got, want), (a, bpt, e, t)


def test_replay_rejects_a_window_that_is_too_small():
    with pytest.raises(cd.CudaDMAError, match="outside"):
        cd.plan.plan_map(cd.PATTERN_SEQUENTIAL, alignment=16, bytes_per_thread=64, bytes_per_elmt=4096,
                         dma_threads=64, map_len=1024)


_DROP_IN_KERNEL = r"""
#include "%s"
// the shape of the reference's special_xfer_* test kernels: objects built by every thread, roles split after
__global__ void k(const float* in, const int* idx, float* out)
{
  __shared__ float buf[4096];
  CudaDMASequential<true, 16, 64, 1024, 64> a(0, 64, 64);
  CudaDMAStrided<true, 16, 64, 256, 64, 8> b(1, 64, 64, 1024, 272);
  CudaDMAIndirect<true, true, 16, 64, 128, 64, 8> c(2, 64, 64);
  CudaDMAHalo<true, 16, 64, 4, 64, 4, false, 32, 32> h(3, 64, 64, 48);
  cudaDMACustom d(4, 64, 64, 64);
  if (a.owns_this_thread()) {
    a.execute_dma(in, buf);
    b.execute_dma<true>(in, buf);
    c.execute_dma<true, LOAD_CACHE_STREAMING, STORE_WRITE_BACK>(idx, in, buf);
    c.prefetch_index<true>(idx + 8);
    c.execute_dma_prefetched<true, LOAD_CACHE_ALL, STORE_WRITE_BACK>(idx + 8, in, buf);
    h.execute_dma(in + 1024, buf + 512);
    d.wait_for_dma_start(); d.finish_async_dma();
  } else {
    a.start_async_dma(); a.wait_for_dma_finish();
    b.start_async_dma(); b.wait_for_dma_finish();
    c.start_async_dma(); c.wait_for_dma_finish();
    c.start_async_dma(); c.wait_for_dma_finish();
    h.start_async_dma(); h.wait_for_dma_finish();
    d.start_async_dma(); d.wait_for_dma_finish();
    out[threadIdx.x] = buf[threadIdx.x];
  }
}
static_assert(WARP_SIZE == 64, "thread groups are sized in wavefronts");
"""


@pytest.mark.parametrize("header,flags", [("cudaDMAv2.h", []), ("hipDMA.h", ["-DWARP_SIZE=64"]), ("cudaDMA.h", []),
                                          ("cudaDMAv2.h", ["-DDEBUG_CUDADMA"]), ("cudaDMAv2.h", ["-DHIPDMA_LDS_ONLY_FENCE"]),
                                          ("cudaDMAv2.h", ["-DHIPDMA_SPIN_LIMIT=0"])])
def test_headers_compile_standalone_for_gfx950(tmp_path, header, flags):
    """The drop-in boundary is the include line: a kernel that names only the reference's header must build
    (device pass only, no GPU needed), also with the reference's DEBUG_CUDADMA switch."""
    import shutil
    import subprocess
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(hipcc):
        pytest.skip("no hipcc")
    src = tmp_path / "drop_in.hip"
    src.write_text(_DROP_IN_KERNEL % header)
    cmd = [hipcc, "-std=c++17", "-O1", "--offload-arch=gfx950", "--cuda-device-only", "-c", str(src), "-o", str(tmp_path / "k.o"),
           "-I", os.path.join(ROOT, "include"), "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"] + flags
    res = subprocess.run(cmd, capture_output=True, text=True, timeout=300)
    assert res.returncode == 0, res.stderr[-2000:]


# ---- the harness refuses, on the host, a run whose transfer would leave the caller's buffers ----
def _fake_run(case_id, case, io, **over):
    """cudadma_run_case with pointers that are never dereferenced: every refusal tested here happens before
    the first HIP call."""
    import ctypes
    from cudadma_amd._lib import RunArgs
    kw = dict(d_in=0x10000, d_out=0x20000, d_index=0, lds_bytes=io.lds_bytes, src_offset_bytes=io.src_offset,
              dst_offset_bytes=io.dst_offset, src_stride=io.src_stride, dst_stride=io.dst_stride, pitch=io.pitch,
              call_style=cd.CALL_UNQUALIFIED, two_phase=0, reps=io.reps, rep_src_bytes=io.rep_src_bytes,
              rep_index_elmts=io.rep_index_elmts, reverse=0, out_bytes=0, dst_pitch=io.dst_pitch,
              in_bytes=io.input.size, out_capacity=io.reps * io.lds_bytes, index_elmts=0)
    kw.update(over)
    r = RunArgs(**kw)
    return cd.harness_lib().cudadma_run_case(case_id, ctypes.byref(r), None), cd.lib().cudadma_last_error().decode()


@pytest.mark.parametrize("pattern", [cd.PATTERN_SEQUENTIAL, cd.PATTERN_STRIDED, cd.PATTERN_HALO])
def test_run_case_refuses_transfers_that_leave_the_buffers(pattern):
    from tests.cases import CaseIO
    cases = cd.harness.all_cases()
    case_id = next(i for i, c in enumerate(cases) if c.pattern == pattern and c.level >= 2 and c.bytes_per_elmt > 0
                   and (c.num_elmts > 1 or pattern != cd.PATTERN_STRIDED))
    case = cases[case_id]
    io = CaseIO(case, flavour=0, reps=2)
    ERANGE = -3
    rc, msg = _fake_run(case_id, case, io, in_bytes=io.input.size // 2)
    assert rc == ERANGE and "input buffer" in msg, msg
    rc, msg = _fake_run(case_id, case, io, lds_bytes=(io.lds_bytes // 2) // 16 * 16, out_capacity=io.reps * io.lds_bytes)
    assert rc == ERANGE and "LDS window" in msg, msg
    rc, msg = _fake_run(case_id, case, io, out_capacity=io.reps * io.lds_bytes - 16)
    assert rc == ERANGE and "out_capacity" in msg, msg
    if pattern == cd.PATTERN_STRIDED:
        rc, msg = _fake_run(case_id, case, io, src_stride=io.src_stride * 4)
        assert rc == ERANGE and "input buffer" in msg, msg
        rc, msg = _fake_run(case_id, case, io, dst_stride=io.dst_stride * 4)
        assert rc == ERANGE and "LDS window" in msg, msg
    if pattern == cd.PATTERN_HALO:
        rc, msg = _fake_run(case_id, case, io, pitch=io.pitch * 3)
        assert rc == ERANGE and "input buffer" in msg, msg
        rc, msg = _fake_run(case_id, case, io, dst_pitch=(case.dimx + 2 * case.radius) * 3)
        assert rc == ERANGE and "LDS window" in msg, msg
        rc, msg = _fake_run(case_id, case, io, dst_pitch=case.dimx + 2 * case.radius - 1)
        assert rc == -1 and "dst_pitch" in msg, msg


def test_run_case_refuses_a_short_index_list():
    from tests.cases import CaseIO
    cases = cd.harness.all_cases()
    case_id = next(i for i, c in enumerate(cases) if c.pattern == cd.PATTERN_GATHER and c.num_elmts > 2)
    io = CaseIO(cases[case_id], flavour=0, reps=2)
    rc, msg = _fake_run(case_id, cases[case_id], io, d_index=0x30000, index_elmts=cases[case_id].num_elmts)
    assert rc == -3 and "index_elmts" in msg, msg


def test_run_case_keeps_the_index_ahead_style_to_the_indexed_cases():
    from tests.cases import CaseIO
    cases = cd.harness.all_cases()
    case_id = next(i for i, c in enumerate(cases) if c.pattern == cd.PATTERN_STRIDED and c.level >= 2)
    io = CaseIO(cases[case_id], flavour=0, reps=1)
    rc, msg = _fake_run(case_id, cases[case_id], io, call_style=cd.CALL_INDEX_AHEAD)
    assert rc == -1 and "index-ahead" in msg, msg


def test_plan_extents_are_the_footprint_of_the_closed_form():
    """cudadma_plan_extents (the replay the harness checks buffers with) against the footprint the oracle's
    closed form writes, for every compiled case."""
    from tests.cases import CaseIO
    for case in cd.harness.all_cases():
        io = CaseIO(case, flavour=2, reps=1)
        want = io.expected_map()
        touched = np.flatnonzero(want >= 0)
        idx = io.index[:case.num_elmts] if io.index is not None else None
        ext = cd.plan.plan_extents(case.pattern, alignment=case.alignment, bytes_per_thread=case.bytes_per_thread,
                                   bytes_per_elmt=case.bytes_per_elmt, dma_threads=case.dma_threads,
                                   num_elmts=case.num_elmts, src_stride=io.src_stride, dst_stride=io.dst_stride,
                                   radius=case.radius, corners=case.corners,
                                   dimx=(case.dimx if case.pattern == cd.PATTERN_HALO else 0), dimy=case.dimy,
                                   pitch=io.pitch, dst_pitch=io.dst_pitch, index=idx) \
            if not (idx is not None and case.num_elmts == 0) else (0, 0, 0, 0)
        dst_origin = io.dst_offset
        src_origin = io.src_offset
        if case.pattern == cd.PATTERN_HALO:
            dst_origin += (case.radius * io.dst_cells + case.radius) * case.bytes_per_elmt
            src_origin += (case.radius * io.pitch + case.radius) * case.bytes_per_elmt
        if touched.size == 0:
            assert ext[3] == ext[2]
            continue
        assert (dst_origin + ext[2], dst_origin + ext[3]) == (touched[0], touched[-1] + 1), case
        src_bytes = want[touched]
        assert (src_origin + ext[0], src_origin + ext[1]) == (src_bytes.min(), src_bytes.max() + 1), case


def test_the_top_level_holds_only_what_belongs_there():
    """A stray file at the repository root (a shell redirect gone wrong, a result left behind) travels to every GPU run and
    into history: the tracked top-level entries are the ones named here and the records the round driver writes."""
    import subprocess
    if not os.path.isdir(os.path.join(ROOT, ".git")):
        pytest.skip("not a git checkout")
    tracked = subprocess.check_output(["git", "-C", ROOT, "ls-files"], text=True).splitlines()
    top = sorted({path.split("/")[0] for path in tracked})
    expected = {".gitignore", ".gpurunignore", "README.md", "DESIGN.md", "INTEGRATION.md", "SURVEY.md", "BASELINE.md", "BASELINE.json",
                "VERDICT.md", "ADVICE.md", "__graft_entry__.py", "bench.py", "cudadma_amd", "include", "oracle", "profiles", "tests"}
    records = re.compile(r"^(BENCH|GPUTEST|MULTICHIP|SCALE|COPYCHECK|PROGRESS)(_r\d+)?\.(json|jsonl)$")
    strays = [name for name in top if name not in expected and not records.match(name)]
    assert not strays, f"unexpected entries at the repository root: {strays}"


def _bench(*args):
    import sys
    return subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), *args], capture_output=True, text=True, timeout=300)


def test_bench_refuses_more_than_one_gpu():
    """The build is for one GPU: asking for more ends with a message that says so, before anything touches a device."""
    r = _bench("--gpus", "2")
    assert r.returncode != 0 and "one GPU" in r.stderr and r.stdout.strip() == ""


@pytest.mark.skipif(__import__("torch").cuda.is_available(), reason="this is the behaviour without a GPU")
def test_bench_has_no_cpu_path():
    """Without a GPU the benchmark prints no line and fails: the measured path never falls back to host code."""
    r = _bench("--gpus", "1", "--steps", "1", "--warmup", "0")
    assert r.returncode != 0 and "no GPU" in r.stderr and r.stdout.strip() == ""
