"""GPU parity of the DMA objects: every compiled case of the known-answer harness, called
through the C ABI, against the oracle's closed form, bit for bit and over the whole LDS
buffer (so stray writes outside the footprint fail too).  The variant matrix is the
reference's: warp-specialised or not x one-phase or two-phase x unqualified / global /
fully qualified calls x every template level (cudaDMA_test_strided_v2.cu:693-812), plus
the direct-to-LDS path that only exists here."""
import os

import numpy as np
import pytest
import torch

import cudadma_amd as cd
from tests.cases import CaseIO, case_id_str

pytestmark = pytest.mark.gpu

_CASES = cd.harness.all_cases()


def _styles(case):
    styles = [cd.CALL_UNQUALIFIED, cd.CALL_GLOBAL, cd.CALL_QUALIFIED]
    # the qualifier matrix of include/cudaDMAv2.h:50-63: every load qualifier from a source known to be global
    # and from a generic one, every store qualifier of the reference
    styles += list(cd.CALL_MATRIX_GLOBAL) + list(cd.CALL_MATRIX_GENERIC)
    if case.pattern in (cd.PATTERN_SEQUENTIAL, cd.PATTERN_STRIDED, cd.PATTERN_GATHER) and case.alignment in (4, 16):
        styles += [cd.CALL_LDS_DIRECT, cd.CALL_LDS_DIRECT_SC1, cd.CALL_LDS_DIRECT_NT]
    if case.pattern in (cd.PATTERN_GATHER, cd.PATTERN_SCATTER):
        styles.append(cd.CALL_INDEX_AHEAD)                    # prefetch_index + the _prefetched calls
    if case.pattern == cd.PATTERN_STRIDED and case.bytes_per_elmt % case.alignment == 0:
        styles.append(cd.CALL_LDS_SWIZZLE)                    # permuted chunks, through registers
        if case.alignment in (4, 16):
            styles.append(cd.CALL_LDS_DIRECT_SWIZZLE)         # permuted chunks, global_load_lds where the shape allows
    return styles


@pytest.mark.parametrize("case_id", range(len(_CASES)), ids=[case_id_str(i, c) for i, c in enumerate(_CASES)])
def test_case_matches_oracle(case_id, device):
    case = _CASES[case_id]
    flavour = 0
    for data in ("ramp", "uniform"):
        for style in _styles(case):
            for two_phase in (False, True):
                io = CaseIO(case, flavour=flavour, reps=3, data=data)
                flavour += 1
                want = io.expected(swizzle=style in (cd.CALL_LDS_SWIZZLE, cd.CALL_LDS_DIRECT_SWIZZLE))
                d_in = torch.from_numpy(io.input).to(device)
                d_idx = torch.from_numpy(io.index).to(device) if io.index is not None else None
                d_out = torch.full((io.reps * io.lds_bytes,), 0xEE, dtype=torch.uint8, device=device)
                print(f"case {case_id} style {style} two_phase {two_phase} data {data} {case}", flush=True)
                cd.harness.run_case(case_id, d_in, d_out, lds_bytes=io.lds_bytes, d_index=d_idx,
                                    src_offset_bytes=io.src_offset, dst_offset_bytes=io.dst_offset,
                                    src_stride=io.src_stride, dst_stride=io.dst_stride, pitch=io.pitch,
                                    call_style=style, two_phase=two_phase, reps=io.reps,
                                    rep_src_bytes=io.rep_src_bytes, rep_index_elmts=io.rep_index_elmts,
                                    dst_pitch=io.dst_pitch)
                torch.cuda.synchronize()
                got = d_out.cpu().numpy().reshape(io.reps, io.lds_bytes)
                if not np.array_equal(got, want):
                    bad = np.argwhere(got != want)
                    raise AssertionError(
                        f"style {style} two_phase {two_phase} data {data}: {len(bad)} wrong bytes, first at rep "
                        f"{bad[0][0]} byte {bad[0][1]} (got {got[tuple(bad[0])]}, want {want[tuple(bad[0])]})")


@pytest.mark.parametrize("case_id", range(len(_CASES)), ids=[case_id_str(i, c) for i, c in enumerate(_CASES)])
def test_case_reverse_direction_matches_oracle(case_id, device):
    """The same objects moving LDS -> global through the generic-pointer calls: the reference's
    ld/st wrappers are direction-agnostic (include/cudaDMAv2.h:107-114,553-558), its tests never try it."""
    case = _CASES[case_id]
    # the unqualified calls, and two of the four qualified calls that take a generic source (the pair rotates with
    # the case number): there the store qualifier acts on global memory
    generic = cd.CALL_MATRIX_GENERIC
    plan = ((0, False, cd.CALL_UNQUALIFIED), (1, True, cd.CALL_UNQUALIFIED),
            (2, bool(case_id & 1), generic[case_id % 4]), (3, not (case_id & 1), generic[(case_id + 2) % 4]))
    if case.pattern in (cd.PATTERN_GATHER, cd.PATTERN_SCATTER):
        plan += ((4, True, cd.CALL_INDEX_AHEAD), (5, False, cd.CALL_INDEX_AHEAD))      # index words requested ahead
    for flavour, two_phase, style in plan:
        io = CaseIO(case, flavour=flavour, reps=2, data="uniform", reverse=True)
        if io.lds_bytes > 64 * 1024 - 256:
            pytest.skip("source image does not fit the harness LDS window")
        want = io.expected()
        d_in = torch.from_numpy(io.input).to(device)
        d_idx = torch.from_numpy(io.index).to(device) if io.index is not None else None
        d_out = torch.zeros(io.reps * io.out_bytes, dtype=torch.uint8, device=device)
        print(f"reverse case {case_id} style {style} two_phase {two_phase} {case}", flush=True)
        cd.harness.run_case(case_id, d_in, d_out, lds_bytes=io.lds_bytes, d_index=d_idx,
                            src_offset_bytes=io.src_offset, dst_offset_bytes=io.dst_offset,
                            src_stride=io.src_stride, dst_stride=io.dst_stride, pitch=io.pitch,
                            call_style=style, two_phase=two_phase, reps=io.reps,
                            rep_src_bytes=io.rep_src_bytes, rep_index_elmts=io.rep_index_elmts,
                            reverse=True, out_bytes=io.out_bytes, dst_pitch=io.dst_pitch)
        torch.cuda.synchronize()
        got = d_out.cpu().numpy().reshape(io.reps, io.out_bytes)
        if not np.array_equal(got, want):
            bad = np.argwhere(got != want)
            raise AssertionError(f"style {style} two_phase {two_phase}: {len(bad)} wrong bytes, first at rep {bad[0][0]} byte {bad[0][1]}")


def _runtime_draw(case, rng):
    """Other values for the parameters the case's level leaves to run time, drawn as the reference's
    sweep draws them (src/tests/test_strided/param_sweep_v2.py:51-75: element size |ceil(N(256,256))|
    floats, 1-32 elements, 1-16 DMA warps), kept inside the harness's LDS window.  Returns the keyword
    arguments for run_case and the case description as it then runs."""
    import types
    c = types.SimpleNamespace(**{f: getattr(case, f) for f, _ in case._fields_})
    kw = {}
    halo = case.pattern == cd.PATTERN_HALO
    max_threads = 1024 - (64 if case.warp_specialized else 0)
    if (case.level <= 1) if halo else (case.level <= 2):
        c.dma_threads = kw["dma_threads"] = 64 * int(rng.integers(1, min(16, max_threads // 64) + 1))
    if halo:
        if case.level <= 2:
            unit = max(1, case.alignment // case.bytes_per_elmt)
            c.dimx = kw["dimx"] = unit * int(rng.integers(1, max(2, 48 // unit)))
            c.dimy = kw["dimy"] = int(rng.integers(1, 41))
        return kw, c
    if case.level == 1:
        c.bytes_per_elmt = kw["bytes_per_elmt"] = 4 * max(1, abs(int(np.ceil(rng.normal(256, 256)))))
    if case.pattern != cd.PATTERN_SEQUENTIAL and case.level <= 3:
        c.num_elmts = kw["num_elmts"] = int(rng.integers(1, 33))
        row = (c.bytes_per_elmt + 15) // 16 * 16 + 48               # an LDS row with the widest padding CaseIO adds
        while (c.num_elmts + 3) * row > 60000:                      # the harness's LDS window
            c.num_elmts = kw["num_elmts"] = max(1, c.num_elmts // 2)
            if c.num_elmts == 1 and 4 * row > 60000:
                c.bytes_per_elmt = kw["bytes_per_elmt"] = 4 * int(rng.integers(1, 2048))
                row = (c.bytes_per_elmt + 15) // 16 * 16 + 48
    elif case.pattern == cd.PATTERN_SEQUENTIAL and case.level == 1 and c.bytes_per_elmt > 60000:
        c.bytes_per_elmt = kw["bytes_per_elmt"] = 60000
    return kw, c


_RUNTIME_CASES = [i for i, c in enumerate(_CASES)
                  if (c.level <= 2 if c.pattern == cd.PATTERN_HALO else c.level <= (2 if c.pattern == cd.PATTERN_SEQUENTIAL else 3))]


@pytest.mark.parametrize("case_id", _RUNTIME_CASES, ids=[case_id_str(i, _CASES[i]) for i in _RUNTIME_CASES])
def test_runtime_parameters_swept(case_id, device):
    """One compiled case, other run-time sizes: what the reference's endless param_sweep_v2.py loop does by
    recompiling.  Every draw is first replayed on the host (the device objects' own index arithmetic,
    which refuses a step outside the buffers) and only then launched."""
    case = _CASES[case_id]
    rng = np.random.default_rng(7000 + case_id)
    for draw in range(int(os.environ.get("CUDADMA_SWEEP_DRAWS", "6"))):     # more draws for an occasional longer hunt
        kw, c = _runtime_draw(case, rng)
        style = _styles(c)[draw % len(_styles(c))]
        two_phase = bool(draw & 1)
        io = CaseIO(c, flavour=draw, reps=2, data="uniform")
        if io.lds_bytes > 64 * 1024 - 256:
            continue
        got_map, _, doubles = io.replay_map()
        assert doubles == 0 and np.array_equal(got_map, io.expected_map()), f"host replay disagrees for {kw}"
        want = io.expected(swizzle=style in (cd.CALL_LDS_SWIZZLE, cd.CALL_LDS_DIRECT_SWIZZLE))
        d_in = torch.from_numpy(io.input).to(device)
        d_idx = torch.from_numpy(io.index).to(device) if io.index is not None else None
        d_out = torch.full((io.reps * io.lds_bytes,), 0xEE, dtype=torch.uint8, device=device)
        print(f"case {case_id} draw {draw} {kw} style {style} two_phase {two_phase}", flush=True)
        cd.harness.run_case(case_id, d_in, d_out, lds_bytes=io.lds_bytes, d_index=d_idx,
                            src_offset_bytes=io.src_offset, dst_offset_bytes=io.dst_offset,
                            src_stride=io.src_stride, dst_stride=io.dst_stride, pitch=io.pitch,
                            call_style=style, two_phase=two_phase, reps=io.reps,
                            rep_src_bytes=io.rep_src_bytes, rep_index_elmts=io.rep_index_elmts,
                            dst_pitch=io.dst_pitch, **kw)
        torch.cuda.synchronize()
        got = d_out.cpu().numpy().reshape(io.reps, io.lds_bytes)
        if not np.array_equal(got, want):
            bad = np.argwhere(got != want)
            raise AssertionError(f"draw {draw} {kw} style {style} two_phase {two_phase}: {len(bad)} wrong bytes, "
                                 f"first at rep {bad[0][0]} byte {bad[0][1]}")


def test_runtime_parameters_of_a_compile_time_case_are_refused(device):
    full = next(i for i, c in enumerate(_CASES) if c.pattern == cd.PATTERN_STRIDED and c.level == 4)
    io = CaseIO(_CASES[full], reps=1)
    d_in = torch.from_numpy(io.input).to(device)
    d_out = torch.zeros(io.lds_bytes, dtype=torch.uint8, device=device)
    for kw in ({"bytes_per_elmt": 64}, {"dma_threads": 64}, {"num_elmts": 3}, {"dimx": 8}):
        with pytest.raises(cd.CudaDMAError):
            cd.harness.run_case(full, d_in, d_out, lds_bytes=io.lds_bytes, src_stride=io.src_stride,
                                dst_stride=io.dst_stride, **kw)


def test_halo_case_passes_the_reference_checker(device):
    """check_halo of the reference on the GPU output of the cudaDMAHalo (older interface) cases."""
    from tests import oracle_lib as ol
    from tests.oracle_lib import ptr
    O = ol.load()
    ran = 0
    for case_id, case in enumerate(_CASES):
        if case.pattern != cd.PATTERN_HALO or case.level != 0:
            continue
        io = CaseIO(case, flavour=1, reps=1, data="uniform")
        d_in = torch.from_numpy(io.input).to(device)
        d_out = torch.zeros(io.lds_bytes, dtype=torch.uint8, device=device)
        cd.harness.run_case(case_id, d_in, d_out, lds_bytes=io.lds_bytes, src_offset_bytes=io.src_offset,
                            dst_offset_bytes=io.dst_offset, pitch=io.pitch, reps=1)
        torch.cuda.synchronize()
        got = d_out.cpu().numpy()
        assert O.oracle_halo_check(ptr(io.input, io.src_offset), ptr(got, io.dst_offset), case.bytes_per_elmt,
                                   case.radius, case.corners, case.dimx, case.dimy, io.pitch) == 1
        ran += 1
    assert ran >= 4


def test_unmatched_waits_end_and_are_reported(device):
    """Unbalanced start_async_dma / finish_async_dma counts must not hang the GPU: with the poll limit
    forced down from the host side both waits give up, the kernel finishes, and the failure record says
    that two wavefronts gave up (the reference would hang; its DEBUG_CUDADMA build asserts,
    include/cudaDMAv2.h:1564-1576)."""
    import ctypes
    assert cd.device_status(clear=True) == (0, 0)
    flags = torch.zeros(2, dtype=torch.int32, device=device)
    cd._lib.check(cd.harness_lib().cudadma_selftest_bounded_wait(ctypes.c_void_p(flags.data_ptr()), None))
    torch.cuda.synchronize()
    assert flags.tolist() == [1, 1]
    bits, waves = cd.device_status(clear=False)
    assert bits == cd.STATUS_WAIT_GAVE_UP and waves == 2
    assert cd.device_status(clear=True) == (cd.STATUS_WAIT_GAVE_UP, 2)     # the record stays until it is cleared
    assert cd.device_status(clear=True) == (0, 0)


def test_every_translation_unit_with_dma_objects_reports(device):
    assert cd.lib().cudadma_device_status_sources() >= 20


@pytest.mark.parametrize("entry", ["cudadma_selftest_global_handoff", "cudadma_selftest_global_handoff_lds_only"])
def test_global_memory_crosses_the_handshake(device, entry):
    """Global memory written before a signal is seen after the matching wait, in both directions: the compute
    wavefront produces the source in global memory, the DMA wavefronts move it global -> global, the compute
    wavefront reads the destination (bar.sync / bar.arrive order all memory, include/cudaDMAv2.h:65-75).
    The default build (fences over all address spaces) is the contract and must deliver every word.  The build with
    fences over LDS only promises nothing about global memory (its fences leave the compiler free to move the global
    accesses across the hand-off, although on this chip both builds wait the same way): for it the test only asks that
    the kernel ends with an empty failure record."""
    import ctypes
    scratch = torch.zeros(4096, dtype=torch.int32, device=device)
    wrong = torch.zeros(1, dtype=torch.int32, device=device)
    cd._lib.check(getattr(cd.harness_lib(), entry)(ctypes.c_void_p(scratch.data_ptr()), ctypes.c_void_p(wrong.data_ptr()), 300, None))
    torch.cuda.synchronize()
    assert cd.device_status(clear=False) == (0, 0)
    if not entry.endswith("_lds_only"):
        assert wrong.item() == 0


def test_split_wait_sees_every_phase(device):
    """peek_dma_finish() + wait_for_dma_finish(peeked): the data of every phase is seen, both when the
    peek already found the buffer full and when the wait has to poll."""
    import ctypes
    out = torch.zeros(2, dtype=torch.int32, device=device)
    phases = 200
    cd._lib.check(cd.harness_lib().cudadma_selftest_split_wait(ctypes.c_void_p(out.data_ptr()), phases, None))
    torch.cuda.synchronize()
    wrong, early = out.tolist()
    assert wrong == 0
    assert 0 < early < phases, f"both branches of the split wait should have run ({early} early of {phases})"


@pytest.mark.parametrize("phases", [1, 16, 17, 1000])
def test_all_sixteen_ids_keep_their_own_counts(device, phases):
    """Sixteen sync-only objects, one per dmaID, used round-robin with the DMA side up to sixteen phases
    ahead: no id may see another id's signals."""
    import ctypes
    out = torch.zeros(1, dtype=torch.int32, device=device)
    cd._lib.check(cd.harness_lib().cudadma_selftest_all_ids(ctypes.c_void_p(out.data_ptr()), phases, None))
    torch.cuda.synchronize()
    assert out.item() == 0
