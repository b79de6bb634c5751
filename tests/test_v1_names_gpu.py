"""The first-generation class names (cudaDMASequential, cudaDMAStrided, cudaDMAIndirect with the
constructor forms of include/cudaDMA.h) against the oracle's closed forms, whole LDS window compared."""
import ctypes

import numpy as np
import pytest

import cudadma_amd as cd
from tests import oracle_lib as ol
from tests.oracle_lib import ptr

torch = pytest.importorskip("torch")
pytestmark = pytest.mark.gpu


def _cases():
    try:
        L = cd.harness_lib()
    except cd.CudaDMAError:
        return []
    out = []
    for i in range(L.cudadma_v1_num_cases()):
        c = cd.V1Case()
        cd._lib.check(L.cudadma_v1_get_case(i, ctypes.byref(c)))
        out.append((i, c, L.cudadma_v1_case_text(i).decode()))
    return out


_CASES = _cases()


@pytest.mark.parametrize("case_id", range(len(_CASES)), ids=[t for _, _, t in _CASES])
def test_v1_case(case_id):
    if not torch.cuda.is_available():
        pytest.skip("needs a GPU")
    dev = torch.device("cuda:0")
    _, c, text = _CASES[case_id]
    O = ol.load()
    rng = np.random.default_rng(100 + case_id)
    e, n = c.bytes_per_elmt, c.num_elmts
    src = rng.integers(0, 256, size=64 * 1024, dtype=np.uint8)
    src[src == 0xA5] = 0x5A                               # keep the sentinel out of the data
    want = np.full(c.window_bytes, 0xA5, dtype=np.uint8)
    index = None
    if c.pattern == cd.PATTERN_SEQUENTIAL:
        O.oracle_sequential(ptr(src), ptr(want), e)
    elif c.pattern == cd.PATTERN_STRIDED:
        O.oracle_strided(ptr(src), ptr(want), e, n, c.src_stride, c.dst_stride)
    elif c.pattern == cd.PATTERN_GATHER:
        index = rng.integers(0, src.size // e, size=n).astype(np.int32)
        index[1::4] = index[0]                             # repeated records
        O.oracle_gather(ptr(index), ptr(src), ptr(want), e, n, c.dst_stride)
    else:
        index = rng.permutation(c.window_bytes // e)[:n].astype(np.int32)
        O.oracle_scatter(ptr(index), ptr(src), ptr(want), e, n, c.src_stride)
    d_src = torch.from_numpy(src).to(dev)
    d_idx = torch.from_numpy(index).to(dev) if index is not None else None
    d_out = torch.zeros(c.window_bytes, dtype=torch.uint8, device=dev)
    print(f"v1 case {case_id}: {text}", flush=True)
    cd._lib.check(cd.harness_lib().cudadma_v1_run_case(case_id, ctypes.c_void_p(d_src.data_ptr()),
                                               ctypes.c_void_p(d_idx.data_ptr()) if d_idx is not None else None,
                                               ctypes.c_void_p(d_out.data_ptr()), None))
    torch.cuda.synchronize()
    got = d_out.cpu().numpy()
    assert np.array_equal(got, want), f"{text}: first difference at byte {int(np.argmax(got != want))}"
    assert (want != 0xA5).sum() == (e if c.pattern == cd.PATTERN_SEQUENTIAL else e * n) or c.pattern == cd.PATTERN_GATHER


def test_v1_case_table():
    assert len(_CASES) >= 20
    assert {c.pattern for _, c, _ in _CASES} == {0, 1, 2, 3}
    assert cd.harness_lib().cudadma_v1_case_text(len(_CASES)) is None
