"""The entry point that allocates nothing: cudadma_selftest_global_handoff_noalloc against
cudadma_selftest_global_handoff, whose staging memory the caller brings.  Collected last on purpose."""
import ctypes

import pytest
import torch

import cudadma_amd as cd

pytestmark = pytest.mark.gpu


def _with_callers_memory(device, phases):
    scratch = torch.zeros(4096, dtype=torch.int32, device=device)
    wrong = torch.zeros(1, dtype=torch.int32, device=device)
    cd._lib.check(cd.harness_lib().cudadma_selftest_global_handoff(
        ctypes.c_void_p(scratch.data_ptr()), ctypes.c_void_p(wrong.data_ptr()), phases, None))
    torch.cuda.synchronize()
    return int(wrong.item()), scratch


def _without_allocation(wrong, phases):
    wrong.zero_()
    cd._lib.check(cd.harness_lib().cudadma_selftest_global_handoff_noalloc(ctypes.c_void_p(wrong.data_ptr()), phases, None))
    torch.cuda.synchronize()
    return int(wrong.item())


def test_no_alloc_entry_point_matches_the_one_that_takes_a_workspace(device):
    """Two calls in a row, the second smaller: each must report what the existing entry point reports for the same
    number of phases (no word read back wrong), leave the failure record empty and leave the device's free memory
    as it was."""
    wrong = torch.zeros(1, dtype=torch.int32, device=device)
    expected_big, staged = _with_callers_memory(device, 300)        # also loads the code object both entry points share
    free_before = torch.cuda.mem_get_info()[0]
    got_big = _without_allocation(wrong, 300)
    got_small = _without_allocation(wrong, 7)
    free_after = torch.cuda.mem_get_info()[0]
    expected_small, _ = _with_callers_memory(device, 7)
    assert (got_big, got_small) == (expected_big, expected_small) == (0, 0)
    assert cd.device_status(clear=False) == (0, 0)
    assert free_after == free_before, "the entry point that allocates nothing changed the device's free memory"
    # the caller's workspace of the existing entry point holds the last phase's words in both halves: the kernel ran
    half = staged.numel() // 2
    assert torch.equal(staged[:half], staged[half:]) and int(staged.count_nonzero()) > 0


def test_no_alloc_entry_point_refuses_what_it_cannot_run(device):
    wrong = torch.zeros(1, dtype=torch.int32, device=device)
    L = cd.harness_lib()
    for phases in (0, -1, cd._lib.NOALLOC_MAX_PHASES + 1):
        assert L.cudadma_selftest_global_handoff_noalloc(ctypes.c_void_p(wrong.data_ptr()), phases, None) == -1
        assert b"phases" in cd.lib().cudadma_last_error()
    assert L.cudadma_selftest_global_handoff_noalloc(None, 4, None) == -1
    torch.cuda.synchronize()
    assert int(wrong.item()) == 0
