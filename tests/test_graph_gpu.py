"""The workload entry points under HIP graph capture: they only launch kernels on the stream
they are given (no allocation, no synchronisation), so a captured sequence must replay with the
same results as eager launches, on every replay and with the inputs changed between replays."""
import numpy as np
import pytest
import torch

import cudadma_amd as cd
from cudadma_amd import examples as ex
from cudadma_amd import workloads as wl

pytestmark = pytest.mark.gpu


def test_captured_workloads_replay_like_eager_launches(device):
    n, tiles, recs, n_idx, g = 1024, 64, 4096, 32 * 512, 64
    src = wl.fill_uniform(torch.empty(n * n, dtype=torch.float32, device=device), 7).view(n, n)
    seq_in = wl.fill_uniform(torch.empty(tiles * wl.SEQ_TILE_BYTES // 4, dtype=torch.float32, device=device), 8)
    table = wl.fill_uniform(torch.empty(recs * wl.REC_FLOATS, dtype=torch.float32, device=device), 9)
    idx = wl.fill_indices(torch.empty(n_idx, dtype=torch.int32, device=device), recs, 9)
    p = 2 * wl.STENCIL_RADIUS
    grid = wl.fill_uniform(torch.empty((g + p) ** 3, dtype=torch.float32, device=device), 10).view(g + p, g + p, g + p)
    x = wl.fill_uniform(torch.empty(1 << 16, dtype=torch.float32, device=device), 11)

    out_t = torch.empty_like(src)
    out_s = torch.empty_like(seq_in)
    out_g = torch.empty(n_idx // wl.RECS_PER_TILE * wl.REC_FLOATS, dtype=torch.float32, device=device)
    out_h = torch.empty((g, g, g), dtype=torch.float32, device=device)
    y = torch.zeros_like(x)

    def launch_all():
        wl.strided_transpose(src, out_t, 0)
        wl.sequential_copy(seq_in, out_s, 0)
        wl.gather_rowsum(table, idx, out_g, 0)
        wl.halo_stencil(grid, out_h, 0)
        ex.saxpy(0.5, x, y, 3)

    launch_all()                                     # first calls outside capture (device queries are cached here)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    y.zero_()
    with torch.cuda.graph(graph):
        launch_all()
    for replay in range(3):
        # new inputs in the same buffers, eager result first
        wl.fill_uniform(src.view(-1), 100 + replay)
        wl.fill_uniform(seq_in, 200 + replay)
        wl.fill_uniform(grid.view(-1), 300 + replay)
        y.zero_()
        launch_all()
        torch.cuda.synchronize()
        want = [t.clone() for t in (out_t, out_s, out_g, out_h, y)]
        for t in (out_t, out_s, out_g, out_h):
            t.fill_(float("nan"))
        y.zero_()
        graph.replay()
        torch.cuda.synchronize()
        for name, got, ref in zip(("transpose", "sequential", "gather", "halo", "saxpy"), (out_t, out_s, out_g, out_h, y), want):
            assert torch.equal(got.view(torch.int32), ref.view(torch.int32)), f"{name}, replay {replay}"
    assert torch.equal(out_t, src.t())


def test_workloads_on_two_streams_at_once(device):
    """The handshake words live in each kernel's own LDS, so kernels of different workloads running
    concurrently on two streams cannot disturb each other."""
    n, recs, n_idx = 2048, 1 << 16, 32 * 4096
    src = wl.fill_uniform(torch.empty(n * n, dtype=torch.float32, device=device), 21).view(n, n)
    table = wl.fill_uniform(torch.empty(recs * wl.REC_FLOATS, dtype=torch.float32, device=device), 22)
    idx = wl.fill_indices(torch.empty(n_idx, dtype=torch.int32, device=device), recs, 22)
    out_t = torch.empty_like(src)
    out_g = torch.empty(n_idx * wl.REC_FLOATS, dtype=torch.float32, device=device)
    torch.cuda.synchronize()
    s1, s2 = torch.cuda.Stream(), torch.cuda.Stream()
    for _ in range(10):
        with torch.cuda.stream(s1):
            wl.strided_transpose(src, out_t, 0)
        with torch.cuda.stream(s2):
            wl.gather_copy(table, idx, out_g, 0)
    torch.cuda.synchronize()
    assert torch.equal(out_t, src.t())
    want = table.view(recs, wl.REC_FLOATS)[idx.long()].reshape(-1)
    assert torch.equal(out_g.view(torch.int32), want.view(torch.int32))
