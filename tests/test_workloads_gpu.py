"""GPU parity of the five benchmark workloads, called through the C ABI.
Small shapes are compared with the oracle element by element; the full benchmark shapes are
checked through properties that do not need a host pass over gigabytes where one would
be slow (double transpose = identity, gather of identity indices = table, linearity)."""
import numpy as np
import pytest
import torch

import cudadma_amd as cd
from cudadma_amd import workloads as wl
from tests import oracle_lib as ol
from tests.oracle_lib import ptr

pytestmark = pytest.mark.gpu


def _variants(w):
    return wl.variants(w)                # the variant numbers the loaded library holds (no GPU needed)


# ------------------------------------------------------------------ generators
def test_device_generators_match_the_host_statement(device):
    n = 1 << 20
    got = wl.fill_uniform(torch.empty(n + 3, dtype=torch.float32, device=device), 1001).cpu().numpy()
    assert np.array_equal(got, ol.uniform(n + 3, 1001))
    idx = wl.fill_indices(torch.empty(n, dtype=torch.int32, device=device), 4096 * 1024, 1003).cpu().numpy()
    assert np.array_equal(idx, ol.indices(n, 4096 * 1024, 1003))


def test_device_generators_match_the_golden_vectors(device):
    """tests/golden/vectors.json was written by pure-Python integer arithmetic, without the oracle."""
    import json
    import os
    with open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "vectors.json")) as f:
        g = json.load(f)
    for seed, bits in g["uniform_bits"].items():
        got = wl.fill_uniform(torch.empty(len(bits), dtype=torch.float32, device=device), int(seed))
        assert [int(v) for v in got.cpu().numpy().view(np.uint32)] == bits
    idx = g["indices"]
    got = wl.fill_indices(torch.empty(idx["n"], dtype=torch.int32, device=device), idx["n_records"], idx["seed"])
    assert [int(v) for v in got.cpu().numpy()] == idx["values"]
    for perm in g["permutations"]:
        got = wl.fill_permutation(torch.empty(1 << perm["log2_n"], dtype=torch.int32, device=device), perm["seed"])
        assert [int(v) for v in got.cpu().numpy()[:len(perm["head"])]] == perm["head"]


@pytest.mark.parametrize("log2_n", [1, 5, 16, 22])
def test_device_permutation_is_one(device, log2_n):
    got = wl.fill_permutation(torch.empty(1 << log2_n, dtype=torch.int32, device=device), 1006)
    assert torch.equal(torch.sort(got).values, torch.arange(1 << log2_n, dtype=torch.int32, device=device))
    assert np.array_equal(got.cpu().numpy(), ol.permutation(log2_n, 1006))


# ------------------------------------------------------------------ config 1
@pytest.mark.parametrize("variant", _variants(wl.SEQUENTIAL))
@pytest.mark.parametrize("tiles", [1, 3, 257, 4096])
def test_sequential_copy(device, variant, tiles):
    n = tiles * wl.SEQ_TILE_BYTES // 4
    src = wl.fill_uniform(torch.empty(n, dtype=torch.float32, device=device), 1001)
    dst = torch.full_like(src, float("nan"))
    print(f"sequential variant {variant} tiles {tiles}", flush=True)
    wl.sequential_copy(src, dst, variant)
    torch.cuda.synchronize()
    assert torch.equal(dst.view(torch.int32), src.view(torch.int32))       # bit-exact, config 1
    if tiles <= 257:
        want = np.empty(n, dtype=np.float32)
        host = ol.uniform(n, 1001)
        ol.load().oracle_copy(ptr(host), ptr(want), n)
        assert np.array_equal(dst.cpu().numpy().view(np.uint32), want.view(np.uint32))


@pytest.mark.parametrize("variant", [0, 5, 6])          # what the library picks beyond the Infinity Cache, and its two walks
def test_sequential_copy_of_a_gibibyte(device, variant):
    """The size of the benchmark's sequential_hbm row: 65 536 tiles, source and destination cut from one allocation."""
    m = (1 << 30) // 4
    pool = torch.empty(2 * m, dtype=torch.float32, device=device)
    src = wl.fill_uniform(pool[:m], 1001)
    dst = pool[m:]
    dst.fill_(float("nan"))
    wl.sequential_copy(src, dst, variant)
    torch.cuda.synchronize()
    assert torch.equal(dst.view(torch.int32), src.view(torch.int32))
    head = ol.uniform(1 << 16, 1001)                       # and the source is what the oracle's generator says
    assert np.array_equal(dst[:1 << 16].cpu().numpy().view(np.uint32), head.view(np.uint32))


def test_sequential_copy_beyond_four_gibibytes(device):
    """5 GiB: byte offsets past 2^32 on both sides (327 680 tiles)."""
    m = 5 * (1 << 28)
    pool = torch.empty(2 * m, dtype=torch.float32, device=device)
    src = wl.fill_uniform(pool[:m], 1001)
    dst = pool[m:]
    dst.fill_(float("nan"))
    wl.sequential_copy(src, dst)
    torch.cuda.synchronize()
    assert torch.equal(dst.view(torch.int32), src.view(torch.int32))


def test_sequential_copy_rejects_ragged_sizes(device):
    src = torch.zeros(5000, dtype=torch.float32, device=device)
    with pytest.raises(cd.CudaDMAError, match="multiple"):
        wl.sequential_copy(src, torch.empty_like(src))
    empty = torch.zeros(0, dtype=torch.float32, device=device)
    wl.sequential_copy(empty, torch.empty_like(empty))                     # empty input is a no-op


def test_plain_copy(device):
    src = wl.fill_uniform(torch.empty(1 << 22, dtype=torch.float32, device=device), 7)
    dst = torch.zeros_like(src)
    wl.plain_copy(src, dst)
    torch.cuda.synchronize()
    assert torch.equal(dst, src)


# ------------------------------------------------------------------ config 2
@pytest.mark.parametrize("variant", _variants(wl.STRIDED))
@pytest.mark.parametrize("n", [64, 192, 1024, 2048, 2112])       # 1, 3, 16, 32 and 33 tiles per side
def test_strided_transpose_small(device, variant, n):
    host = ol.uniform(n * n, 1002).reshape(n, n)
    want = np.empty_like(host)
    ol.load().oracle_transpose(ptr(host), ptr(want), n)
    src = torch.from_numpy(host).to(device)
    dst = torch.full_like(src, float("nan"))
    print(f"transpose variant {variant} n {n}", flush=True)
    wl.strided_transpose(src, dst, variant)
    torch.cuda.synchronize()
    assert np.array_equal(dst.cpu().numpy().view(np.uint32), want.view(np.uint32))


@pytest.mark.parametrize("variant", [0, 10, 1, 4, 11, 14])
@pytest.mark.parametrize("band,workgroups", [(0, 0), (1, 0), (3, 7), (5, 300), (256, 255), (1000, 100000)])
def test_strided_transpose_under_every_tuning(device, variant, band, workgroups):
    """The tile order and the number of workgroups are tuning knobs: the result does not depend on them."""
    n = 1344                                                     # 21 tiles per side
    host = ol.uniform(n * n, 77).reshape(n, n)
    src = torch.from_numpy(host).to(device)
    dst = torch.full_like(src, float("nan"))
    try:
        wl.set_tuning("transpose_band", band)
        wl.set_tuning("transpose_workgroups", workgroups)
        wl.strided_transpose(src, dst, variant)
        torch.cuda.synchronize()
    finally:
        wl.set_tuning("transpose_band", 0)
        wl.set_tuning("transpose_workgroups", 0)
    assert np.array_equal(dst.cpu().numpy().view(np.uint32), np.ascontiguousarray(host.T).view(np.uint32))


_SPLITS = wl.transpose_splits()              # loads the library at collection time (no GPU needed)


@pytest.mark.parametrize("split", _SPLITS)
@pytest.mark.parametrize("n,workgroups", [(64, 0), (1344, 0), (1344, 5), (2112, 700)])
def test_strided_transpose_under_every_split(device, split, n, workgroups):
    """Variant 10 with every compiled split of the workgroup (DMA wavefronts, compute wavefronts, tiles requested ahead):
    the result does not depend on it, whether a workgroup gets one tile, several, or an odd number of them."""
    host = ol.uniform(n * n, 78).reshape(n, n)
    src = torch.from_numpy(host).to(device)
    dst = torch.full_like(src, float("nan"))
    try:
        wl.set_tuning("transpose_split", split)
        wl.set_tuning("transpose_workgroups", workgroups)
        print(f"transpose split {split} n {n} workgroups {workgroups}", flush=True)
        wl.strided_transpose(src, dst, 10)
        torch.cuda.synchronize()
    finally:
        wl.set_tuning("transpose_split", 0)
        wl.set_tuning("transpose_workgroups", 0)
    assert np.array_equal(dst.cpu().numpy().view(np.uint32), np.ascontiguousarray(host.T).view(np.uint32))
    with pytest.raises(cd.CudaDMAError, match="split"):
        try:
            wl.set_tuning("transpose_split", 999)
            wl.strided_transpose(src, dst, 10)
        finally:
            wl.set_tuning("transpose_split", 0)


@pytest.mark.parametrize("variant", [0, 1, 11, 14])               # the reported kernel, its even split and the two forms with two LDS tiles
def test_strided_transpose_full_size(device, variant):
    n = 16384
    src = wl.fill_uniform(torch.empty(n * n, dtype=torch.float32, device=device), 1002).view(n, n)
    dst = torch.empty_like(src)
    wl.strided_transpose(src, dst, variant)
    torch.cuda.synchronize()
    # rows of the oracle's statement on a sample of the output, then transpose twice = identity
    host_rows = ol.uniform(n * n, 1002).reshape(n, n)
    for c in (0, 1, 63, 64, 8191, n - 1):
        assert np.array_equal(dst[c].cpu().numpy(), host_rows[:, c])
    del host_rows
    back = torch.empty_like(src)
    wl.strided_transpose(dst, back, variant)
    torch.cuda.synchronize()
    assert torch.equal(back.view(torch.int32), src.view(torch.int32))


def test_strided_transpose_beyond_four_gibibytes(device):
    """33 792 x 33 792 floats = 4.25 GiB per matrix: element offsets past 2^30, byte offsets past 2^32."""
    n = 33792
    src = wl.fill_uniform(torch.empty(n * n, dtype=torch.float32, device=device), 1002).view(n, n)
    dst = torch.full((n, n), float("nan"), dtype=torch.float32, device=device)
    wl.strided_transpose(src, dst)
    torch.cuda.synchronize()
    for r0 in range(0, n, 4096):                            # against the source read the other way, in bands
        r1 = min(r0 + 4096, n)
        assert torch.equal(dst[r0:r1].view(torch.int32), src[:, r0:r1].t().contiguous().view(torch.int32)), r0


# ------------------------------------------------------------------ config 3
@pytest.mark.parametrize("variant", _variants(wl.GATHER))
@pytest.mark.parametrize("n_tiles", [1, 5, 4099])
def test_gather_small(device, variant, n_tiles):
    recs = 1 << 16
    n_idx = n_tiles * wl.RECS_PER_TILE
    table = ol.uniform(recs * wl.REC_FLOATS, 1003)
    idx = ol.indices(n_idx, recs, 1003)
    want_copy = np.empty(n_idx * wl.REC_FLOATS, dtype=np.float32)
    want_sum = np.empty(n_tiles * wl.REC_FLOATS, dtype=np.float32)
    O = ol.load()
    O.oracle_gather_copy(ptr(table), ptr(idx), ptr(want_copy), n_idx, wl.REC_FLOATS)
    O.oracle_gather_rowsum(ptr(table), ptr(idx), ptr(want_sum), n_idx, wl.REC_FLOATS, wl.RECS_PER_TILE)
    d_table = torch.from_numpy(table).to(device)
    d_idx = torch.from_numpy(idx).to(device)
    print(f"gather variant {variant} tiles {n_tiles}", flush=True)
    got_copy = wl.gather_copy(d_table, d_idx, torch.full((want_copy.size,), float("nan"), device=device), variant)
    got_sum = wl.gather_rowsum(d_table, d_idx, torch.full((want_sum.size,), float("nan"), device=device), variant)
    torch.cuda.synchronize()
    assert np.array_equal(got_copy.cpu().numpy().view(np.uint32), want_copy.view(np.uint32))
    assert np.array_equal(got_sum.cpu().numpy().view(np.uint32), want_sum.view(np.uint32))


@pytest.mark.parametrize("recs", [4 * 1024 * 1024, 32 * 1024 * 1024])     # the configuration's table, and the 4 GiB one of the benchmark's gather_hbm row
def test_gather_full_size(device, recs):
    n_idx = 32 * 1024 * 1024
    table = wl.fill_uniform(torch.empty(recs * wl.REC_FLOATS, dtype=torch.float32, device=device), 1003)
    idx = wl.fill_indices(torch.empty(n_idx, dtype=torch.int32, device=device), recs, 1003)
    out = torch.empty(n_idx * wl.REC_FLOATS, dtype=torch.float32, device=device)
    wl.gather_copy(table, idx, out, 0)
    torch.cuda.synchronize()
    # every record against torch's own gather, in slabs to bound memory
    t2 = table.view(recs, wl.REC_FLOATS)
    o2 = out.view(n_idx, wl.REC_FLOATS)
    slab = 1 << 22
    for s in range(0, n_idx, slab):
        assert torch.equal(o2[s:s + slab].view(torch.int32), t2[idx[s:s + slab].long()].view(torch.int32))
    # the headline consumer on the oracle's statement for a sample of tiles
    sums = torch.empty(n_idx // wl.RECS_PER_TILE * wl.REC_FLOATS, dtype=torch.float32, device=device)
    wl.gather_rowsum(table, idx, sums, 0)
    torch.cuda.synchronize()
    tiles = o2.view(-1, wl.RECS_PER_TILE, wl.REC_FLOATS)
    sample = torch.arange(0, tiles.shape[0], 997, device=device)
    t = tiles[sample].cpu().numpy()
    acc = t[:, 0, :].copy()
    for r in range(1, wl.RECS_PER_TILE):
        acc = acc + t[:, r, :]
    assert np.array_equal(sums.view(-1, wl.REC_FLOATS)[sample].cpu().numpy().view(np.uint32), acc.view(np.uint32))
    # one draw in ten repeats one of the 1024 draws before it (the "10 % duplicates" of the configuration): count the
    # positions of the device-generated list whose value already occurs among the 1024 before it; chance adds
    # 1024 / 4 Mi = 0.02 % of the positions at most
    sample = idx[:1 << 18].cpu().numpy()
    windows = np.lib.stride_tricks.sliding_window_view(sample, 1025)[::37]          # [..., :1024] before, [..., 1024] the draw
    rate = float((windows[:, :1024] == windows[:, 1024:]).any(axis=1).mean())
    assert 0.07 <= rate <= 0.13, rate
    # empty index list is a no-op
    wl.gather_copy(table, idx[:0], out[:0], 0)


# ------------------------------------------------------------------ scatter, LDS -> global
@pytest.mark.parametrize("variant", _variants(wl.SCATTER))
@pytest.mark.parametrize("n_tiles", [1, 5, 2048, 4099])
def test_scatter_small(device, variant, n_tiles):
    log2_recs = 18
    recs = 1 << log2_recs
    n_idx = n_tiles * wl.RECS_PER_TILE                      # 2048 tiles name a quarter of the table, 4099 about half
    records = ol.uniform(n_idx * wl.REC_FLOATS, 1006)
    idx = np.ascontiguousarray(ol.permutation(log2_recs, 1006)[:n_idx])
    want = np.full(recs * wl.REC_FLOATS, np.float32(-7.0))   # records no index names keep this value
    ol.load().oracle_scatter_copy(ptr(records), ptr(idx), ptr(want), n_idx, wl.REC_FLOATS)
    d_table = torch.full((recs * wl.REC_FLOATS,), -7.0, dtype=torch.float32, device=device)
    print(f"scatter variant {variant} tiles {n_tiles}", flush=True)
    wl.scatter_copy(torch.from_numpy(records).to(device), torch.from_numpy(idx).to(device), d_table, variant)
    torch.cuda.synchronize()
    assert np.array_equal(d_table.cpu().numpy().view(np.uint32), want.view(np.uint32))


@pytest.mark.parametrize("log2_recs", [22, 25])          # the benchmark's 512 MiB table, and one of 4 GiB (64-bit offsets)
def test_scatter_full_size(device, log2_recs):
    """Records of 128 B scattered by a permutation, then gathered back by the same indices."""
    recs = 1 << log2_recs
    records = wl.fill_uniform(torch.empty(recs * wl.REC_FLOATS, dtype=torch.float32, device=device), 1006)
    idx = wl.fill_permutation(torch.empty(recs, dtype=torch.int32, device=device), 1006)
    table = torch.full((recs * wl.REC_FLOATS,), float("nan"), dtype=torch.float32, device=device)
    for variant in (_variants(wl.SCATTER) if log2_recs == 22 else [0]):
        print(f"scatter full size variant {variant}", flush=True)
        table.fill_(float("nan"))
        wl.scatter_copy(records, idx, table, variant)
        torch.cuda.synchronize()
        # torch's own indexing states the same thing: row idx[i] of the table is record i
        r2 = records.view(recs, wl.REC_FLOATS)
        t2 = table.view(recs, wl.REC_FLOATS)
        slab = 1 << 20
        for s in range(0, recs, slab):
            assert torch.equal(t2[idx[s:s + slab].long()].view(torch.int32), r2[s:s + slab].view(torch.int32))
    back = torch.empty_like(records)
    wl.gather_copy(table, idx, back, 0)
    torch.cuda.synchronize()
    assert torch.equal(back.view(torch.int32), records.view(torch.int32))
    # an empty index list is a no-op
    wl.scatter_copy(records[:0], idx[:0], table, 0)


def test_scatter_argument_checks(device):
    recs = 1 << 10
    records = torch.zeros(33 * wl.REC_FLOATS, dtype=torch.float32, device=device)
    table = torch.zeros(recs * wl.REC_FLOATS, dtype=torch.float32, device=device)
    idx = torch.zeros(33, dtype=torch.int32, device=device)
    with pytest.raises(cd.CudaDMAError):
        wl.scatter_copy(records, idx, table, 0)                       # 33 is not a multiple of 32
    with pytest.raises(cd.CudaDMAError):
        wl.scatter_copy(records[:32 * wl.REC_FLOATS], idx[:32], table, wl.num_variants(wl.SCATTER))
    with pytest.raises(ValueError):
        wl.fill_permutation(torch.empty(48, dtype=torch.int32, device=device), 1)


# ------------------------------------------------------------------ config 4
STENCIL_RTOL = 1e-5       # benchmark config 4: fp32 within 1e-5 relative of the host reference


def _wide_tiles_refuse(device, variant, shape):
    """Variants 6 and 7 use tiles of 64 x 16 cells: a grid they do not tile is refused on the host, before any launch,
    and the output buffer stays as it was."""
    nx, ny, nz = shape
    p = 2 * wl.STENCIL_RADIUS
    d_in = torch.zeros((nz + p, ny + p, nx + p), dtype=torch.float32, device=device)
    d_out = torch.full((nz, ny, nx), 7.0, dtype=torch.float32, device=device)
    with pytest.raises(cd.CudaDMAError, match="multiple of"):
        wl.halo_stencil(d_in, d_out, variant)
    torch.cuda.synchronize()
    assert bool((d_out == 7.0).all())


@pytest.mark.parametrize("variant", _variants(wl.HALO))
@pytest.mark.parametrize("shape", [(32, 32, 5), (64, 96, 70), (128, 64, 130)])
def test_halo_stencil_small(device, variant, shape):
    nx, ny, nz = shape
    if variant >= 6 and (nx % 64 or ny % 16):
        return _wide_tiles_refuse(device, variant, shape)
    p = 2 * wl.STENCIL_RADIUS
    g = ol.uniform((nx + p) * (ny + p) * (nz + p), 1004).reshape(nz + p, ny + p, nx + p)
    want = np.empty((nz, ny, nx), dtype=np.float32)
    ol.load().oracle_stencil25(ptr(g), ptr(want), nx, ny, nz, wl.STENCIL_RADIUS)
    d_in = torch.from_numpy(g).to(device)
    d_out = torch.full((nz, ny, nx), float("nan"), dtype=torch.float32, device=device)
    print(f"stencil variant {variant} shape {shape}", flush=True)
    wl.halo_stencil(d_in, d_out, variant)
    torch.cuda.synchronize()
    got = d_out.cpu().numpy()
    err = np.abs(got - want)
    assert np.all(err <= STENCIL_RTOL * np.maximum(np.abs(want), 1.0)), float(err.max())


@pytest.mark.parametrize("variant", [0, 1, 2, 6, 7])
@pytest.mark.parametrize("ring", [8, 12])
@pytest.mark.parametrize("remap", [1, 2, 4])
@pytest.mark.parametrize("shape", [(64, 128, 21), (192, 256, 9), (96, 64, 40)])
def test_halo_stencil_under_every_tuning(device, variant, ring, remap, shape):
    """The depth of the DMA wavefront's ring of halo objects and the numbering of the workgroups (slabs per XCD;
    none; compact blocks per XCD where the tile grid divides by 2 x 4: the first two shapes) are tuning knobs: the
    result does not depend on them."""
    nx, ny, nz = shape
    if variant >= 6 and (nx % 64 or ny % 16):
        return _wide_tiles_refuse(device, variant, shape)
    p = 2 * wl.STENCIL_RADIUS
    g = ol.uniform((nx + p) * (ny + p) * (nz + p), 4004).reshape(nz + p, ny + p, nx + p)
    want = np.empty((nz, ny, nx), dtype=np.float32)
    ol.load().oracle_stencil25(ptr(g), ptr(want), nx, ny, nz, wl.STENCIL_RADIUS)
    d_in = torch.from_numpy(g).to(device)
    d_out = torch.full((nz, ny, nx), float("nan"), dtype=torch.float32, device=device)
    print(f"stencil variant {variant} ring {ring} remap {remap} shape {shape}", flush=True)
    try:
        wl.set_tuning("stencil_ring", ring)
        wl.set_tuning("stencil_xcd_remap", remap)
        wl.halo_stencil(d_in, d_out, variant)
        torch.cuda.synchronize()
    finally:
        wl.set_tuning("stencil_ring", 0)
        wl.set_tuning("stencil_xcd_remap", 0)
    got = d_out.cpu().numpy()
    err = np.abs(got - want)
    assert np.all(err <= STENCIL_RTOL * np.maximum(np.abs(want), 1.0)), float(err.max())


@pytest.mark.parametrize("variant", [0, 1, 6])  # the kernel the benchmark reports, its form with the empty/full handshake, and wide tiles
def test_halo_stencil_full_size(device, variant):
    n = 512
    p = 2 * wl.STENCIL_RADIUS
    d_in = wl.fill_uniform(torch.empty((n + p) ** 3, dtype=torch.float32, device=device), 1004).view(n + p, n + p, n + p)
    d_out = torch.empty((n, n, n), dtype=torch.float32, device=device)
    wl.halo_stencil(d_in, d_out, variant)
    torch.cuda.synchronize()
    # slabs of the host statement
    g = ol.uniform((n + p) ** 3, 1004).reshape(n + p, n + p, n + p)
    for z0 in (0, 250, n - 3):
        want = np.empty((3, n, n), dtype=np.float32)
        ol.load().oracle_stencil25(ptr(np.ascontiguousarray(g[z0:z0 + 3 + p])), ptr(want), n, n, 3, wl.STENCIL_RADIUS)
        got = d_out[z0:z0 + 3].cpu().numpy()
        assert np.all(np.abs(got - want) <= STENCIL_RTOL * np.maximum(np.abs(want), 1.0))
    # a constant field has zero Laplacian everywhere (catches a wrong tile or plane anywhere in the grid)
    d_in.fill_(1.0)
    wl.halo_stencil(d_in, d_out, variant)
    torch.cuda.synchronize()
    assert float(d_out.abs().max()) <= 1e-5


@pytest.mark.parametrize("variant", [0, 6])
def test_halo_stencil_beyond_four_gibibytes(device, variant):
    """1024 x 1024 x 1032 cells: input and output each pass 2^32 bytes; the last planes against the host statement."""
    nx = ny = 1024
    nz = 1032
    p = 2 * wl.STENCIL_RADIUS
    d_in = wl.fill_uniform(torch.empty((nz + p) * (ny + p) * (nx + p), dtype=torch.float32, device=device), 1004).view(nz + p, ny + p, nx + p)
    d_out = torch.full((nz, ny, nx), float("nan"), dtype=torch.float32, device=device)
    wl.halo_stencil(d_in, d_out, variant)
    torch.cuda.synchronize()
    for z0 in (0, 517, nz - 3):
        slab = np.ascontiguousarray(d_in[z0:z0 + 3 + p].cpu().numpy())
        want = np.empty((3, ny, nx), dtype=np.float32)
        ol.load().oracle_stencil25(ptr(slab), ptr(want), nx, ny, 3, wl.STENCIL_RADIUS)
        got = d_out[z0:z0 + 3].cpu().numpy()
        assert np.all(np.abs(got - want) <= STENCIL_RTOL * np.maximum(np.abs(want), 1.0)), z0
    d_in.fill_(1.0)
    wl.halo_stencil(d_in, d_out, variant)
    torch.cuda.synchronize()
    assert float(d_out.abs().max()) <= 1e-5


# ------------------------------------------------------------------ config 5
GEMM_RTOL = 1e-2          # benchmark config 5: within 1e-2 relative of the fp32 host GEMM


def test_device_normal_bf16_generator_matches_the_host_statement(device):
    """cudadma_fill_normal_bf16 (what the benchmark's GEMM inputs come from, seeds 1005 and 2005) bit for bit against
    the oracle's generator."""
    n = 1 << 20
    for seed in (1005, 2005):
        want = np.empty(n, dtype=np.uint16)
        ol.load().oracle_fill_normal_bf16(ptr(want), n, seed)
        got = wl.fill_normal_bf16(torch.empty(n, dtype=torch.bfloat16, device=device), seed)
        torch.cuda.synchronize()
        assert np.array_equal(got.view(torch.int16).cpu().numpy().view(np.uint16), want)


def test_device_normal_bf16_generator_matches_the_golden_vectors(device):
    """The same generator against tests/golden/vectors.json (Box-Muller draws written with Python's math module, without
    the oracle; draws near a bf16 rounding boundary left out)."""
    import json
    import os
    with open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "vectors.json")) as f:
        golden = json.load(f)["normal_bf16"]
    for seed, pairs in golden.items():
        n = pairs[-1][0] + 1
        got = wl.fill_normal_bf16(torch.empty(n, dtype=torch.bfloat16, device=device), int(seed))
        torch.cuda.synchronize()
        bits = got.view(torch.int16).cpu().numpy().view(np.uint16)
        assert [[i, int(bits[i])] for i, _ in pairs] == pairs


def _bf16_inputs(m, n, k):
    a = np.empty(m * k, dtype=np.uint16)
    b = np.empty(k * n, dtype=np.uint16)
    O = ol.load()
    O.oracle_fill_normal_bf16(ptr(a), a.size, 1005)
    O.oracle_fill_normal_bf16(ptr(b), b.size, 2005)
    return a.reshape(m, k), b.reshape(k, n)


@pytest.mark.parametrize("variant", _variants(wl.GEMM))
@pytest.mark.parametrize("shape", [(128, 128, 128), (256, 384, 256), (512, 512, 512), (768, 256, 384), (256, 128, 128),
                                   (1024, 256, 896), (256, 256, 128), (256, 512, 640), (768, 1280, 640)])
def test_gemm_small(device, shape, variant):
    m, n, k = shape
    tile_m, tile_n = {0: (128, 128), 1: (128, 128), 2: (128, 256), 3: (256, 128), 4: (256, 128), 5: (256, 256), 6: (256, 256), 7: (256, 256), 8: (256, 256), 9: (256, 256)}[variant]
    if m % tile_m or n % tile_n:
        # a tile shape that does not divide the problem is refused, not rounded
        with pytest.raises(cd.CudaDMAError, match="this variant needs"):
            wl.gemm_bf16(torch.zeros((m, k), dtype=torch.bfloat16, device=device),
                         torch.zeros((k, n), dtype=torch.bfloat16, device=device),
                         torch.zeros((m, n), dtype=torch.float32, device=device), variant)
        return
    a, b = _bf16_inputs(m, n, k)
    want = np.empty((m, n), dtype=np.float32)
    ol.load().oracle_gemm_bf16(ptr(a), ptr(b), ptr(want), m, n, k)
    d_a = torch.from_numpy(a.view(np.int16)).to(device).view(torch.bfloat16)
    d_b = torch.from_numpy(b.view(np.int16)).to(device).view(torch.bfloat16)
    d_c = torch.full((m, n), float("nan"), dtype=torch.float32, device=device)
    print(f"gemm {shape} variant {variant}", flush=True)
    wl.gemm_bf16(d_a, d_b, d_c, variant)
    torch.cuda.synchronize()
    got = d_c.cpu().numpy()
    scale = np.sqrt(k)                      # typical magnitude of an entry
    assert np.all(np.abs(got - want) <= GEMM_RTOL * np.maximum(np.abs(want), scale)), \
        float(np.max(np.abs(got - want)))
    # much tighter in practice: both sides accumulate the same exact bf16 products in fp32
    assert float(np.max(np.abs(got - want))) <= 1e-4 * scale * np.sqrt(k)


@pytest.mark.parametrize("variant", _variants(wl.GEMM))
def test_gemm_full_size(device, variant):
    m = n = k = 4096
    a, b = _bf16_inputs(m, n, k)
    d_a = torch.from_numpy(a.view(np.int16)).to(device).view(torch.bfloat16)
    d_b = torch.from_numpy(b.view(np.int16)).to(device).view(torch.bfloat16)
    d_c = torch.empty((m, n), dtype=torch.float32, device=device)
    wl.gemm_bf16(d_a, d_b, d_c, variant)
    torch.cuda.synchronize()
    got = d_c.cpu().numpy()
    O = ol.load()
    rng = np.random.default_rng(5)
    for row, col in zip(rng.integers(0, m, 400), rng.integers(0, n, 400)):
        want = O.oracle_gemm_bf16_entry(ptr(a), ptr(b), n, k, int(row), int(col))
        assert abs(got[row, col] - want) <= GEMM_RTOL * max(abs(want), 64.0)
    # every tile against the matrix cores' own library path on the same bits
    ref = torch.matmul(d_a.float(), d_b.float())
    assert float((d_c - ref).abs().max()) <= 1e-2 * 64.0


def test_gemm_rejects_ragged_shapes(device):
    a = torch.zeros((100, 128), dtype=torch.bfloat16, device=device)
    b = torch.zeros((128, 128), dtype=torch.bfloat16, device=device)
    c = torch.zeros((100, 128), dtype=torch.float32, device=device)
    with pytest.raises(cd.CudaDMAError, match="multiples"):
        wl.gemm_bf16(a, b, c)


def test_variants_the_library_does_not_hold_are_refused(device):
    """Kernels that only serve the parameter sweeps are left out of the library unless it is built with
    -DHIPDMA_SWEEP_VARIANTS: their variant numbers stay reserved, have no name and are refused before any launch."""
    src = torch.zeros((256, 256), dtype=torch.float32, device=device)
    dst = torch.full_like(src, 7.0)
    for v in set(range(wl.num_variants(wl.STRIDED))) - set(wl.variants(wl.STRIDED)):
        with pytest.raises(cd.CudaDMAError, match="HIPDMA_SWEEP_VARIANTS"):
            wl.strided_transpose(src, dst, v)
    for v in set(range(wl.num_variants(wl.HALO))) - set(wl.variants(wl.HALO)):
        with pytest.raises(cd.CudaDMAError, match="HIPDMA_SWEEP_VARIANTS"):
            wl.halo_stencil(torch.zeros((40, 40, 40), dtype=torch.float32, device=device),
                            torch.zeros((32, 32, 32), dtype=torch.float32, device=device), v)
    a = torch.zeros((256, 256), dtype=torch.bfloat16, device=device)
    for v in set(range(wl.num_variants(wl.GEMM))) - set(wl.variants(wl.GEMM)):
        with pytest.raises(cd.CudaDMAError, match="HIPDMA_SWEEP_VARIANTS"):
            wl.gemm_bf16(a, a, torch.zeros((256, 256), dtype=torch.float32, device=device), v)
    torch.cuda.synchronize()
    assert bool((dst == 7.0).all())
    for split in {311, 312, 221, 222, 313, 228, 411} - set(wl.transpose_splits()):
        wl.set_tuning("transpose_split", split)
        try:
            with pytest.raises(cd.CudaDMAError, match="HIPDMA_SWEEP_VARIANTS"):
                wl.strided_transpose(src, dst, wl.TRANSPOSE_SPLIT_VARIANT)
        finally:
            wl.set_tuning("transpose_split", 0)


# ------------------------------------------------------------------ streaming yardsticks
@pytest.mark.parametrize("workgroups", [1, 7, 512])
def test_yardsticks_move_what_they_say(device, workgroups):
    src = wl.fill_uniform(torch.empty(256 * 256, dtype=torch.float32, device=device), 77)
    nbytes = src.numel() * 4
    for mode, label in enumerate(wl.PROBE_MODES):
        dst = torch.full_like(src, -3.0)
        print(f"yardstick {label} workgroups {workgroups}", flush=True)
        moved = wl.probe_memory(mode, None if label.startswith("write") else src, None if label.startswith("read") else dst, workgroups)
        torch.cuda.synchronize()
        assert moved == nbytes * ((0 if label.startswith("write") else 1) + (0 if label.startswith("read") else 1))
        if label.startswith("read"):
            continue
        if label.startswith("write"):
            assert bool((dst == 1.0).all())
        else:
            assert torch.equal(dst.view(torch.int32), src.view(torch.int32))


@pytest.mark.parametrize("workgroups", [1, 5, 300])
def test_pattern_yardsticks_move_what_they_say(device, workgroups):
    """The yardsticks with the patterns' own addresses, bit for bit against numpy: the xor of the gathered records per tile
    of 32 indices, the scatter by a permutation, the per-workgroup xor of the transposition's source tiles and the
    transposition's destination tiles written in its order."""
    recs, n_idx = 4096, 32 * 96
    table = ol.uniform(recs * 32, 1003)
    idx = ol.indices(n_idx, recs, 1003)
    d_out = torch.zeros(n_idx // 32 * 32, dtype=torch.int32, device=device)
    print(f"pattern yardstick gather_xor workgroups {workgroups}", flush=True)
    moved = wl.probe_pattern("gather_xor", torch.from_numpy(table).to(device), torch.from_numpy(idx).to(device), d_out, workgroups)
    torch.cuda.synchronize()
    assert moved == n_idx * 132 + n_idx // 32 * 128
    want = np.bitwise_xor.reduce(table.view(np.uint32).reshape(recs, 32)[idx].reshape(-1, 32, 32), axis=1)
    assert np.array_equal(d_out.cpu().numpy().view(np.uint32).reshape(-1, 32), want)

    log2 = 12
    records = ol.uniform((1 << log2) * 32, 1006)
    perm = ol.permutation(log2, 1006)
    d_table = torch.full(((1 << log2) * 32,), float("nan"), dtype=torch.float32, device=device)
    print(f"pattern yardstick scatter workgroups {workgroups}", flush=True)
    moved = wl.probe_pattern("scatter", torch.from_numpy(records).to(device), torch.from_numpy(perm).to(device), d_table, workgroups)
    torch.cuda.synchronize()
    assert moved == (1 << log2) * 260
    want = np.empty_like(records).reshape(-1, 32)
    want[perm] = records.reshape(-1, 32)
    assert np.array_equal(d_table.cpu().numpy().view(np.uint32), want.reshape(-1).view(np.uint32))

    n = 320                                                       # 5 x 5 tiles
    host = ol.uniform(n * n, 1002).reshape(n, n)
    d_x = torch.zeros(workgroups * 4, dtype=torch.int32, device=device)
    print(f"pattern yardstick tile_read workgroups {workgroups}", flush=True)
    moved = wl.probe_pattern("tile_read", torch.from_numpy(host).to(device), None, d_x, workgroups)
    torch.cuda.synchronize()
    assert moved == n * n * 4
    tps = n // 64
    want = np.zeros((workgroups, 4), dtype=np.uint32)
    words = host.view(np.uint32)
    for t in range(tps * tps):
        tx, ty = t // tps, t % tps
        tile = words[ty * 64:(ty + 1) * 64, tx * 64:(tx + 1) * 64].reshape(-1, 4)
        want[t % workgroups] ^= np.bitwise_xor.reduce(tile, axis=0)
    assert np.array_equal(d_x.cpu().numpy().view(np.uint32).reshape(-1, 4), want)

    print(f"pattern yardstick tile_copy workgroups {workgroups}", flush=True)
    for side, piece in ((320, 256), (512, 1024), (512, 2048), (320, 1024)):
        mat = ol.uniform(side * side, 1002).reshape(side, side)
        d_h = torch.from_numpy(mat).to(device)
        d_c = torch.zeros((side, side), dtype=torch.float32, device=device)
        wl.set_tuning("probe_piece_bytes", piece)
        try:
            if (side * 4) % piece:
                with pytest.raises(cd.CudaDMAError, match="multiple of the piece"):
                    wl.probe_pattern("tile_copy", d_h, None, d_c, workgroups)
                continue
            moved = wl.probe_pattern("tile_copy", d_h, None, d_c, workgroups)
        finally:
            wl.set_tuning("probe_piece_bytes", 0)
        torch.cuda.synchronize()
        assert moved == 2 * side * side * 4
        t = side // 64
        want = mat.reshape(t, 64, t, 64).transpose(2, 1, 0, 3).reshape(side, side)          # tiles swapped, not transposed inside
        assert np.array_equal(d_c.cpu().numpy().view(np.uint32), np.ascontiguousarray(want).view(np.uint32))

    buf = ol.uniform(1 << 16, 3)                                   # 256 KiB: 1024 granules of 256 B
    d_x = torch.zeros(workgroups * 4, dtype=torch.int32, device=device)
    for mask in (1, 0b1000000001, 0b101010):
        print(f"pattern yardstick masked_read mask {mask} workgroups {workgroups}", flush=True)
        moved = wl.probe_pattern("masked_read", torch.from_numpy(buf).to(device), None, d_x, workgroups, n_records=mask)
        torch.cuda.synchronize()
        assert moved == buf.nbytes // 2
        granules = buf.view(np.uint32).reshape(-1, 16, 4)
        even = np.array([bin(g & mask).count("1") % 2 == 0 for g in range(granules.shape[0])])
        want = np.bitwise_xor.reduce(granules[even].reshape(-1, 4), axis=0)
        got = np.bitwise_xor.reduce(d_x.cpu().numpy().view(np.uint32).reshape(-1, 4), axis=0)    # over the workgroups
        assert np.array_equal(got, want)

    d_m = torch.zeros((n, n), dtype=torch.int32, device=device)
    print(f"pattern yardstick tile_write workgroups {workgroups}", flush=True)
    moved = wl.probe_pattern("tile_write", None, None, d_m, workgroups)
    torch.cuda.synchronize()
    assert moved == n * n * 4
    assert np.array_equal(d_m.cpu().numpy().reshape(-1), np.arange(n * n, dtype=np.int32))


def test_yardstick_argument_checks(device):
    t = torch.zeros(64 * 64, dtype=torch.float32, device=device)
    i = torch.zeros(64, dtype=torch.int32, device=device)
    with pytest.raises(cd.CudaDMAError, match="multiple of 32"):
        wl.probe_pattern("gather_xor", t, i[:40], t.clone(), 4)
    with pytest.raises(cd.CudaDMAError, match="multiple of 64"):
        wl.probe_pattern("tile_write", None, None, torch.zeros((40, 40), dtype=torch.float32, device=device), 4)
    with pytest.raises(cd.CudaDMAError, match="workgroups"):
        wl.probe_pattern("scatter", t, i, t.clone(), 0)
    with pytest.raises(cd.CudaDMAError):
        wl.probe_pattern(len(wl.PATTERN_PROBE_MODES), t, i, t.clone(), 4)
    t = torch.zeros(64 * 64, dtype=torch.float32, device=device)
    with pytest.raises(cd.CudaDMAError):
        wl.probe_memory(len(wl.PROBE_MODES), t, t.clone(), 4)
    with pytest.raises(cd.CudaDMAError):
        wl.probe_memory("copy", t, t.clone(), 0)
    with pytest.raises(cd.CudaDMAError, match="NULL"):
        wl.probe_memory("copy", t, None, 4)


# ------------------------------------------------------------------ read-bandwidth probe (perf_sequential)
_PROBE_QUALIFIERS = [(wl.LOAD_CACHE_ALL, wl.STORE_WRITE_BACK), (wl.LOAD_CACHE_STREAMING, wl.STORE_LDS), (wl.LOAD_CACHE_ALL, wl.STORE_LDS),
                     (wl.LOAD_CACHE_ALL, wl.STORE_LDS_DIRECT), (wl.LOAD_CACHE_STREAMING, wl.STORE_LDS_DIRECT),
                     (wl.LOAD_CACHE_STREAMING, wl.STORE_WRITE_BACK)]


@pytest.mark.parametrize("qualifiers", _PROBE_QUALIFIERS, ids=lambda q: f"load{q[0]}-store{q[1]}")
@pytest.mark.parametrize("buffering", range(4))
@pytest.mark.parametrize("elmt,waves,loops,groups", [(32, 1, 1, 3), (48, 2, 5, 7), (4096, 2, 8, 64), (16384, 4, 3, 33),
                                                     (2064, 7, 2, 5), (16, 1, 9, 2)])
def test_perf_sequential_checksum(device, buffering, elmt, waves, loops, groups, qualifiers):
    """Every byte of every element reaches LDS: per-workgroup sum of the 32-bit words, modulo 2^32, for every
    compiled pair of load and store qualifier (the reference's defaults, non-temporal loads, ds_write_b128,
    global_load_lds)."""
    lq, sq = qualifiers
    total = groups * elmt * loops
    rng = np.random.default_rng(elmt + waves)
    words = rng.integers(0, 2 ** 32, size=total // 4 + 64, dtype=np.uint64).astype(np.uint32)
    src = torch.from_numpy(words.view(np.int32)).to(device)
    sums = torch.zeros(groups, dtype=torch.int32, device=device)
    print(f"perf_sequential elmt {elmt} waves {waves} loops {loops} groups {groups} buffering {buffering} qualifiers {qualifiers}", flush=True)
    n = wl.perf_sequential(src, elmt, waves, buffering, loops, groups, sums, lq, sq)
    torch.cuda.synchronize()
    assert n == total
    want = words[:total // 4].reshape(groups, -1).astype(np.uint64).sum(axis=1).astype(np.uint32)
    assert np.array_equal(sums.cpu().numpy().view(np.uint32), want)


def test_perf_sequential_argument_checks(device):
    src = torch.zeros(1024, dtype=torch.int32, device=device)
    with pytest.raises(cd.CudaDMAError, match="multiple of 16"):
        wl.perf_sequential(src, 40, 1, 0, 1, 1)
    with pytest.raises(cd.CudaDMAError, match="must be 16-byte aligned and hold"):
        wl.perf_sequential(src, 4096, 1, 1, 2, 1)
    with pytest.raises(cd.CudaDMAError, match="unknown buffering"):
        wl.perf_sequential(src, 64, 1, 4, 1, 1)
    with pytest.raises(cd.CudaDMAError, match="the probe is compiled for"):
        wl.perf_sequential(src, 64, 1, 1, 1, 1, None, 1, wl.STORE_LDS)        # LOAD_CACHE_GLOBAL is not among them
    with pytest.raises(cd.CudaDMAError, match="the probe is compiled for"):
        wl.perf_sequential(src, 64, 1, 1, 1, 1, None, wl.LOAD_CACHE_ALL, 2)       # nor a store to global memory
