"""Pins the CPU oracle (oracle/oracle.c) without the reference, which cannot be
built here (CUDA + inline PTX).  Each function is checked against
  * the expectations of the reference's own tests (ramp input + exact compare,
    src/tests/test_*/cudaDMA_test_*_v2.cu; check_halo of
    src/tests/test_halo/cudaDMA_test_halo.cu:91-164, restated independently in numpy),
  * the library routine it must reduce to (numpy copy / slicing / take / .T / matmul,
    torch's bf16 rounding),
  * what the mathematics fixes (splitmix64 known answer, stencil exact on polynomials).
"""
import numpy as np
import pytest

from tests import oracle_lib as ol
from tests.oracle_lib import ptr


@pytest.fixture(scope="module")
def O():
    return ol.load()


# ------------------------------------------------------------------ generators
def test_splitmix64_known_answer(O):
    # first output of the published splitmix64 generator seeded with 0
    assert O.oracle_splitmix64(0) == 0xE220A8397B1DCDAF
    # and the mixing function restated with Python integers
    def mix(x):
        m = (1 << 64) - 1
        z = (x + 0x9E3779B97F4A7C15) & m
        z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & m
        z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & m
        return z ^ (z >> 31)
    for x in (1, 2, 1001, 2**63 + 12345, 2**64 - 1):
        assert O.oracle_splitmix64(x) == mix(x)
        assert O.oracle_hash32(x, 7) == mix((x + 7) & ((1 << 64) - 1)) >> 32


def test_uniform_formula_and_range(O):
    n = 100003
    u = ol.uniform(n, 1001)
    h = np.array([O.oracle_hash32(1001, i) for i in range(2000)], dtype=np.uint64)
    expect = ((h >> 8).astype(np.float64) * 2.0 ** -23 - 1.0).astype(np.float32)
    assert np.array_equal(u[:2000], expect)
    assert u.min() >= -1.0 and u.max() < 1.0
    assert abs(float(u.mean())) < 0.01 and abs(float(u.var()) - 1.0 / 3.0) < 0.01
    assert not np.array_equal(u, ol.uniform(n, 1002))


def test_ramp_is_the_reference_input(O):
    assert np.array_equal(ol.ramp(4099), np.arange(4099, dtype=np.float32))


def test_indices_range_and_repeats(O):
    n, recs = 200000, 4096 * 16
    idx = ol.indices(n, recs, 1003)
    assert idx.min() >= 0 and idx.max() < recs
    base = np.array([O.oracle_hash32(1003, i) % recs for i in range(3000)], dtype=np.int32)
    r = np.array([O.oracle_hash32(1003 ^ 0x5bd1e995, i) for i in range(3000)], dtype=np.int64)
    for i in range(3000):
        if i > 1024 and r[i] % 10 == 0:
            j = i - 1 - (r[i] // 10) % 1024
            assert idx[i] == base[j]
        else:
            assert idx[i] == base[i]
    forced = sum(1 for i in range(1025, 3000) if r[i] % 10 == 0) / (3000 - 1025)
    assert 0.07 < forced < 0.13


def test_bf16_rounding_matches_torch(O):
    import torch
    x = np.concatenate([ol.uniform(5000, 5) * 100.0, np.array([0.0, -0.0, 1.0, 1.00390625, 1.01171875, 3.3895314e38,
                                                              np.inf, -np.inf, 1e-40], dtype=np.float32)])
    got = np.array([O.oracle_f32_to_bf16(float(v)) for v in x], dtype=np.uint16)
    want = torch.from_numpy(x).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(got, want)
    back = np.array([O.oracle_bf16_to_f32(int(v)) for v in got], dtype=np.float32)
    assert np.array_equal(back, torch.from_numpy(x).to(torch.bfloat16).to(torch.float32).numpy())


# ------------------------------------------------------------------ transfers
@pytest.mark.parametrize("nbytes", [0, 4, 8, 12, 16, 20, 1024, 4100, 16384])
@pytest.mark.parametrize("off", [0, 1, 3])
def test_sequential_is_memcpy_on_the_ramp(O, nbytes, off):
    # cudaDMA_test_sequential_v2.cu:416-418,501-512: ramp in, exact compare of the moved floats
    src = ol.ramp(nbytes // 4 + off + 8)
    dst = np.zeros_like(src)
    O.oracle_sequential(ptr(src, off * 4), ptr(dst, off * 4), nbytes)
    want = np.zeros_like(src)
    want[off:off + nbytes // 4] = src[off:off + nbytes // 4]
    assert np.array_equal(dst, want)      # also: nothing outside the footprint


@pytest.mark.parametrize("e,n,ss,ds", [(4, 1, 4, 4), (12, 7, 16, 32), (256, 64, 65536 // 64, 272), (1000, 9, 1024, 1000),
                                       (128, 32, 128, 128), (132, 31, 256, 144)])
def test_strided_is_numpy_slicing(O, e, n, ss, ds):
    # cudaDMA_test_strided_v2.cu:561-563,659-677
    src = ol.ramp(n * ss // 4 + 64).view(np.uint8)
    dst = np.zeros(n * ds + 64, dtype=np.uint8)
    O.oracle_strided(ptr(src), ptr(dst), e, n, ss, ds)
    want = np.zeros_like(dst)
    want_rows = np.lib.stride_tricks.as_strided(want, shape=(n, e), strides=(ds, 1))
    src_rows = np.lib.stride_tricks.as_strided(src, shape=(n, e), strides=(ss, 1))
    want_rows[...] = src_rows
    assert np.array_equal(dst, want)
    if e == ss == ds:                     # equal strides and packed rows: plain memcpy
        assert np.array_equal(dst[:n * e], src[:n * e])


@pytest.mark.parametrize("e,n,alt", [(4, 5, 0), (128, 32, 0), (128, 32, 64), (128, 32, 128), (128, 32, 144), (20, 9, 32)])
def test_gather_is_take_and_scatter_inverts_it(O, e, n, alt):
    # cudaDMA_test_indirect_v2.cu:558-560,659-690 (ramp source, non-overlapping element offsets)
    rng = np.random.default_rng(e * 1000 + n)
    table_elems = 3 * n + 5
    table = ol.ramp(table_elems * e // 4).view(np.uint8).reshape(table_elems, e)
    index = rng.permutation(table_elems)[:n].astype(np.int32)
    stride = max(alt, e)
    dst = np.zeros(n * stride + 16, dtype=np.uint8)
    O.oracle_gather(ptr(index), ptr(table), ptr(dst), e, n, alt)
    want = np.zeros_like(dst)
    for r in range(n):
        want[r * stride:r * stride + e] = np.take(table, index[r], axis=0)
    assert np.array_equal(dst, want)
    # duplicates are allowed in a gather
    dup = index.copy()
    dup[n // 2:] = dup[0]
    O.oracle_gather(ptr(dup), ptr(table), ptr(dst), e, n, alt)
    assert np.array_equal(dst[(n - 1) * stride:(n - 1) * stride + e], table[dup[0]])
    # scatter of the gathered rows puts every touched element back where it came from
    back = np.zeros_like(table)
    O.oracle_gather(ptr(index), ptr(table), ptr(dst), e, n, alt)
    O.oracle_scatter(ptr(index), ptr(dst), ptr(back), e, n, alt)
    want_back = np.zeros_like(table)
    want_back[index] = table[index]
    assert np.array_equal(back, want_back)


def numpy_check_halo(idata, odata, radius, corners, dimx, dimy, pitch):
    """check_halo of the reference (cudaDMA_test_halo.cu:91-164) on 2-D views of cells."""
    i2 = idata[:(dimy + 2 * radius) * pitch].reshape(dimy + 2 * radius, pitch, -1)
    o2 = odata[:(dimy + 2 * radius) * (dimx + 2 * radius)].reshape(dimy + 2 * radius, dimx + 2 * radius, -1)
    c0, c1 = (0, dimx + 2 * radius) if corners else (radius, radius + dimx)
    ok = np.array_equal(i2[:radius, c0:c1], o2[:radius, c0:c1])
    ok &= np.array_equal(i2[radius + dimy:, c0:c1], o2[radius + dimy:, c0:c1])
    ok &= np.array_equal(i2[radius:radius + dimy, :radius], o2[radius:radius + dimy, :radius])
    ok &= np.array_equal(i2[radius:radius + dimy, radius + dimx:radius + dimx + radius],
                         o2[radius:radius + dimy, radius + dimx:])
    return bool(ok)


@pytest.mark.parametrize("es", [4, 8, 16])
@pytest.mark.parametrize("radius,corners,dimx,dimy,extra", [(1, 0, 8, 8, 0), (3, 1, 17, 9, 5), (4, 0, 32, 32, 0),
                                                            (8, 1, 63, 20, 3), (2, 1, 13, 21, 1)])
def test_halo_matches_the_reference_checker(O, es, radius, corners, dimx, dimy, extra):
    cells = es // 4
    pitch = dimx + 2 * radius + extra
    rng = np.random.default_rng(radius * 100 + dimx)
    # cudaDMA_test_halo.cu:245-246: rand()%10 cells
    idata = rng.integers(0, 10, size=(dimy + 2 * radius) * pitch * cells).astype(np.float32).reshape(-1, cells)
    odata = np.zeros(((dimx + 2 * radius) * (dimy + 2 * radius), cells), dtype=np.float32)
    src_origin = (radius * pitch + radius) * es
    dst_origin = (radius * (dimx + 2 * radius) + radius) * es
    O.oracle_halo(ptr(idata, src_origin), ptr(odata, dst_origin), es, radius, corners, dimx, dimy, pitch)
    assert numpy_check_halo(idata, odata, radius, corners, dimx, dimy, pitch)
    assert O.oracle_halo_check(ptr(idata), ptr(odata), es, radius, corners, dimx, dimy, pitch) == 1
    # stricter than the reference: interior (and corners when off) stay zero
    o2 = odata.reshape(dimy + 2 * radius, dimx + 2 * radius, cells)
    assert not o2[radius:radius + dimy, radius:radius + dimx].any()
    if not corners:
        assert not o2[:radius, :radius].any() and not o2[-radius:, -radius:].any()
    # total bytes moved = ring area
    ring = 2 * radius * (dimx + (2 * radius if corners else 0)) + 2 * radius * dimy
    i2 = idata.reshape(dimy + 2 * radius, pitch, cells)[:, :dimx + 2 * radius]
    assert np.count_nonzero(o2 != 0) <= ring * cells
    mask = np.ones((dimy + 2 * radius, dimx + 2 * radius), dtype=bool)
    mask[radius:radius + dimy, radius:radius + dimx] = False
    if not corners:
        for ys in (slice(0, radius), slice(radius + dimy, None)):
            for xs in (slice(0, radius), slice(radius + dimx, None)):
                mask[ys, xs] = False
    assert np.array_equal(o2[mask], i2[mask])
    # the checker itself notices a wrong cell
    bad = odata.copy()
    bad[radius * (dimx + 2 * radius)] += 1.0          # first cell of the left panel
    assert O.oracle_halo_check(ptr(idata), ptr(bad), es, radius, corners, dimx, dimy, pitch) == 0
    assert not numpy_check_halo(idata, bad, radius, corners, dimx, dimy, pitch)


@pytest.mark.parametrize("es", [4, 8, 16])
@pytest.mark.parametrize("radius,corners,dimx,dimy,extra,dst_extra", [(1, 0, 8, 8, 0, 1), (3, 1, 17, 9, 5, 3), (4, 0, 32, 32, 0, 8),
                                                                      (8, 1, 63, 20, 3, 1), (2, 1, 13, 21, 1, 0)])
def test_halo_with_a_destination_pitch(O, es, radius, corners, dimx, dimy, extra, dst_extra):
    """oracle_halo_pitched against numpy slicing of the two padded tiles: the ring lands in rows of dst_pitch
    cells, nothing else is written, and dst_pitch = dimx + 2*radius is oracle_halo itself."""
    cells = es // 4
    pitch = dimx + 2 * radius + extra
    dst_pitch = dimx + 2 * radius + dst_extra
    rows = dimy + 2 * radius
    rng = np.random.default_rng(radius * 31 + dimx + dst_extra)
    idata = rng.integers(1, 1000, size=(rows, pitch, cells)).astype(np.float32)
    odata = np.zeros((rows, dst_pitch, cells), dtype=np.float32)
    O.oracle_halo_pitched(ptr(idata, (radius * pitch + radius) * es), ptr(odata, (radius * dst_pitch + radius) * es),
                          es, radius, corners, dimx, dimy, pitch, dst_pitch)
    want = np.zeros_like(odata)
    c0, c1 = (0, dimx + 2 * radius) if corners else (radius, radius + dimx)
    want[:radius, c0:c1] = idata[:radius, c0:c1]
    want[radius + dimy:, c0:c1] = idata[radius + dimy:, c0:c1]
    want[radius:radius + dimy, :radius] = idata[radius:radius + dimy, :radius]
    want[radius:radius + dimy, radius + dimx:2 * radius + dimx] = idata[radius:radius + dimy, radius + dimx:2 * radius + dimx]
    assert np.array_equal(odata, want)
    if dst_extra == 0:
        ref = np.zeros_like(odata)
        O.oracle_halo(ptr(idata, (radius * pitch + radius) * es), ptr(ref, (radius * dst_pitch + radius) * es),
                      es, radius, corners, dimx, dimy, pitch)
        assert np.array_equal(ref, odata)


# ------------------------------------------------------------------ workloads
def test_copy_and_transpose(O):
    a = ol.uniform(256 * 256, 1002).reshape(256, 256)
    out = np.empty_like(a)
    O.oracle_copy(ptr(a), ptr(out), a.size)
    assert np.array_equal(out, a)
    O.oracle_transpose(ptr(a), ptr(out), 256)
    assert np.array_equal(out, a.T)
    ramp = ol.ramp(192 * 192).reshape(192, 192)
    out = np.empty_like(ramp)
    O.oracle_transpose(ptr(ramp), ptr(out), 192)
    assert out[5, 7] == 7 * 192 + 5


def test_gather_copy_and_rowsum(O):
    recs, n_idx = 4096, 32 * 300
    table = ol.uniform(recs * 32, 1003).reshape(recs, 32)
    idx = ol.indices(n_idx, recs, 1003)
    out = np.empty((n_idx, 32), dtype=np.float32)
    O.oracle_gather_copy(ptr(table), ptr(idx), ptr(out), n_idx, 32)
    assert np.array_equal(out, table[idx])
    sums = np.empty((n_idx // 32, 32), dtype=np.float32)
    O.oracle_gather_rowsum(ptr(table), ptr(idx), ptr(sums), n_idx, 32, 32)
    tiles = table[idx].reshape(-1, 32, 32)
    acc = tiles[:, 0, :].copy()
    for r in range(1, 32):
        acc = acc + tiles[:, r, :]                    # float32, ascending record order
    assert np.array_equal(sums, acc)
    # a different order gives different bits somewhere: the order is part of the statement
    rev = tiles[:, 31, :].copy()
    for r in range(30, -1, -1):
        rev = rev + tiles[:, r, :]
    assert not np.array_equal(sums, rev)
    assert np.allclose(sums, tiles.astype(np.float64).sum(axis=1), rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("log2_n", [1, 2, 3, 7, 12, 20])
@pytest.mark.parametrize("seed", [0, 1006, 2**63 + 5])
def test_permutation_is_one(O, log2_n, seed):
    p = ol.permutation(log2_n, seed)
    assert np.array_equal(np.sort(p), np.arange(1 << log2_n, dtype=np.int32))
    if log2_n >= 12:                                     # and not the identity or a plain rotation
        assert np.count_nonzero(np.diff(p.astype(np.int64)) == 1) < (1 << log2_n) // 16
        assert not np.array_equal(p, ol.permutation(log2_n, seed + 1))


def test_scatter_copy_inverts_gather_copy(O):
    log2_recs, n_idx = 12, 32 * 100
    recs = 1 << log2_recs
    records = ol.uniform(n_idx * 32, 1006).reshape(n_idx, 32)
    idx = np.ascontiguousarray(ol.permutation(log2_recs, 1006)[:n_idx])
    table = np.full((recs, 32), np.float32(-7.0))
    O.oracle_scatter_copy(ptr(records), ptr(idx), ptr(table), n_idx, 32)
    want = np.full((recs, 32), np.float32(-7.0))
    want[idx] = records                                   # numpy's own scatter
    assert np.array_equal(table, want)
    back = np.empty_like(records)
    O.oracle_gather_copy(ptr(table), ptr(idx), ptr(back), n_idx, 32)
    assert np.array_equal(back, records)
    # the same statement as one transfer of the scatter object over the whole list
    table2 = np.full((recs, 32), np.float32(-7.0))
    O.oracle_scatter(ptr(idx), ptr(records), ptr(table2), 128, n_idx, 0)
    assert np.array_equal(table2, want)


def stencil_numpy64(g, nx, ny, nz, p):
    c = [3.0 * (-205.0 / 72.0), 8.0 / 5.0, -1.0 / 5.0, 8.0 / 315.0, -1.0 / 560.0]
    g = g.astype(np.float64)
    core = (slice(p, p + nz), slice(p, p + ny), slice(p, p + nx))
    out = c[0] * g[core]
    for r in range(1, 5):
        for ax in range(3):
            for s in (-r, r):
                sl = list(core)
                sl[ax] = slice(core[ax].start + s, core[ax].stop + s)
                out = out + c[r] * g[tuple(sl)]
    return out


def test_stencil_against_numpy_and_polynomials(O):
    nx, ny, nz, p = 32, 32, 12, 4
    g = ol.uniform((nx + 2 * p) * (ny + 2 * p) * (nz + 2 * p), 1004).reshape(nz + 2 * p, ny + 2 * p, nx + 2 * p)
    out = np.empty((nz, ny, nx), dtype=np.float32)
    O.oracle_stencil25(ptr(g), ptr(out), nx, ny, nz, p)
    ref = stencil_numpy64(g, nx, ny, nz, p)
    assert np.max(np.abs(out - ref)) <= 1e-5 * np.max(np.abs(ref))
    # a constant field has zero Laplacian; x^2 + 2y^2 + 3z^2 has Laplacian 12; the 8th-order
    # stencil is exact for polynomials up to degree 9, so x^4 at x gives 12 x^2
    z, y, x = np.meshgrid(np.arange(nz + 2 * p), np.arange(ny + 2 * p), np.arange(nx + 2 * p), indexing="ij")
    for field, want in ((np.ones_like(x), lambda X, Y, Z: 0.0 * X),
                        (x * x + 2 * y * y + 3 * z * z, lambda X, Y, Z: 12.0 + 0.0 * X),
                        (x ** 4 // 1, lambda X, Y, Z: 12.0 * X * X)):
        f32 = field.astype(np.float32)
        O.oracle_stencil25(ptr(f32), ptr(out), nx, ny, nz, p)
        core = want(x[p:-p, p:-p, p:-p].astype(np.float64), None, None)
        scale = max(1.0, float(np.max(np.abs(f32))))
        assert np.max(np.abs(out - core)) <= 2e-5 * scale, (np.max(np.abs(out - core)), scale)
    # anisotropy check: a wrong axis pitch would mix y and z
    f32 = (z.astype(np.float32)) ** 2
    O.oracle_stencil25(ptr(f32), ptr(out), nx, ny, nz, p)
    assert np.max(np.abs(out - 2.0)) < 1e-2


def test_gemm_bf16(O):
    m, n, k = 96, 80, 160
    a = np.empty(m * k, dtype=np.uint16)
    b = np.empty(k * n, dtype=np.uint16)
    O.oracle_fill_normal_bf16(ptr(a), a.size, 1005)
    O.oracle_fill_normal_bf16(ptr(b), b.size, 2005)
    def widen(u):
        return (u.astype(np.uint32) << 16).view(np.float32)
    af, bf = widen(a).reshape(m, k), widen(b).reshape(k, n)
    assert abs(float(af.mean())) < 0.05 and abs(float(af.std()) - 1.0) < 0.05   # normal(0,1)
    c = np.empty((m, n), dtype=np.float32)
    O.oracle_gemm_bf16(ptr(a), ptr(b), ptr(c), m, n, k)
    ref = af.astype(np.float64) @ bf.astype(np.float64)
    assert np.max(np.abs(c - ref)) <= 1e-4 * np.max(np.abs(ref))
    assert abs(O.oracle_gemm_bf16_entry(ptr(a), ptr(b), n, k, 5, 7) - c[5, 7]) <= 1e-5 * abs(c[5, 7]) + 1e-6


# ---- consumers of the reference's example programs ----

def _round_f32(fr):
    """The float32 nearest to an exact rational (ties to even), decided with exact arithmetic."""
    from fractions import Fraction
    c = np.float32(float(fr))
    best = c
    for cand in (np.nextafter(c, np.float32(-np.inf)), np.nextafter(c, np.float32(np.inf))):
        dc, db = abs(Fraction(float(cand)) - fr), abs(Fraction(float(best)) - fr)
        if dc < db or (dc == db and (int(np.float32(cand).view(np.uint32)) & 1) == 0):
            best = cand
    return np.float32(best)


def test_saxpy_is_one_correctly_rounded_operation(O):
    """y = fma(a, x, y): checked against exact rational arithmetic (a plain a*x rounded before the add
    would differ on some of these samples), and against the reference's own tolerance on all."""
    from fractions import Fraction
    n = 4096
    x, y0 = ol.uniform(n, 71), ol.uniform(n, 72)
    a = np.float32(0.8401877)           # first rand()/RAND_MAX of glibc srand(0), as saxpy_cudaDMA.cu:89-93 draws it
    y = y0.copy()
    O.oracle_saxpy(a, ptr(x), ptr(y), n)
    two_step = (a * x + y0).astype(np.float32)
    assert np.max(np.abs(y - two_step)) <= 1e-6          # the example's PASSED criterion (saxpy_cudaDMA.cu:171)
    assert not np.array_equal(y, two_step)               # ... and the fused form is distinguishable from it
    for i in range(0, n, 13):
        want = _round_f32(Fraction(float(a)) * Fraction(float(x[i])) + Fraction(float(y0[i])))
        assert y[i] == want, i


def test_sgemv_known_answer_of_the_reference_driver(O):
    """The reference's driver fills A[j*n+i] = (i*j)%11, x[j] = j%11, alpha = 2 at n = m = 896
    (sgemv_dma.cu:752-771, 72-73): small integers, so every order of summation is exact and the
    answer is plain integer arithmetic."""
    n = m = 896
    i, j = np.meshgrid(np.arange(n), np.arange(m), indexing="ij")
    a_int = (i * j) % 11                                  # [row i, column j]
    x_int = np.arange(m) % 11
    a = np.asfortranarray(a_int.astype(np.float32))       # column-major, lda = n
    x = x_int.astype(np.float32)
    y = np.empty(n, dtype=np.float32)
    O.oracle_sgemv(n, m, 2.0, ptr(a), n, ptr(x), ptr(y))
    assert np.array_equal(y.astype(np.int64), 2 * (a_int @ x_int))


def test_sgemv_order_lda_and_fusion(O):
    from fractions import Fraction
    n, m, lda = 5, 24, 9
    a = ol.uniform(lda * m, 81)
    x = ol.uniform(m, 82)
    y = np.empty(n, dtype=np.float32)
    alpha = np.float32(1.7)
    O.oracle_sgemv(n, m, alpha, ptr(a), lda, ptr(x), ptr(y))
    for row in range(n):
        res = np.float32(0.0)
        for col in range(m):
            res = _round_f32(Fraction(float(a[row + col * lda])) * Fraction(float(x[col])) + Fraction(float(res)))
        assert y[row] == np.float32(alpha * res)
    # against numpy in double, as a sanity bound that would catch a transposed matrix or a wrong lda
    ref = a.reshape(m, lda)[:, :n].T.astype(np.float64) @ x.astype(np.float64)
    assert np.max(np.abs(y - alpha * ref)) < 1e-5


def _stencil2d_numpy(src, dimx, dimy, dimz, r, reach):
    """Same additions in the same order, one numpy float32 operation per step."""
    g = src.reshape(dimz + 2 * r, dimy + 2 * r, dimx + 2 * r, 2)
    core = lambda dy, dx: g[r:r + dimz, r + dy:r + dy + dimy, r + dx:r + dx + dimx, :]
    acc = core(0, 0).copy()
    for d in range(1, reach + 1):
        acc = acc + core(0, -d)
    for d in range(1, reach + 1):
        acc = acc + core(0, d)
    for d in range(1, reach + 1):
        acc = acc + core(-d, 0)
    for d in range(1, reach + 1):
        acc = acc + core(d, 0)
    return acc / np.float32(4 * r + 1)


@pytest.mark.parametrize("r,reach", [(4, 3), (4, 4), (2, 1), (1, 0)])
def test_stencil2d_against_numpy_and_closed_forms(O, r, reach):
    dimx, dimy, dimz = 24, 10, 3
    total = (dimx + 2 * r) * (dimy + 2 * r) * (dimz + 2 * r)
    src = ol.uniform(2 * total, 91)
    dst = np.full(2 * total, 7.5, dtype=np.float32)
    O.oracle_stencil2d(ptr(src), ptr(dst), dimx, dimy, dimz, r, reach)
    got = dst.reshape(dimz + 2 * r, dimy + 2 * r, dimx + 2 * r, 2)
    assert np.array_equal(got[r:-r, r:-r, r:-r, :], _stencil2d_numpy(src, dimx, dimy, dimz, r, reach))
    mask = np.ones(got.shape, dtype=bool)
    mask[r:-r, r:-r, r:-r, :] = False
    assert np.all(got[mask] == 7.5)                       # nothing outside the interior is written
    # a constant field: (1 + 4*reach) / (4r + 1), which is 1 only when the whole radius is summed
    one = np.ones(2 * total, dtype=np.float32)
    O.oracle_stencil2d(ptr(one), ptr(dst), dimx, dimy, dimz, r, reach)
    want = np.float32(1 + 4 * reach) / np.float32(4 * r + 1)
    assert np.all(got[r:-r, r:-r, r:-r, :] == want)
    # a field that depends on z only: the stencil must not look across slices
    zf = np.repeat(np.arange(dimz + 2 * r, dtype=np.float32), (dimy + 2 * r) * (dimx + 2 * r) * 2)
    O.oracle_stencil2d(ptr(zf), ptr(dst), dimx, dimy, dimz, r, reach)
    for z in range(dimz):
        assert np.allclose(got[r + z, r:-r, r:-r, :], (z + r) * want, rtol=1e-6)


# ---- the committed golden vectors (tests/golden/vectors.json, written by make_vectors.py without the oracle) ----

def _golden():
    import json
    import os
    with open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "vectors.json")) as f:
        return json.load(f)


def test_golden_generators(O):
    g = _golden()
    for x, want in g["splitmix64"].items():
        assert O.oracle_splitmix64(int(x)) == int(want)
    for seed, bits in g["uniform_bits"].items():
        got = ol.uniform(len(bits), int(seed)).view(np.uint32)
        assert [int(v) for v in got] == bits
    idx = g["indices"]
    assert [int(v) for v in ol.indices(idx["n"], idx["n_records"], idx["seed"])] == idx["values"]
    for perm in g["permutations"]:
        if perm["log2_n"] <= 22:                       # the 2^31 case is checked on its formula below
            got = ol.permutation(perm["log2_n"], perm["seed"])
            assert [int(v) for v in got[:len(perm["head"])]] == perm["head"]


def test_golden_normal_bf16(O):
    """Box-Muller draws written by make_vectors.py with Python's math module (draws near a bf16 rounding boundary left
    out): pins which hash feeds the radius and which the angle, the cosine, and the rounding to bf16."""
    for seed, pairs in _golden()["normal_bf16"].items():
        n = pairs[-1][0] + 1
        got = np.empty(n, dtype=np.uint16)
        O.oracle_fill_normal_bf16(ptr(got), n, int(seed))
        assert [[i, int(got[i])] for i, _ in pairs] == pairs


def test_golden_strided_ramp_and_halo_ring(O):
    g = _golden()
    for case in g["strided_ramp"]:
        e, n, ss, ds = case["e_floats"], case["n"], case["src_stride_floats"], case["dst_stride_floats"]
        src = ol.ramp(n * ss + e)
        dst = np.full(n * ds + e, -1.0, dtype=np.float32)
        O.oracle_strided(ptr(src), ptr(dst), 4 * e, n, 4 * ss, 4 * ds)
        assert [int(v) for v in dst] == case["dst"]
    for case in g["halo_ring"]:
        dx, dy, r, c, p = case["dimx"], case["dimy"], case["radius"], case["corners"], case["pitch"]
        rows, w = dy + 2 * r, dx + 2 * r
        src = (np.arange(rows * p, dtype=np.int64) + 1)
        dst = np.zeros(rows * w, dtype=np.int64)
        O.oracle_halo(ptr(src, 8 * (r * p + r)), ptr(dst, 8 * (r * w + r)), 8, r, c, dx, dy, p)
        assert [int(v) for v in dst] == case["dst"]
        assert O.oracle_halo_check(ptr(src), ptr(dst), 8, r, c, dx, dy, p) == 1


def test_golden_sgemv_of_the_reference_driver(O):
    g = _golden()["sgemv_reference_driver"]
    n, m = g["n"], g["m"]
    i, j = np.meshgrid(np.arange(n), np.arange(m), indexing="ij")
    a = np.asfortranarray(((i * j) % 11).astype(np.float32))
    x = (np.arange(m) % 11).astype(np.float32)
    y = np.empty(n, dtype=np.float32)
    O.oracle_sgemv(n, m, float(g["alpha"]), ptr(a), n, ptr(x), ptr(y))
    assert [int(v) for v in y] == g["y"]


# ---- the swizzled LDS layout (an addition of this library) ----

def _bitrev(v, bits):
    out = 0
    for _ in range(bits):
        out = (out << 1) | (v & 1)
        v >>= 1
    return out


# chunk bytes, chunks per row, bits of the key, rows per 256-byte bank line
@pytest.mark.parametrize("chunk,chunks,bits,rows_per_line", [(16, 16, 4, 1), (16, 8, 3, 2), (16, 20, 2, 4), (4, 64, 6, 1),
                                                              (8, 1, 0, 32), (16, 6, 1, 8), (4, 5, 0, 64), (16, 32, 4, 1),
                                                              (4, 16, 4, 4)])
def test_strided_swizzled_is_a_row_wise_xor_permutation(O, chunk, chunks, bits, rows_per_line):
    e, n = chunk * chunks, 37
    ss, ds = e + 3 * chunk, e + chunk
    rng = np.random.default_rng(chunks)
    src = rng.integers(0, 256, size=n * ss, dtype=np.uint8)
    plain = np.zeros(n * ds, dtype=np.uint8)
    swz = np.zeros(n * ds, dtype=np.uint8)
    O.oracle_strided(ptr(src), ptr(plain), e, n, ss, ds)
    O.oracle_strided_swizzled(ptr(src), ptr(swz), e, n, ss, ds, chunk)
    p = plain.reshape(n, ds)[:, :e].reshape(n, chunks, chunk)
    s = swz.reshape(n, ds)[:, :e].reshape(n, chunks, chunk)
    key = np.array([_bitrev((r // rows_per_line) & ((1 << bits) - 1), bits) for r in range(n)])
    pos = np.arange(chunks)[None, :] ^ key[:, None]                          # position of chunk c in row r
    assert pos.max() < chunks
    want = np.empty_like(p)
    want[np.arange(n)[:, None], pos] = p                                     # numpy scatter, no oracle arithmetic
    assert np.array_equal(s, want)
    assert np.array_equal(swz.reshape(n, ds)[:, e:], plain.reshape(n, ds)[:, e:])   # padding untouched
    # an involution: reading position c ^ key(r) gives chunk c back
    assert np.array_equal(s[np.arange(n)[:, None], pos], p)
    if bits:
        assert not np.array_equal(s, p)


def test_swizzle_keys_spread_over_the_bank_line():
    """What the layout is for, checked on the key function alone: sixteen consecutive rows of a 256-byte row get
    sixteen different keys (column reads), two rows sharing a bank line get the same key but sixteen consecutive
    128-byte rows cover all sixteen 16-byte units, and four consecutive rows land in four different quarters."""
    key16 = [_bitrev(r & 15, 4) for r in range(16)]
    assert sorted(key16) == list(range(16))
    assert sorted(k >> 2 for k in key16[:4]) == [0, 1, 2, 3] and sorted(k >> 2 for k in key16[8:12]) == [0, 1, 2, 3]
    units = {((r & 1) * 8 + (5 ^ _bitrev((r >> 1) & 7, 3))) for r in range(16)}      # chunk 5 of 128-byte rows
    assert len(units) == 16
