"""The reference's example programs (saxpy, sgemv, 2-D stencil in five buffering styles)
on the wave64 DMA objects, through the C ABI, bit-exact against the CPU oracle."""
import numpy as np
import pytest

import cudadma_amd as cd
from cudadma_amd import examples as ex
from tests import oracle_lib as ol
from tests.oracle_lib import ptr

torch = pytest.importorskip("torch")
pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def dev():
    if not torch.cuda.is_available():
        pytest.skip("needs a GPU")
    cd.lib()
    return torch.device("cuda:0")


def test_variant_tables(dev):
    assert ex.num_variants(ex.SAXPY) == 4 and ex.num_variants(ex.SGEMV) == 4 and ex.num_variants(ex.STENCIL2D) == 5
    assert "double buffer" in ex.variant_name(ex.STENCIL2D, 1)
    with pytest.raises(IndexError):
        ex.variant_name(ex.SAXPY, 4)


@pytest.mark.parametrize("variant", range(4))
@pytest.mark.parametrize("n", [1024, 3 * 1024, 1024 * 1031, 1 << 24])
def test_saxpy(dev, variant, n):
    O = ol.load()
    x, y = ol.uniform(n, 11), ol.uniform(n, 12)
    a = 0.8401877
    want = y.copy()
    O.oracle_saxpy(a, ptr(x), ptr(want), n)
    dx, dy = torch.from_numpy(x).to(dev), torch.from_numpy(y).to(dev)
    ex.saxpy(a, dx, dy, variant)
    torch.cuda.synchronize()
    assert np.array_equal(dy.cpu().numpy(), want)


def test_saxpy_ragged_and_empty(dev):
    O = ol.load()
    x, y = ol.uniform(1000, 13), ol.uniform(1000, 14)
    want = y.copy()
    O.oracle_saxpy(-1.5, ptr(x), ptr(want), 1000)
    dx, dy = torch.from_numpy(x).to(dev), torch.from_numpy(y).to(dev)
    ex.saxpy(-1.5, dx, dy, 0)                              # the baseline takes any length
    assert np.array_equal(dy.cpu().numpy(), want)
    with pytest.raises(cd.CudaDMAError, match="multiple of 1024"):
        ex.saxpy(1.0, dx, dy, 2)
    e = torch.empty(0, dtype=torch.float32, device=dev)
    ex.saxpy(1.0, e, e, 3)


@pytest.mark.parametrize("variant", range(4))
def test_sgemv_reference_driver_case(dev, variant):
    """A[j*n+i] = (i*j)%11, x[j] = j%11, alpha = 2 (sgemv_dma.cu:752-771): exact in any order.
    The reference runs n = m = 896; m is rounded to 1024 here so every variant's column multiple divides it."""
    n, m = 896, 1024
    i, j = np.meshgrid(np.arange(n), np.arange(m), indexing="ij")
    a_int = (i * j) % 11
    x_int = np.arange(m) % 11
    a = torch.from_numpy(np.ascontiguousarray(a_int.T.astype(np.float32))).to(dev)     # (m, lda = n)
    x = torch.from_numpy(x_int.astype(np.float32)).to(dev)
    y = torch.full((n,), -1.0, dtype=torch.float32, device=dev)
    ex.sgemv(2.0, a, x, y, variant=variant)
    torch.cuda.synchronize()
    assert np.array_equal(y.cpu().numpy().astype(np.int64), 2 * (a_int @ x_int))


@pytest.mark.parametrize("variant", range(4))
@pytest.mark.parametrize("n,m,lda", [(128, 512, 128), (200, 1024, 256), (1000, 1536, 1024), (4096, 4096, 4096)])
def test_sgemv_random(dev, variant, n, m, lda):
    O = ol.load()
    a = ol.uniform(m * lda, 21).reshape(m, lda)
    x = ol.uniform(m, 22)
    want = np.empty(n, dtype=np.float32)
    O.oracle_sgemv(n, m, 1.25, ptr(a), lda, ptr(x), ptr(want))
    da, dx = torch.from_numpy(a).to(dev), torch.from_numpy(x).to(dev)
    dy = torch.full((lda,), 3.0, dtype=torch.float32, device=dev)
    ex.sgemv(1.25, da, dx, dy, n=n, variant=variant)
    torch.cuda.synchronize()
    got = dy.cpu().numpy()
    assert np.array_equal(got[:n], want)
    assert np.all(got[n:] == 3.0)                          # rows beyond n are not written


def test_sgemv_argument_checks(dev):
    a = torch.zeros((96, 128), dtype=torch.float32, device=dev)
    x = torch.zeros(96, dtype=torch.float32, device=dev)
    y = torch.zeros(128, dtype=torch.float32, device=dev)
    with pytest.raises(cd.CudaDMAError, match="multiple of 256"):
        ex.sgemv(1.0, a, x, y, variant=0)
    a2 = torch.zeros((64, 100), dtype=torch.float32, device=dev)
    with pytest.raises(cd.CudaDMAError, match="must cover 128 rows"):
        ex.sgemv(1.0, a2, torch.zeros(64, dtype=torch.float32, device=dev), y, variant=2)


@pytest.mark.parametrize("variant", range(5))
@pytest.mark.parametrize("full_cross", [False, True])
@pytest.mark.parametrize("dims", [(32, 4, 2), (96, 20, 6), (960, 160, 8)])
def test_stencil2d(dev, variant, full_cross, dims):
    """Reference geometry (params_directed.h: 960 x 160 tiles of 32 x 4, radius 4) at a few depths."""
    O = ol.load()
    dimx, dimy, dimz = dims
    r = ex.STENCIL2D_RADIUS
    shape = (dimz + 2 * r, dimy + 2 * r, dimx + 2 * r, 2)
    src = ol.uniform(int(np.prod(shape)), 31)
    want = np.full(src.size, -7.0, dtype=np.float32)
    O.oracle_stencil2d(ptr(src), ptr(want), dimx, dimy, dimz, r, r if full_cross else r - 1)
    dsrc = torch.from_numpy(src).to(dev).view(shape)
    ddst = torch.full(shape, -7.0, dtype=torch.float32, device=dev)
    ex.stencil2d(dsrc, ddst, variant, full_cross)
    torch.cuda.synchronize()
    assert np.array_equal(ddst.cpu().numpy().ravel(), want)


def test_stencil2d_argument_checks(dev):
    r = ex.STENCIL2D_RADIUS
    odd = torch.zeros((3 + 2 * r, 4 + 2 * r, 32 + 2 * r, 2), dtype=torch.float32, device=dev)
    with pytest.raises(cd.CudaDMAError, match="must be even"):
        ex.stencil2d(odd, odd.clone(), 1)
    ex.stencil2d(odd, odd.clone(), 0)                      # one buffer: any depth
    bad = torch.zeros((2 + 2 * r, 5 + 2 * r, 32 + 2 * r, 2), dtype=torch.float32, device=dev)
    with pytest.raises(cd.CudaDMAError, match="multiple of"):
        ex.stencil2d(bad, bad.clone(), 0)
