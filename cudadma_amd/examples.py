"""Python face of the example consumers (saxpy, sgemv, 2-D stencil): the programs
the reference ships under src/examples/, here as launchers in libcudadma_amd.so.
Every function takes torch CUDA tensors and launches on torch's current stream."""
import ctypes

import torch

from ._lib import check, lib

SAXPY, SGEMV, STENCIL2D = range(3)
STENCIL2D_RADIUS = 4
STENCIL2D_TILE = (32, 4)


def _stream():
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _p(t):
    return ctypes.c_void_p(t.data_ptr())


def _need(t, what):
    if not (t.is_cuda and t.is_contiguous() and t.dtype == torch.float32):
        raise ValueError(f"{what} must be a contiguous CUDA tensor of float32")


def num_variants(example):
    return lib().cudadma_example_num_variants(example)


def variant_name(example, variant):
    name = lib().cudadma_example_variant_name(example, variant)
    if name is None:
        raise IndexError(f"example {example} has no variant {variant}")
    return name.decode()


def saxpy(a, x, y, variant=3):
    """y <- a*x + y in place (one fused multiply-add per element)."""
    _need(x, "x")
    _need(y, "y")
    if x.numel() != y.numel():
        raise ValueError("x and y differ in length")
    check(lib().cudadma_example_saxpy(variant, float(a), _p(x), _p(y), x.numel(), _stream()))
    return y


def sgemv(alpha, a, x, y, n=None, variant=3):
    """y[:n] <- alpha * A x.  `a` is the column-major matrix as a (m, lda) tensor: a[j, i] = A[i, j]."""
    _need(a, "a")
    _need(x, "x")
    _need(y, "y")
    m, lda = a.shape
    n = lda if n is None else n
    if x.numel() != m or y.numel() < n:
        raise ValueError("x must have m entries and y at least n")
    check(lib().cudadma_example_sgemv(variant, n, m, float(alpha), _p(a), lda, _p(x), _p(y), _stream()))
    return y


def stencil2d(src, dst, variant=0, full_cross=False):
    """src, dst: (dimz+8, dimy+8, dimx+8, 2) float32; interior points of dst are written."""
    _need(src, "src")
    _need(dst, "dst")
    if src.dim() != 4 or src.shape[3] != 2 or src.shape != dst.shape:
        raise ValueError("src and dst must both be (dimz+8, dimy+8, dimx+8, 2)")
    r = STENCIL2D_RADIUS
    dimz, dimy, dimx = (int(s) - 2 * r for s in src.shape[:3])
    check(lib().cudadma_example_stencil2d(variant, _p(src), _p(dst), dimx, dimy, dimz, int(bool(full_cross)), _stream()))
    return dst
