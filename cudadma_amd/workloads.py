"""Python face of the benchmark workloads.  Every function takes torch CUDA
tensors, launches on torch's current stream and returns the output tensor; all
compute happens in libcudadma_amd.so."""
import ctypes

import torch

from ._lib import check, lib

SEQUENTIAL, STRIDED, GATHER, HALO, GEMM, SCATTER = range(6)

REC_FLOATS = 32          # 128-byte records
RECS_PER_TILE = 32
SEQ_TILE_BYTES = 16 * 1024
STENCIL_RADIUS = 4
TRANSPOSE_SPLIT_VARIANT = 10           # cudadma_strided_transpose variant whose wavefront split follows the knob "transpose_split"
# knob values = 100 x DMA wavefronts + 10 x compute wavefronts + tiles ahead; transpose_splits() lists those the loaded library
# holds (311, 312, 221, 222; a library built with -DHIPDMA_SWEEP_VARIANTS also every other split, "tiles ahead" 3 to 7 with three
# DMA wavefronts and one compute wavefront for a tile requested in pieces: 3 halves (1.5 tiles), 5, 6 and 7 quarters (1.25, 1.5,
# 1.75 tiles) and 3 quarters (0.75) in flight, and 8 for one tile in flight without a pause)
TRANSPOSE_TWO_LDS_TILES_VARIANT = 11    # two LDS tiles and two CudaDMAStrided objects (manual double buffering in LDS)
TRANSPOSE_DOUBLE_LDS_VARIANT = 14       # two LDS tiles filled in turn by one object, one tile of loads in flight
HALO_WIDE_TILES_VARIANT = 6            # cudadma_halo_stencil variant 0 with tiles of 64 x 16 cells
GEMM_WARP_SPECIALISED_VARIANT = 7      # the cudadma_gemm_bf16 variant in which DMA wavefronts feed compute wavefronts


def _stream():
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _p(t):
    return ctypes.c_void_p(t.data_ptr())


def _need(t, dtype, what):
    if not (t.is_cuda and t.is_contiguous() and t.dtype == dtype):
        raise ValueError(f"{what} must be a contiguous CUDA tensor of {dtype}")


def num_variants(workload):
    return lib().cudadma_num_variants(workload)


def variant_name(workload, variant):
    return lib().cudadma_variant_name(workload, variant).decode()


def variants(workload):
    """The variant numbers of `workload` that the loaded library holds."""
    return [v for v in range(num_variants(workload)) if variant_name(workload, v)]


def transpose_splits():
    """The values of the knob "transpose_split" that the loaded library holds."""
    n = lib().cudadma_transpose_splits(None, 0)
    codes = (ctypes.c_int * n)()
    lib().cudadma_transpose_splits(codes, n)
    return sorted(codes)


def set_workgroups_per_cu(value):
    return lib().cudadma_set_workgroups_per_cu(int(value))


def set_tuning(name, value):
    rc = lib().cudadma_set_tuning(name.encode(), int(value))
    if rc < 0:
        check(rc)
    return rc


def fill_uniform(out, seed):
    _need(out, torch.float32, "out")
    check(lib().cudadma_fill_uniform(_p(out), out.numel(), seed, _stream()))
    return out


def fill_normal_bf16(out, seed):
    """out: bfloat16 tensor; receives normal(0,1) values from the seeded generator (the GEMM inputs of config 5)."""
    _need(out, torch.bfloat16, "out")
    check(lib().cudadma_fill_normal_bf16(_p(out), out.numel(), seed, _stream()))
    return out


def fill_indices(out, n_records, seed):
    _need(out, torch.int32, "out")
    check(lib().cudadma_fill_indices(_p(out), out.numel(), n_records, seed, _stream()))
    return out


def fill_permutation(out, seed):
    """out: int32 tensor of 2^k elements; receives a seeded permutation of [0, 2^k)."""
    _need(out, torch.int32, "out")
    n = out.numel()
    if n < 2 or n & (n - 1):
        raise ValueError("out must hold a power of two of elements, at least 2")
    check(lib().cudadma_fill_permutation(_p(out), n.bit_length() - 1, seed, _stream()))
    return out


def plain_copy(src, dst):
    check(lib().cudadma_plain_copy(_p(src), _p(dst), src.numel() * src.element_size(), _stream()))
    return dst


def sequential_copy(src, dst, variant=0):
    _need(src, torch.float32, "src")
    _need(dst, torch.float32, "dst")
    if dst.numel() != src.numel():
        raise ValueError("src and dst differ in size")
    check(lib().cudadma_sequential_copy(_p(src), _p(dst), src.numel() * 4, variant, _stream()))
    return dst


def strided_transpose(src, dst, variant=0):
    _need(src, torch.float32, "src")
    _need(dst, torch.float32, "dst")
    n = src.shape[0]
    if src.dim() != 2 or src.shape[1] != n or tuple(dst.shape) != (n, n):
        raise ValueError("src and dst must be n x n")
    check(lib().cudadma_strided_transpose(_p(src), _p(dst), n, variant, _stream()))
    return dst


def gather_copy(table, idx, out, variant=0):
    _need(table, torch.float32, "table")
    _need(idx, torch.int32, "idx")
    _need(out, torch.float32, "out")
    if out.numel() != idx.numel() * REC_FLOATS:
        raise ValueError("out must hold one record per index")
    check(lib().cudadma_gather_copy(_p(table), _p(idx), _p(out), table.numel() // REC_FLOATS, idx.numel(),
                                    variant, _stream()))
    return out


def gather_rowsum(table, idx, out, variant=0):
    _need(table, torch.float32, "table")
    _need(idx, torch.int32, "idx")
    _need(out, torch.float32, "out")
    if out.numel() != idx.numel() // RECS_PER_TILE * REC_FLOATS:
        raise ValueError("out must hold one record per tile of 32 indices")
    check(lib().cudadma_gather_rowsum(_p(table), _p(idx), _p(out), table.numel() // REC_FLOATS, idx.numel(),
                                      variant, _stream()))
    return out


def scatter_copy(records, idx, table, variant=0):
    """table[idx[i]] = records[i]; idx holds distinct record numbers of the table."""
    _need(records, torch.float32, "records")
    _need(idx, torch.int32, "idx")
    _need(table, torch.float32, "table")
    if records.numel() != idx.numel() * REC_FLOATS:
        raise ValueError("records must hold one record per index")
    check(lib().cudadma_scatter_copy(_p(records), _p(idx), _p(table), table.numel() // REC_FLOATS, idx.numel(),
                                     variant, _stream()))
    return table


def halo_stencil(grid_in, grid_out, variant=0):
    """grid_in: (nz+8, ny+8, nx+8) padded input, grid_out: (nz, ny, nx)."""
    _need(grid_in, torch.float32, "grid_in")
    _need(grid_out, torch.float32, "grid_out")
    nz, ny, nx = grid_out.shape
    p = 2 * STENCIL_RADIUS
    if tuple(grid_in.shape) != (nz + p, ny + p, nx + p):
        raise ValueError("grid_in must be the output shape plus 8 in every dimension")
    check(lib().cudadma_halo_stencil(_p(grid_in), _p(grid_out), nx, ny, nz, variant, _stream()))
    return grid_out


BUFFERING_NONE, BUFFERING_SINGLE, BUFFERING_DOUBLE, BUFFERING_MANUAL = range(4)
BUFFERING_NAMES = ("none", "single", "double", "manual")


LOAD_CACHE_ALL, LOAD_CACHE_STREAMING = 0, 2                 # CUDADMA_LOAD_CACHE_* of the C header
STORE_WRITE_BACK, STORE_LDS, STORE_LDS_DIRECT = 0, 4, 5     # CUDADMA_STORE_*


def perf_sequential(src, elmt_bytes, dma_wavefronts, buffering, loop_iters, workgroups, sums=None,
                    load_qualifier=LOAD_CACHE_ALL, store_qualifier=STORE_WRITE_BACK):
    """The read-bandwidth probe of the sequential object (all parameters at run time).  Returns the
    bytes one launch reads.  `sums` (uint32/int32, one zeroed word per workgroup) switches the checksum on.
    The qualifiers are those of the objects' fully qualified calls; the defaults are the reference's."""
    if not (src.is_cuda and src.is_contiguous()):
        raise ValueError("src must be a contiguous CUDA tensor")
    if sums is not None and not (sums.is_cuda and sums.is_contiguous() and sums.element_size() == 4 and sums.numel() >= workgroups):
        raise ValueError("sums must hold one 32-bit word per workgroup")
    n = lib().cudadma_perf_sequential(_p(src), src.numel() * src.element_size(), _p(sums) if sums is not None else None,
                                      elmt_bytes, dma_wavefronts, buffering, loop_iters, workgroups,
                                      load_qualifier, store_qualifier, _stream())
    if n < 0:
        check(int(n))
    return int(n)


PROBE_MODES = ("read", "write", "write_nontemporal", "copy", "copy_nontemporal", "vendor_copy", "read_nontemporal")


def probe_memory(mode, src, dst, workgroups):
    """One launch of a streaming yardstick (mode: index into PROBE_MODES or its name; "vendor_copy" is
    hipMemcpyDtoDAsync and ignores `workgroups`).  src / dst are CUDA tensors of the same size in bytes (None
    where the mode does not use one).  Returns bytes read + bytes written."""
    if isinstance(mode, str):
        mode = PROBE_MODES.index(mode)
    t = src if src is not None else dst
    nbytes = t.numel() * t.element_size()
    if src is not None and dst is not None and dst.numel() * dst.element_size() != nbytes:
        raise ValueError("src and dst differ in size")
    n = lib().cudadma_probe_memory(mode, _p(src) if src is not None else None, _p(dst) if dst is not None else None,
                                   nbytes, int(workgroups), _stream())
    if n < 0:
        check(int(n))
    return int(n)


def probe_clock(ticks, iterations=1 << 16):
    """One launch of the clock probe; `ticks`: int64 CUDA tensor of two elements (shader-clock ticks, 100 MHz ticks)."""
    _need(ticks, torch.int64, "ticks")
    check(lib().cudadma_probe_clock(_p(ticks), int(iterations), _stream()))
    return ticks


PATTERN_PROBE_MODES = ("gather_xor", "scatter", "tile_read", "tile_write", "tile_copy", "masked_read")


def probe_pattern(mode, src, idx, out, workgroups, n_records=0):
    """One launch of a yardstick with a pattern's own addresses (mode: index into PATTERN_PROBE_MODES or its name).
    gather_xor: src = table, idx = int32 indices, out = one 128-byte row per 32 indices; scatter: src = records,
    idx = int32 indices, out = table of n_records records; tile_read: src = n x n float matrix, out = 16 bytes per
    workgroup; tile_write: out = n x n matrix; tile_copy: src and out n x n matrices; masked_read: src = buffer of a power of
    two of bytes, n_records = the bit mask over the index of its 256-byte granules, out = 16 bytes per workgroup.  Returns the
    algorithmic bytes moved."""
    if isinstance(mode, str):
        mode = PATTERN_PROBE_MODES.index(mode)
    if mode in (0, 1):
        _need(idx, torch.int32, "idx")
        n = idx.numel()
        if not n_records:
            n_records = (src if mode == 0 else out).numel() * (src if mode == 0 else out).element_size() // 128
    elif mode == 5:
        n = src.numel() * src.element_size()
    else:
        n = (src if mode in (2, 4) else out).shape[0]
    moved = lib().cudadma_probe_pattern(mode, _p(src) if src is not None else None, _p(idx) if idx is not None else None,
                                        _p(out), n, n_records, int(workgroups), _stream())
    if moved < 0:
        check(int(moved))
    return int(moved)


def gemm_bf16(a, b, c, variant=0):
    """a: (m, k) and b: (k, n) torch.bfloat16, c: (m, n) float32; returns c = a @ b with fp32 accumulation."""
    _need(a, torch.bfloat16, "a")
    _need(b, torch.bfloat16, "b")
    _need(c, torch.float32, "c")
    m, k = a.shape
    k2, n = b.shape
    if k2 != k or tuple(c.shape) != (m, n):
        raise ValueError("shapes do not agree")
    check(lib().cudadma_gemm_bf16(_p(a), _p(b), _p(c), m, n, k, variant, _stream()))
    return c
