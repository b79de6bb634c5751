"""Host-side planner: replay of the thread -> byte assignment and diagnose() reports.  Needs no GPU."""
import ctypes

import numpy as np

from ._lib import PlanQuery, check, lib


def plan_map(pattern, *, alignment, bytes_per_thread, bytes_per_elmt, dma_threads, num_elmts=0, src_stride=0,
             dst_stride=0, radius=0, corners=0, dimx=0, dimy=0, pitch=0, dst_pitch=0, index=None, src_origin=0,
             dst_origin=0, map_len):
    """Returns (map, steps, double_writes): map[d] = source byte landing on destination byte d, -1 if untouched."""
    idx = None
    if index is not None:
        idx = np.ascontiguousarray(index, dtype=np.int32)
    q = PlanQuery(pattern=pattern, alignment=alignment, bytes_per_thread=bytes_per_thread,
                  bytes_per_elmt=bytes_per_elmt, dma_threads=dma_threads, num_elmts=num_elmts,
                  src_stride=src_stride, dst_stride=dst_stride, radius=radius, corners=int(corners), dimx=dimx,
                  dimy=dimy, pitch=pitch, index=(idx.ctypes.data if idx is not None else 0), dst_pitch=dst_pitch)
    out = np.empty(map_len, dtype=np.int32)
    steps = ctypes.c_int(0)
    rc = lib().cudadma_plan_map(ctypes.byref(q), src_origin, dst_origin, ctypes.c_void_p(out.ctypes.data), map_len,
                                ctypes.byref(steps))
    if rc < 0:
        check(rc)
    return out, steps.value, rc


def plan_extents(pattern, *, alignment, bytes_per_thread, bytes_per_elmt, dma_threads, num_elmts=0, src_stride=0,
                 dst_stride=0, radius=0, corners=0, dimx=0, dimy=0, pitch=0, dst_pitch=0, index=None):
    """(src_min, src_end, dst_min, dst_end): byte offsets relative to the transfer's pointers that any DMA
    thread reads / writes."""
    idx = np.ascontiguousarray(index, dtype=np.int32) if index is not None else None
    q = PlanQuery(pattern=pattern, alignment=alignment, bytes_per_thread=bytes_per_thread,
                  bytes_per_elmt=bytes_per_elmt, dma_threads=dma_threads, num_elmts=num_elmts,
                  src_stride=src_stride, dst_stride=dst_stride, radius=radius, corners=int(corners), dimx=dimx,
                  dimy=dimy, pitch=pitch, index=(idx.ctypes.data if idx is not None else 0), dst_pitch=dst_pitch)
    ext = (ctypes.c_longlong * 4)()
    check(lib().cudadma_plan_extents(ctypes.byref(q), ctypes.byref(ext)))
    return tuple(ext)


def diagnose(pattern, alignment, bytes_per_thread, bytes_per_elmt, dma_threads, num_elmts=0, full_template=True,
             verbose=False):
    check(lib().cudadma_diagnose(pattern, alignment, bytes_per_thread, bytes_per_elmt, dma_threads, num_elmts,
                                 int(full_template), int(verbose)))
