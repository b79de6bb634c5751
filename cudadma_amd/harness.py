"""Python face of the known-answer harness (cudadma_num_cases / cudadma_get_case /
cudadma_run_case).  Device memory comes from the caller as torch tensors."""
import ctypes

from . import _lib
from ._lib import Case, RunArgs, check
from ._lib import harness_lib as lib


def num_cases():
    return lib().cudadma_num_cases()


def get_case(case_id):
    c = Case()
    check(lib().cudadma_get_case(case_id, ctypes.byref(c)))
    return c


def all_cases():
    return [get_case(i) for i in range(num_cases())]


def _ptr(t):
    return ctypes.c_void_p(t.data_ptr()) if t is not None else ctypes.c_void_p(0)


def run_case(case_id, d_in, d_out, *, lds_bytes, d_index=None, src_offset_bytes=0, dst_offset_bytes=0,
             src_stride=0, dst_stride=0, pitch=0, call_style=_lib.CALL_UNQUALIFIED, two_phase=False, reps=1,
             rep_src_bytes=0, rep_index_elmts=0, reverse=False, out_bytes=0, stream=None,
             bytes_per_elmt=0, dma_threads=0, num_elmts=0, dimx=0, dimy=0, dst_pitch=0,
             in_bytes=None, out_capacity=None, index_elmts=None):
    """Launch one case.  d_in / d_out / d_index are torch CUDA tensors; d_out must
    hold reps * lds_bytes bytes.  bytes_per_elmt, dma_threads, num_elmts, dimx and dimy (0 = the
    case's own) replace the parameters the case's level passes to its constructor at run time; dst_pitch
    (halo, cells, 0 = dimx + 2*radius) is the destination row pitch.  in_bytes, out_capacity and index_elmts
    default to the sizes of the tensors: the library replays the transfer on the host and refuses one that
    would leave them.  Raises CudaDMAError when the library rejects the arguments."""
    need = reps * (out_bytes if reverse else lds_bytes)
    if d_out.numel() * d_out.element_size() < need:
        raise ValueError("d_out is smaller than reps * (out_bytes if reverse else lds_bytes)")
    r = RunArgs(
        d_in=d_in.data_ptr(), d_out=d_out.data_ptr(), d_index=(d_index.data_ptr() if d_index is not None else 0),
        lds_bytes=lds_bytes, src_offset_bytes=src_offset_bytes, dst_offset_bytes=dst_offset_bytes,
        src_stride=src_stride, dst_stride=dst_stride, pitch=pitch, call_style=call_style,
        two_phase=int(bool(two_phase)), reps=reps, rep_src_bytes=rep_src_bytes, rep_index_elmts=rep_index_elmts,
        reverse=int(bool(reverse)), out_bytes=out_bytes, rt_bytes_per_elmt=bytes_per_elmt,
        rt_dma_threads=dma_threads, rt_num_elmts=num_elmts, rt_dimx=dimx, rt_dimy=dimy, dst_pitch=dst_pitch,
        in_bytes=(d_in.numel() * d_in.element_size() if in_bytes is None else in_bytes),
        out_capacity=(d_out.numel() * d_out.element_size() if out_capacity is None else out_capacity),
        index_elmts=((d_index.numel() if d_index is not None else 0) if index_elmts is None else index_elmts))
    check(lib().cudadma_run_case(case_id, ctypes.byref(r), ctypes.c_void_p(stream or 0)))
