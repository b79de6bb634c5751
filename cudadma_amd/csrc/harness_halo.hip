// Known-answer cases for CudaDMAHalo and the older cudaDMAHalo interface
// (counterpart of src/tests/test_halo/cudaDMA_test_halo.cu).  Origins point at
// the first interior cell: source RADIUS rows and RADIUS cells into the padded
// input, destination likewise into the (dimx+2R) x (dimy+2R) LDS tile.
#include "harness.hpp"

namespace {
using harness::Args;
using harness::kComputeThreads;

template<int ES> struct cell_of;
template<> struct cell_of<4>  { typedef float type; };
template<> struct cell_of<8>  { typedef float2 type; };
template<> struct cell_of<16> { typedef float4 type; };

// LEVEL 0 is the older class cudaDMAHalo<ELMT_TYPE,RADIUS,CORNERS,ALIGNMENT>.
template<bool WS, int LEVEL, int A, int BPT, int ES, int T, int R, bool C, int DX, int DY> struct Make;
template<int A, int BPT, int ES, int T, int R, bool C, int DX, int DY> struct Make<true, 0, A, BPT, ES, T, R, C, DX, DY> {
  typedef cudaDMAHalo<typename cell_of<ES>::type, R, C, A> type;
  static __device__ __forceinline__ type make(const Args& a)
  { return type(1, a.dma_threads, kComputeThreads, kComputeThreads, a.dimx, a.dimy, a.pitch); }
};
template<int A, int BPT, int ES, int T, int R, bool C, int DX, int DY> struct Make<true, 1, A, BPT, ES, T, R, C, DX, DY> {
  typedef CudaDMAHalo<true, A, BPT, ES, 0, R, C> type;
  static __device__ __forceinline__ type make(const Args& a)
  { return type(1, a.dma_threads, kComputeThreads, kComputeThreads, a.dimx, a.dimy, a.pitch, a.dst_pitch); }
};
template<int A, int BPT, int ES, int T, int R, bool C, int DX, int DY> struct Make<true, 2, A, BPT, ES, T, R, C, DX, DY> {
  typedef CudaDMAHalo<true, A, BPT, ES, T, R, C> type;
  static __device__ __forceinline__ type make(const Args& a)
  { return type(2, kComputeThreads, kComputeThreads, a.dimx, a.dimy, a.pitch, a.dst_pitch); }
};
template<int A, int BPT, int ES, int T, int R, bool C, int DX, int DY> struct Make<true, 3, A, BPT, ES, T, R, C, DX, DY> {
  typedef CudaDMAHalo<true, A, BPT, ES, T, R, C, DX, DY> type;
  static __device__ __forceinline__ type make(const Args& a)
  { return type(3, kComputeThreads, kComputeThreads, a.pitch, a.dst_pitch); }
};
template<int A, int BPT, int ES, int T, int R, bool C, int DX, int DY> struct Make<false, 1, A, BPT, ES, T, R, C, DX, DY> {
  typedef CudaDMAHalo<false, A, BPT, ES, 0, R, C> type;
  static __device__ __forceinline__ type make(const Args& a) { return type(a.dimx, a.dimy, a.pitch, 0, 0, a.dst_pitch); }
};
template<int A, int BPT, int ES, int T, int R, bool C, int DX, int DY> struct Make<false, 2, A, BPT, ES, T, R, C, DX, DY> {
  typedef CudaDMAHalo<false, A, BPT, ES, T, R, C> type;
  static __device__ __forceinline__ type make(const Args& a) { return type(a.dimx, a.dimy, a.pitch, 0, a.dst_pitch); }
};
template<int A, int BPT, int ES, int T, int R, bool C, int DX, int DY> struct Make<false, 3, A, BPT, ES, T, R, C, DX, DY> {
  typedef CudaDMAHalo<false, A, BPT, ES, T, R, C, DX, DY> type;
  static __device__ __forceinline__ type make(const Args& a) { return type(a.pitch, 0, a.dst_pitch); }
};

template<bool WS, int LEVEL, int A, int BPT, int ES, int T, int R, bool C, int DX, int DY, bool MATRIX>
__global__ void __launch_bounds__(1024) halo_kernel(const Args a)
{
  extern __shared__ __attribute__((aligned(16))) unsigned lds[];
  auto dma = Make<WS, LEVEL, A, BPT, ES, T, R, C, DX, DY>::make(a);
  harness::run_body<WS>(dma, a, lds, [&](const int rep) __attribute__((always_inline)) {
    const char* src = (a.reverse ? (const char*)lds + a.src_offset : a.in + a.src_offset + (size_t)rep * a.rep_src_bytes) +
                      (size_t)(R * a.pitch + R) * ES;
    const int dst_pitch = a.dst_pitch > 0 ? a.dst_pitch : a.dimx + 2 * R;
    char* dst = (a.reverse ? a.out + (size_t)rep * a.out_bytes + a.dst_offset : (char*)lds + a.dst_offset) +
                (size_t)(R * dst_pitch + R) * ES;
    if constexpr (MATRIX) harness::do_transfer_matrix<false>(dma, a.call_style, a.two_phase, src, dst);
    else harness::do_transfer(dma, a.call_style, a.two_phase, src, dst);
  });
}

template<bool WS, int LEVEL, int A, int BPT, int ES, int T, int R, bool C, int DX, int DY>
int launch(const Args& a, hipStream_t s)
{ return harness::launch_case(halo_kernel<WS, LEVEL, A, BPT, ES, T, R, C, DX, DY, false>, halo_kernel<WS, LEVEL, A, BPT, ES, T, R, C, DX, DY, true>, WS, a, s); }

#define HALO_CASE(ORDER, WS, LEVEL, A, BPT, ES, T, R, C, DX, DY)                                          \
  static harness::Registrar reg_halo_##ORDER(                                                              \
      cudadma_case_t{CUDADMA_PATTERN_HALO, WS, LEVEL, A, BPT, ES, T, 0, R, C, DX, DY},                     \
      launch<WS, LEVEL, A, BPT, ES, T, R, bool(C), DX, DY>, ORDER);
#include "cases_halo.inc"
#undef HALO_CASE
}  // namespace
