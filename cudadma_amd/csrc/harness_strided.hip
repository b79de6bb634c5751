// Known-answer cases for CudaDMAStrided
// (counterpart of src/tests/test_strided/cudaDMA_test_strided_v2.cu).
#include "harness.hpp"

namespace {
using harness::Args;
using harness::kComputeThreads;

// ONE_STRIDE picks the constructor that takes one elmt_stride for both sides
// (the host then has to pass src_stride == dst_stride); otherwise the
// constructor with separate source and destination strides is used.
template<bool WS, int LEVEL, bool ONE_STRIDE, int A, int BPT, int E, int T, int N> struct Make;
template<bool ONE, int A, int BPT, int E, int T, int N> struct Make<true, 1, ONE, A, BPT, E, T, N> {
  typedef CudaDMAStrided<true, A, BPT> type;
  static __device__ __forceinline__ type make(const Args& a)
  {
    if constexpr (ONE) return type(1, a.dma_threads, kComputeThreads, kComputeThreads, a.bytes_per_elmt, a.num_elmts, a.src_stride);
    else return type(1, a.dma_threads, kComputeThreads, kComputeThreads, a.bytes_per_elmt, a.num_elmts, a.src_stride, a.dst_stride);
  }
};
template<bool ONE, int A, int BPT, int E, int T, int N> struct Make<true, 2, ONE, A, BPT, E, T, N> {
  typedef CudaDMAStrided<true, A, BPT, E> type;
  static __device__ __forceinline__ type make(const Args& a)
  {
    if constexpr (ONE) return type(2, a.dma_threads, kComputeThreads, kComputeThreads, a.num_elmts, a.src_stride);
    else return type(2, a.dma_threads, kComputeThreads, kComputeThreads, a.num_elmts, a.src_stride, a.dst_stride);
  }
};
template<bool ONE, int A, int BPT, int E, int T, int N> struct Make<true, 3, ONE, A, BPT, E, T, N> {
  typedef CudaDMAStrided<true, A, BPT, E, T> type;
  static __device__ __forceinline__ type make(const Args& a)
  {
    if constexpr (ONE) return type(3, kComputeThreads, kComputeThreads, a.num_elmts, a.src_stride);
    else return type(3, kComputeThreads, kComputeThreads, a.num_elmts, a.src_stride, a.dst_stride);
  }
};
template<bool ONE, int A, int BPT, int E, int T, int N> struct Make<true, 4, ONE, A, BPT, E, T, N> {
  typedef CudaDMAStrided<true, A, BPT, E, T, N> type;
  static __device__ __forceinline__ type make(const Args& a)
  {
    if constexpr (ONE) return type(4, kComputeThreads, kComputeThreads, a.src_stride);
    else return type(4, kComputeThreads, kComputeThreads, a.src_stride, a.dst_stride);
  }
};
template<bool ONE, int A, int BPT, int E, int T, int N> struct Make<false, 1, ONE, A, BPT, E, T, N> {
  typedef CudaDMAStrided<false, A, BPT> type;
  static __device__ __forceinline__ type make(const Args& a)
  {
    if constexpr (ONE) return type(a.bytes_per_elmt, a.num_elmts, a.src_stride);
    else return type(a.bytes_per_elmt, a.num_elmts, a.src_stride, a.dst_stride, a.dma_threads);
  }
};
template<bool ONE, int A, int BPT, int E, int T, int N> struct Make<false, 2, ONE, A, BPT, E, T, N> {
  typedef CudaDMAStrided<false, A, BPT, E> type;
  static __device__ __forceinline__ type make(const Args& a)
  {
    if constexpr (ONE) return type(a.num_elmts, a.src_stride);
    else return type(a.num_elmts, a.src_stride, a.dst_stride);
  }
};
template<bool ONE, int A, int BPT, int E, int T, int N> struct Make<false, 3, ONE, A, BPT, E, T, N> {
  typedef CudaDMAStrided<false, A, BPT, E, T> type;
  static __device__ __forceinline__ type make(const Args& a)
  {
    if constexpr (ONE) return type(a.num_elmts, a.src_stride);
    else return type(a.num_elmts, a.src_stride, a.dst_stride);
  }
};
template<bool ONE, int A, int BPT, int E, int T, int N> struct Make<false, 4, ONE, A, BPT, E, T, N> {
  typedef CudaDMAStrided<false, A, BPT, E, T, N> type;
  static __device__ __forceinline__ type make(const Args& a)
  {
    if constexpr (ONE) return type(a.src_stride);
    else return type(a.src_stride, a.dst_stride);
  }
};

// The direct qualifiers.  With two_phase set and a shape the direct path takes, the transfer goes
// through issue_direct() + wait_direct_loads<0>() with the hand-off done by hand around them
// (the form a kernel uses to keep several direct transfers in flight); otherwise through the
// ordinary calls, which fall back to registers when the shape does not fit.
// Every other repetition issues the transfer in two parts (its first load, then the rest) through
// issue_direct_part().
template<bool WS, int SQ, typename Obj>
__device__ __forceinline__ void direct_transfer(Obj& dma, const int two_phase, const void* src, void* dst, const int rep)
{
  if (two_phase && dma.direct_ready()) {
    if constexpr (WS) dma.wait_for_dma_start();
    if (rep & 1) {
      dma.template issue_direct_part<SQ>(src, dst, 0, 1);
      dma.template issue_direct_part<SQ>(src, dst, 1, 0x3fffffff);
    } else {
      dma.template issue_direct<SQ>(src, dst);
    }
    hipdma::wait_direct_loads<0>();
    if constexpr (WS) dma.finish_async_dma();
  } else {
    harness::do_transfer_direct<SQ>(dma, two_phase, src, dst);
  }
}

template<bool WS, int LEVEL, bool ONE, int A, int BPT, int E, int T, int N, bool MATRIX>
__global__ void __launch_bounds__(1024) strided_kernel(const Args a)
{
  extern __shared__ __attribute__((aligned(16))) unsigned lds[];
  auto dma = Make<WS, LEVEL, ONE, A, BPT, E, T, N>::make(a);
  // swizzled rows are whole chunks: known here when the element size is a template parameter,
  // checked by the host for the level that takes it at run time
  constexpr bool kWholeChunks = (LEVEL == 1) || (E % A) == 0;
  harness::run_body<WS>(dma, a, lds, [&](const int rep) __attribute__((always_inline)) {
    const char* src = a.reverse ? (const char*)lds + a.src_offset : a.in + a.src_offset + (size_t)rep * a.rep_src_bytes;
    char* dst = a.reverse ? a.out + (size_t)rep * a.out_bytes + a.dst_offset : (char*)lds + a.dst_offset;
    if constexpr (MATRIX) {
      harness::do_transfer_matrix<(A == 16 || A == 4)>(dma, a.call_style, a.two_phase, src, dst);
    } else if (a.call_style == CUDADMA_CALL_LDS_DIRECT) {
      if constexpr (A == 16 || A == 4) direct_transfer<WS, STORE_LDS_DIRECT>(dma, a.two_phase, src, dst, rep);
    } else if (a.call_style == CUDADMA_CALL_LDS_SWIZZLE) {
      if constexpr (kWholeChunks) harness::do_transfer_direct<STORE_LDS_SWIZZLE>(dma, a.two_phase, src, dst);
    } else if (a.call_style == CUDADMA_CALL_LDS_DIRECT_SWIZZLE) {
      if constexpr ((A == 16 || A == 4) && kWholeChunks)
        direct_transfer<WS, STORE_LDS_DIRECT_SWIZZLE>(dma, a.two_phase, src, dst, rep);
    } else {
      harness::do_transfer(dma, a.call_style, a.two_phase, src, dst);
    }
  });
}

template<bool WS, int LEVEL, bool ONE, int A, int BPT, int E, int T, int N>
int launch(const Args& a, hipStream_t s)
{
  if (ONE && a.src_stride != a.dst_stride) {
    cudadma_host::set_error("this case was built with the single-stride constructor: src_stride must equal dst_stride");
    return CUDADMA_EINVAL;
  }
  return harness::launch_case(strided_kernel<WS, LEVEL, ONE, A, BPT, E, T, N, false>, strided_kernel<WS, LEVEL, ONE, A, BPT, E, T, N, true>, WS, a, s);
}

// dimx carries the ONE_STRIDE flag in the case description.
#define STRIDED_CASE(ORDER, WS, LEVEL, ONE, A, BPT, E, T, N)                                             \
  static harness::Registrar reg_strided_##ORDER(                                                          \
      cudadma_case_t{CUDADMA_PATTERN_STRIDED, WS, LEVEL, A, BPT, E, T, N, 0, 0, ONE, 0},                  \
      launch<WS, LEVEL, ONE, A, BPT, E, T, N>, ORDER);
#include "cases_strided.inc"
#undef STRIDED_CASE
}  // namespace
