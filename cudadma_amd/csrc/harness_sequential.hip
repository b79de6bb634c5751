// Known-answer cases for CudaDMASequential
// (counterpart of src/tests/test_sequential/cudaDMA_test_sequential_v2.cu).
#include "harness.hpp"

namespace {
using harness::Args;
using harness::kComputeThreads;

template<bool WS, int LEVEL, int A, int BPT, int E, int T> struct Make;
template<int A, int BPT, int E, int T> struct Make<true, 1, A, BPT, E, T> {
  typedef CudaDMASequential<true, A, BPT> type;
  static __device__ __forceinline__ type make(const Args& a)
  { return type(1, a.dma_threads, kComputeThreads, kComputeThreads, a.bytes_per_elmt); }
};
template<int A, int BPT, int E, int T> struct Make<true, 2, A, BPT, E, T> {
  typedef CudaDMASequential<true, A, BPT, E> type;
  static __device__ __forceinline__ type make(const Args& a)
  { return type(2, a.dma_threads, kComputeThreads, kComputeThreads); }
};
template<int A, int BPT, int E, int T> struct Make<true, 3, A, BPT, E, T> {
  typedef CudaDMASequential<true, A, BPT, E, T> type;
  static __device__ __forceinline__ type make(const Args&) { return type(3, kComputeThreads, kComputeThreads); }
};
template<int A, int BPT, int E, int T> struct Make<false, 1, A, BPT, E, T> {
  typedef CudaDMASequential<false, A, BPT> type;
  static __device__ __forceinline__ type make(const Args& a) { return type(a.bytes_per_elmt, a.dma_threads); }
};
template<int A, int BPT, int E, int T> struct Make<false, 2, A, BPT, E, T> {
  typedef CudaDMASequential<false, A, BPT, E> type;
  static __device__ __forceinline__ type make(const Args&) { return type(); }   // thread count from blockDim.x
};
template<int A, int BPT, int E, int T> struct Make<false, 3, A, BPT, E, T> {
  typedef CudaDMASequential<false, A, BPT, E, T> type;
  static __device__ __forceinline__ type make(const Args&) { return type(); }
};

template<bool WS, int LEVEL, int A, int BPT, int E, int T, bool MATRIX>
__global__ void __launch_bounds__(1024) seq_kernel(const Args a)
{
  extern __shared__ __attribute__((aligned(16))) unsigned lds[];
  auto dma = Make<WS, LEVEL, A, BPT, E, T>::make(a);
  harness::run_body<WS>(dma, a, lds, [&](const int rep) __attribute__((always_inline)) {
    const char* src = a.reverse ? (const char*)lds + a.src_offset : a.in + a.src_offset + (size_t)rep * a.rep_src_bytes;
    char* dst = a.reverse ? a.out + (size_t)rep * a.out_bytes + a.dst_offset : (char*)lds + a.dst_offset;
    if constexpr (MATRIX) {
      harness::do_transfer_matrix<(A == 16 || A == 4)>(dma, a.call_style, a.two_phase, src, dst);
    } else if (a.call_style == CUDADMA_CALL_LDS_DIRECT) {
      if constexpr (A == 16 || A == 4) harness::do_transfer_direct(dma, a.two_phase, src, dst);
    } else {
      harness::do_transfer(dma, a.call_style, a.two_phase, src, dst);
    }
  });
}

template<bool WS, int LEVEL, int A, int BPT, int E, int T>
int launch(const Args& a, hipStream_t s)
{ return harness::launch_case(seq_kernel<WS, LEVEL, A, BPT, E, T, false>, seq_kernel<WS, LEVEL, A, BPT, E, T, true>, WS, a, s); }

#define SEQ_CASE(ORDER, WS, LEVEL, A, BPT, E, T)                                                         \
  static harness::Registrar reg_seq_##ORDER(                                                              \
      cudadma_case_t{CUDADMA_PATTERN_SEQUENTIAL, WS, LEVEL, A, BPT, E, T, 0, 0, 0, 0, 0},                 \
      launch<WS, LEVEL, A, BPT, E, T>, ORDER);
#include "cases_sequential.inc"
#undef SEQ_CASE
}  // namespace
