// Known-answer cases for CudaDMAIndirect, gather and scatter
// (counterpart of src/tests/test_indirect/cudaDMA_test_indirect_v2.cu, which
// only runs the gather direction).
#include "harness.hpp"

namespace {
using harness::Args;
using harness::kComputeThreads;

// The dense-side stride travels in dst_stride for a gather and in src_stride for a scatter.
template<bool GATHER> __device__ __forceinline__ int alt_stride(const Args& a) { return GATHER ? a.dst_stride : a.src_stride; }

template<bool G, bool WS, int LEVEL, int A, int BPT, int E, int T, int N> struct Make;
template<bool G, int A, int BPT, int E, int T, int N> struct Make<G, true, 1, A, BPT, E, T, N> {
  typedef CudaDMAIndirect<G, true, A, BPT> type;
  static __device__ __forceinline__ type make(const Args& a)
  { return type(1, a.dma_threads, kComputeThreads, kComputeThreads, a.bytes_per_elmt, a.num_elmts, alt_stride<G>(a)); }
};
template<bool G, int A, int BPT, int E, int T, int N> struct Make<G, true, 2, A, BPT, E, T, N> {
  typedef CudaDMAIndirect<G, true, A, BPT, E> type;
  static __device__ __forceinline__ type make(const Args& a)
  { return type(2, a.dma_threads, kComputeThreads, kComputeThreads, a.num_elmts, alt_stride<G>(a)); }
};
template<bool G, int A, int BPT, int E, int T, int N> struct Make<G, true, 3, A, BPT, E, T, N> {
  typedef CudaDMAIndirect<G, true, A, BPT, E, T> type;
  static __device__ __forceinline__ type make(const Args& a)
  { return type(3, kComputeThreads, kComputeThreads, a.num_elmts, alt_stride<G>(a)); }
};
template<bool G, int A, int BPT, int E, int T, int N> struct Make<G, true, 4, A, BPT, E, T, N> {
  typedef CudaDMAIndirect<G, true, A, BPT, E, T, N> type;
  static __device__ __forceinline__ type make(const Args& a)
  { return type(4, kComputeThreads, kComputeThreads, alt_stride<G>(a)); }
};
template<bool G, int A, int BPT, int E, int T, int N> struct Make<G, false, 1, A, BPT, E, T, N> {
  typedef CudaDMAIndirect<G, false, A, BPT> type;
  static __device__ __forceinline__ type make(const Args& a)
  { return type(a.bytes_per_elmt, a.num_elmts, alt_stride<G>(a), a.dma_threads); }
};
template<bool G, int A, int BPT, int E, int T, int N> struct Make<G, false, 2, A, BPT, E, T, N> {
  typedef CudaDMAIndirect<G, false, A, BPT, E> type;
  static __device__ __forceinline__ type make(const Args& a) { return type(a.num_elmts, alt_stride<G>(a)); }
};
template<bool G, int A, int BPT, int E, int T, int N> struct Make<G, false, 3, A, BPT, E, T, N> {
  typedef CudaDMAIndirect<G, false, A, BPT, E, T> type;
  static __device__ __forceinline__ type make(const Args& a) { return type(a.num_elmts, alt_stride<G>(a)); }
};
template<bool G, int A, int BPT, int E, int T, int N> struct Make<G, false, 4, A, BPT, E, T, N> {
  typedef CudaDMAIndirect<G, false, A, BPT, E, T, N> type;
  static __device__ __forceinline__ type make(const Args& a) { return type(alt_stride<G>(a)); }
};

template<bool G, bool WS, int LEVEL, int A, int BPT, int E, int T, int N, bool MATRIX>
__global__ void __launch_bounds__(1024) indirect_kernel(const Args a)
{
  extern __shared__ __attribute__((aligned(16))) unsigned lds[];
  auto dma = Make<G, WS, LEVEL, A, BPT, E, T, N>::make(a);
  harness::run_body<WS>(dma, a, lds, [&](const int rep) __attribute__((always_inline)) {
    const char* src = a.reverse ? (const char*)lds + a.src_offset : a.in + a.src_offset + (size_t)rep * a.rep_src_bytes;
    const int* index = a.index + (size_t)rep * a.rep_index_elmts;
    char* dst = a.reverse ? a.out + (size_t)rep * a.out_bytes + a.dst_offset : (char*)lds + a.dst_offset;
    if constexpr (MATRIX) {
      harness::do_transfer_indexed_matrix<(G && (A == 16 || A == 4))>(dma, a.call_style, a.two_phase, index, src, dst);
    } else if (a.call_style == CUDADMA_CALL_LDS_DIRECT) {
      if constexpr (G && (A == 16 || A == 4)) {
        if (a.two_phase) {
          dma.template start_xfer_async<true, LOAD_CACHE_ALL, STORE_LDS_DIRECT>(index, src);
          dma.template wait_xfer_finish<true, LOAD_CACHE_ALL, STORE_LDS_DIRECT>(dst);
        } else {
          dma.template execute_dma<true, LOAD_CACHE_ALL, STORE_LDS_DIRECT>(index, src, dst);
        }
      }
    } else if (a.call_style == CUDADMA_CALL_INDEX_AHEAD) {
      if (a.two_phase) {
        // as a multi-buffered kernel does it: the next repetition's index words are requested between the phases
        if (rep == 0) dma.template prefetch_index<true>(index);
        const int next = rep + 1 < a.reps ? rep + 1 : rep;
        dma.template start_xfer_async_prefetched<false, LOAD_CACHE_ALL, STORE_WRITE_BACK>(index, src);
        dma.template prefetch_index<true>(a.index + (size_t)next * a.rep_index_elmts);
        dma.template wait_xfer_finish<false, LOAD_CACHE_ALL, STORE_WRITE_BACK>(dst);
      } else {
        dma.template prefetch_index<true>(index);
        dma.template execute_dma_prefetched<false, LOAD_CACHE_ALL, STORE_WRITE_BACK>(index, src, dst);
      }
    } else {
      harness::do_transfer_indexed(dma, a.call_style, a.two_phase, index, src, dst);
    }
  });
}

template<bool G, bool WS, int LEVEL, int A, int BPT, int E, int T, int N>
int launch(const Args& a, hipStream_t s)
{ return harness::launch_case(indirect_kernel<G, WS, LEVEL, A, BPT, E, T, N, false>, indirect_kernel<G, WS, LEVEL, A, BPT, E, T, N, true>, WS, a, s); }

#define INDIRECT_CASE(ORDER, G, WS, LEVEL, A, BPT, E, T, N)                                              \
  static harness::Registrar reg_indirect_##ORDER(                                                         \
      cudadma_case_t{G ? CUDADMA_PATTERN_GATHER : CUDADMA_PATTERN_SCATTER, WS, LEVEL, A, BPT, E, T, N,    \
                     0, 0, 0, 0},                                                                         \
      launch<G, WS, LEVEL, A, BPT, E, T, N>, ORDER);
#include "cases_indirect.inc"
#undef INDIRECT_CASE
}  // namespace
