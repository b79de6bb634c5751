// The older class names of include/cudaDMA.h on top of the current objects.
//
// The first-generation interface has no BYTES_PER_THREAD parameter: every thread
// keeps four loads in flight (include/cudaDMA.h:30-31), which is what
// BYTES_PER_THREAD = 4*ALIGNMENT says in the current one.  Template parameters
// that are 0 are supplied through the constructor, in the same argument order
// as the current classes:
//
//   cudaDMASequential<DO_SYNC,ALIGNMENT,BYTES_PER_ELMT,DMA_THREADS>            include/cudaDMA.h:644-1166
//   cudaDMAStrided<DO_SYNC,ALIGNMENT,BYTES_PER_ELMT,DMA_THREADS,NUM_ELMTS>     include/cudaDMA.h:1977-2700
//   cudaDMAIndirect<GATHER,DO_SYNC,ALIGNMENT,BYTES_PER_ELMT,DMA_THREADS,NUM_ELMTS>  include/cudaDMA.h:2891-3580
//
// cudaDMAHalo and cudaDMACustom live next to the objects they wrap.
#pragma once

#include <type_traits>

#include "base.hpp"
#include "sequential.hpp"
#include "strided.hpp"
#include "indirect.hpp"

// Base class under its older name (include/cudaDMA.h:50).
typedef CudaDMA cudaDMA;

template<bool DO_SYNC, int ALIGNMENT, int BYTES_PER_ELMT = 0, int DMA_THREADS = 0>
class cudaDMASequential
  : public CudaDMASequential<DO_SYNC, ALIGNMENT, 4 * ALIGNMENT, BYTES_PER_ELMT, DMA_THREADS> {
  typedef CudaDMASequential<DO_SYNC, ALIGNMENT, 4 * ALIGNMENT, BYTES_PER_ELMT, DMA_THREADS> base_t;
public:
  using base_t::base_t;
  // The form that is not warp-specialised is built without arguments when its
  // size is a template parameter (include/cudaDMA.h:860, 1097).
  __device__ __forceinline__ cudaDMASequential() : base_t() {}
};

// With one stride argument the first-generation class strides the source only and packs
// the destination at BYTES_PER_ELMT (SINGLE_STRIDED_BASE, include/cudaDMA.h:1811-1840),
// where the current class applies the one stride to both sides; the constructors below
// spell the packed destination out.
template<bool DO_SYNC, int ALIGNMENT, int BYTES_PER_ELMT = 0, int DMA_THREADS = 0, int NUM_ELMTS = 0>
class cudaDMAStrided
  : public CudaDMAStrided<DO_SYNC, ALIGNMENT, 4 * ALIGNMENT, BYTES_PER_ELMT, DMA_THREADS, NUM_ELMTS> {
  typedef CudaDMAStrided<DO_SYNC, ALIGNMENT, 4 * ALIGNMENT, BYTES_PER_ELMT, DMA_THREADS, NUM_ELMTS> base_t;
  static constexpr int LEVEL = (BYTES_PER_ELMT == 0) ? 1 : (DMA_THREADS == 0) ? 2 : (NUM_ELMTS == 0) ? 3 : 4;
  template<bool C> using when = typename std::enable_if<C, int>::type;
public:
  // ---- warp-specialised ----
  // everything at run time (include/cudaDMA.h:2238-2270)
  template<int L = LEVEL, bool S = DO_SYNC, when<(L == 1) && S> = 0>
  __device__ __forceinline__ cudaDMAStrided(const int dmaID, const int num_dma_threads, const int num_compute_threads,
                                            const int dma_threadIdx_start, const int elmt_size_in_bytes,
                                            const int num_elmts, const int el_stride)
    : base_t(dmaID, num_dma_threads, num_compute_threads, dma_threadIdx_start, elmt_size_in_bytes, num_elmts,
             el_stride, elmt_size_in_bytes) {}
  template<int L = LEVEL, bool S = DO_SYNC, when<(L == 1) && S> = 0>
  __device__ __forceinline__ cudaDMAStrided(const int dmaID, const int num_dma_threads, const int num_compute_threads,
                                            const int dma_threadIdx_start, const int elmt_size_in_bytes,
                                            const int num_elmts, const int src_stride, const int dst_stride)
    : base_t(dmaID, num_dma_threads, num_compute_threads, dma_threadIdx_start, elmt_size_in_bytes, num_elmts,
             src_stride, dst_stride) {}
  // element size static (include/cudaDMA.h:2410-2436)
  template<int L = LEVEL, bool S = DO_SYNC, when<(L == 2) && S> = 0>
  __device__ __forceinline__ cudaDMAStrided(const int dmaID, const int num_dma_threads, const int num_compute_threads,
                                            const int dma_threadIdx_start, const int num_elmts, const int el_stride)
    : base_t(dmaID, num_dma_threads, num_compute_threads, dma_threadIdx_start, num_elmts, el_stride, BYTES_PER_ELMT) {}
  template<int L = LEVEL, bool S = DO_SYNC, when<(L == 2) && S> = 0>
  __device__ __forceinline__ cudaDMAStrided(const int dmaID, const int num_dma_threads, const int num_compute_threads,
                                            const int dma_threadIdx_start, const int num_elmts, const int src_stride,
                                            const int dst_stride)
    : base_t(dmaID, num_dma_threads, num_compute_threads, dma_threadIdx_start, num_elmts, src_stride, dst_stride) {}
  // element size and thread count static (include/cudaDMA.h:2566-2590)
  template<int L = LEVEL, bool S = DO_SYNC, when<(L == 3) && S> = 0>
  __device__ __forceinline__ cudaDMAStrided(const int dmaID, const int num_compute_threads, const int dma_threadIdx_start,
                                            const int num_elmts, const int el_stride)
    : base_t(dmaID, num_compute_threads, dma_threadIdx_start, num_elmts, el_stride, BYTES_PER_ELMT) {}
  template<int L = LEVEL, bool S = DO_SYNC, when<(L == 3) && S> = 0>
  __device__ __forceinline__ cudaDMAStrided(const int dmaID, const int num_compute_threads, const int dma_threadIdx_start,
                                            const int num_elmts, const int src_stride, const int dst_stride)
    : base_t(dmaID, num_compute_threads, dma_threadIdx_start, num_elmts, src_stride, dst_stride) {}
  // everything static (include/cudaDMA.h:1982-2000)
  template<int L = LEVEL, bool S = DO_SYNC, when<(L == 4) && S> = 0>
  __device__ __forceinline__ cudaDMAStrided(const int dmaID, const int num_compute_threads, const int dma_threadIdx_start,
                                            const int el_stride)
    : base_t(dmaID, num_compute_threads, dma_threadIdx_start, el_stride, BYTES_PER_ELMT) {}
  template<int L = LEVEL, bool S = DO_SYNC, when<(L == 4) && S> = 0>
  __device__ __forceinline__ cudaDMAStrided(const int dmaID, const int num_compute_threads, const int dma_threadIdx_start,
                                            const int src_stride, const int dst_stride)
    : base_t(dmaID, num_compute_threads, dma_threadIdx_start, src_stride, dst_stride) {}

  // ---- all threads of the block transfer (include/cudaDMA.h:2171-2180, 2329-2350, 2492-2510, 2645-2660) ----
  template<int L = LEVEL, bool S = DO_SYNC, when<(L == 1) && !S> = 0>
  __device__ __forceinline__ cudaDMAStrided(const int elmt_size_in_bytes, const int num_elmts, const int el_stride)
    : base_t(elmt_size_in_bytes, num_elmts, el_stride, elmt_size_in_bytes) {}
  template<int L = LEVEL, bool S = DO_SYNC, when<(L == 1) && !S> = 0>
  __device__ __forceinline__ cudaDMAStrided(const int elmt_size_in_bytes, const int num_elmts, const int src_stride,
                                            const int dst_stride)
    : base_t(elmt_size_in_bytes, num_elmts, src_stride, dst_stride) {}
  template<int L = LEVEL, bool S = DO_SYNC, when<(L == 2 || L == 3) && !S> = 0>
  __device__ __forceinline__ cudaDMAStrided(const int num_elmts, const int el_stride)
    : base_t(num_elmts, el_stride, BYTES_PER_ELMT) {}
  template<int L = LEVEL, bool S = DO_SYNC, when<(L == 2 || L == 3) && !S> = 0>
  __device__ __forceinline__ cudaDMAStrided(const int num_elmts, const int src_stride, const int dst_stride)
    : base_t(num_elmts, src_stride, dst_stride) {}
  template<int L = LEVEL, bool S = DO_SYNC, when<(L == 4) && !S> = 0>
  __device__ __forceinline__ cudaDMAStrided(const int el_stride)
    : base_t(el_stride, BYTES_PER_ELMT) {}
  template<int L = LEVEL, bool S = DO_SYNC, when<(L == 4) && !S> = 0>
  __device__ __forceinline__ cudaDMAStrided(const int src_stride, const int dst_stride)
    : base_t(src_stride, dst_stride) {}
};

template<bool GATHER, bool DO_SYNC, int ALIGNMENT, int BYTES_PER_ELMT = 0, int DMA_THREADS = 0, int NUM_ELMTS = 0>
class cudaDMAIndirect
  : public CudaDMAIndirect<GATHER, DO_SYNC, ALIGNMENT, 4 * ALIGNMENT, BYTES_PER_ELMT, DMA_THREADS, NUM_ELMTS> {
  typedef CudaDMAIndirect<GATHER, DO_SYNC, ALIGNMENT, 4 * ALIGNMENT, BYTES_PER_ELMT, DMA_THREADS, NUM_ELMTS> base_t;
public:
  using base_t::base_t;
  // Fully templated and not warp-specialised: no constructor arguments (include/cudaDMA.h:3098).
  __device__ __forceinline__ cudaDMAIndirect() : base_t() {}
};
