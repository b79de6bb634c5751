// CudaDMAIndirect: gather or scatter of NUM_ELMTS elements of BYTES_PER_ELMT bytes.
//   GATHER :  dst[i*S + j] = src[index[i]*BYTES_PER_ELMT + j]
//   SCATTER:  dst[index[i]*BYTES_PER_ELMT + j] = src[i*S + j]
// with S = max(alternate_stride, BYTES_PER_ELMT); index[] holds element
// numbers, not byte offsets.  The byte offset on the indexed side is formed in 64 bits, so the indexed buffer
// may be larger than 2 GiB (the reference forms it in int, include/cudaDMAv2.h:9940-9957).
//
// API contract: include/cudaDMAv2.h:9370-14728 (template parameters :9381-9382,
// dense-side stride :9406, call form :9700-9814, addressing :9940-9957 and
// :10199-10217; constructors :10225-10231, :10628-10632, :11431-11436,
// :11825-11828, :12710-12714, :13098-13100, :13983-13986, :14362-14363).
// The work split is the slot grid of grid.hpp; every lane fetches the index of
// the row it works on (lanes of one row read the same word, which the memory
// pipeline serves as one access), all indices of a step before its data loads.
//
// An addition without a counterpart in the reference: prefetch_index() asks for
// the index words of the first step of a later transfer and leaves them in
// flight; start_xfer_async_prefetched() / execute_dma_prefetched() then start
// that transfer from them.  A wavefront's loads return in issue order, so a
// transfer that fetches its index words itself has to wait for every load the
// thread still has in flight (the elements of other objects that share the DMA
// threads) before it can form its first address; with the words requested one
// transfer ahead, the wait covers only loads that are older than they are.
#pragma once

#include "grid.hpp"

template<bool GATHER = true, bool DO_SYNC = false, int ALIGNMENT = 0, int BYTES_PER_THREAD = 4 * ALIGNMENT,
         int BYTES_PER_ELMT = 0, int DMA_THREADS = 0, int NUM_ELMTS = 0>
class CudaDMAIndirect : public CudaDMA {
  static_assert(ALIGNMENT == 4 || ALIGNMENT == 8 || ALIGNMENT == 16, "ALIGNMENT must be 4, 8 or 16");
  static_assert((BYTES_PER_THREAD / ALIGNMENT) > 0, "BYTES_PER_THREAD must hold at least one chunk");
  static_assert((BYTES_PER_THREAD % ALIGNMENT) == 0, "BYTES_PER_THREAD must be a multiple of ALIGNMENT");
  static_assert((BYTES_PER_ELMT % 4) == 0, "sizes are multiples of 4 bytes");
  static constexpr int LEVEL = (BYTES_PER_ELMT == 0) ? 1 : (DMA_THREADS == 0) ? 2 : (NUM_ELMTS == 0) ? 3 : 4;
  static constexpr int MAX_LDS = BYTES_PER_THREAD / ALIGNMENT;
  typedef typename hipdma::detail::chunk_of<ALIGNMENT>::type chunk_t;
  template<bool C> using when = typename std::enable_if<C, int>::type;
public:
  // ---- warp-specialised constructors ----
  template<int L = LEVEL, bool S = DO_SYNC, when<(L == 1) && S> = 0>
  __device__ __forceinline__ CudaDMAIndirect(const int dmaID, const int num_dma_threads, const int num_compute_threads,
                                             const int dma_threadIdx_start, const int elmt_size_in_bytes,
                                             const int num_elements, const int alternate_stride = 0)
    : CudaDMA(dmaID, num_dma_threads, num_compute_threads, dma_threadIdx_start)
  { init(elmt_size_in_bytes, num_elements, num_dma_threads, dma_threadIdx_start, alternate_stride); }

  template<int L = LEVEL, bool S = DO_SYNC, when<(L == 2) && S> = 0>
  __device__ __forceinline__ CudaDMAIndirect(const int dmaID, const int num_dma_threads, const int num_compute_threads,
                                             const int dma_threadIdx_start, const int num_elements,
                                             const int alternate_stride = 0)
    : CudaDMA(dmaID, num_dma_threads, num_compute_threads, dma_threadIdx_start)
  { init(BYTES_PER_ELMT, num_elements, num_dma_threads, dma_threadIdx_start, alternate_stride); }

  template<int L = LEVEL, bool S = DO_SYNC, when<(L == 3) && S> = 0>
  __device__ __forceinline__ CudaDMAIndirect(const int dmaID, const int num_compute_threads,
                                             const int dma_threadIdx_start, const int num_elements,
                                             const int alternate_stride = 0)
    : CudaDMA(dmaID, DMA_THREADS, num_compute_threads, dma_threadIdx_start)
  { init(BYTES_PER_ELMT, num_elements, DMA_THREADS, dma_threadIdx_start, alternate_stride); }

  template<int L = LEVEL, bool S = DO_SYNC, when<(L == 4) && S> = 0>
  __device__ __forceinline__ CudaDMAIndirect(const int dmaID, const int num_compute_threads,
                                             const int dma_threadIdx_start, const int alternate_stride = 0)
    : CudaDMA(dmaID, DMA_THREADS, num_compute_threads, dma_threadIdx_start)
  { init(BYTES_PER_ELMT, NUM_ELMTS, DMA_THREADS, dma_threadIdx_start, alternate_stride); }

  // ---- constructors of the form that is not warp-specialised ----
  template<int L = LEVEL, bool S = DO_SYNC, when<(L == 1) && !S> = 0>
  __device__ __forceinline__ CudaDMAIndirect(const int elmt_size_in_bytes, const int num_elements,
                                             const int alternate_stride = 0, const int num_dma_threads = 0,
                                             const int dma_threadIdx_start = 0)
    : CudaDMA(hipdma::detail::no_sync_t(), threads_or_block(num_dma_threads), dma_threadIdx_start)
  { init(elmt_size_in_bytes, num_elements, threads_or_block(num_dma_threads), dma_threadIdx_start, alternate_stride); }

  template<int L = LEVEL, bool S = DO_SYNC, when<(L == 2) && !S> = 0>
  __device__ __forceinline__ CudaDMAIndirect(const int num_elements, const int alternate_stride = 0,
                                             const int num_dma_threads = 0, const int dma_threadIdx_start = 0)
    : CudaDMA(hipdma::detail::no_sync_t(), threads_or_block(num_dma_threads), dma_threadIdx_start)
  { init(BYTES_PER_ELMT, num_elements, threads_or_block(num_dma_threads), dma_threadIdx_start, alternate_stride); }

  template<int L = LEVEL, bool S = DO_SYNC, when<(L == 3) && !S> = 0>
  __device__ __forceinline__ CudaDMAIndirect(const int num_elements, const int alternate_stride = 0,
                                             const int dma_threadIdx_start = 0)
    : CudaDMA(hipdma::detail::no_sync_t(), DMA_THREADS, dma_threadIdx_start)
  { init(BYTES_PER_ELMT, num_elements, DMA_THREADS, dma_threadIdx_start, alternate_stride); }

  template<int L = LEVEL, bool S = DO_SYNC, when<(L == 4) && !S> = 0>
  __device__ __forceinline__ CudaDMAIndirect(const int alternate_stride = 0, const int dma_threadIdx_start = 0)
    : CudaDMA(hipdma::detail::no_sync_t(), DMA_THREADS, dma_threadIdx_start)
  { init(BYTES_PER_ELMT, NUM_ELMTS, DMA_THREADS, dma_threadIdx_start, alternate_stride); }

public:
  __device__ __forceinline__ void execute_dma(const int* __restrict__ index_ptr, const void* __restrict__ src_ptr,
                                              void* __restrict__ dst_ptr)
  { execute_dma<false, LOAD_CACHE_ALL, STORE_WRITE_BACK>(index_ptr, src_ptr, dst_ptr); }
  __device__ __forceinline__ void start_xfer_async(const int* __restrict__ index_ptr, const void* __restrict__ src_ptr)
  { start_xfer_async<false, LOAD_CACHE_ALL, STORE_WRITE_BACK>(index_ptr, src_ptr); }
  __device__ __forceinline__ void wait_xfer_finish(void* __restrict__ dst_ptr)
  { wait_xfer_finish<false, LOAD_CACHE_ALL, STORE_WRITE_BACK>(dst_ptr); }

  template<bool DMA_GLOBAL_LOAD>
  __device__ __forceinline__ void execute_dma(const int* __restrict__ index_ptr, const void* __restrict__ src_ptr,
                                              void* __restrict__ dst_ptr)
  { execute_dma<DMA_GLOBAL_LOAD, LOAD_CACHE_ALL, STORE_WRITE_BACK>(index_ptr, src_ptr, dst_ptr); }
  template<bool DMA_GLOBAL_LOAD>
  __device__ __forceinline__ void start_xfer_async(const int* __restrict__ index_ptr, const void* __restrict__ src_ptr)
  { start_xfer_async<DMA_GLOBAL_LOAD, LOAD_CACHE_ALL, STORE_WRITE_BACK>(index_ptr, src_ptr); }
  template<bool DMA_GLOBAL_LOAD>
  __device__ __forceinline__ void wait_xfer_finish(void* __restrict__ dst_ptr)
  { wait_xfer_finish<DMA_GLOBAL_LOAD, LOAD_CACHE_ALL, STORE_WRITE_BACK>(dst_ptr); }

  template<bool DMA_GLOBAL_LOAD, int DMA_LOAD_QUAL, int DMA_STORE_QUAL>
  __device__ __forceinline__ void execute_dma(const int* __restrict__ index_ptr, const void* __restrict__ src_ptr,
                                              void* __restrict__ dst_ptr)
  {
    start_xfer_async<DMA_GLOBAL_LOAD, DMA_LOAD_QUAL, DMA_STORE_QUAL>(index_ptr, src_ptr);
    wait_xfer_finish<DMA_GLOBAL_LOAD, DMA_LOAD_QUAL, DMA_STORE_QUAL>(dst_ptr);
  }

  template<bool DMA_GLOBAL_LOAD, int DMA_LOAD_QUAL, int DMA_STORE_QUAL>
  __device__ __forceinline__ void start_xfer_async(const int* __restrict__ index_ptr, const void* __restrict__ src_ptr)
  { start_with<DMA_GLOBAL_LOAD, DMA_LOAD_QUAL, DMA_STORE_QUAL, false>(index_ptr, src_ptr); }

  // Requests the index words of the first step of the transfer that will be started with the same index_ptr
  // by start_xfer_async_prefetched() or execute_dma_prefetched(); returns with the loads in flight.
  // DMA_GLOBAL_LOAD says whether index_ptr points to global memory.
  template<bool DMA_GLOBAL_LOAD = false>
  __device__ __forceinline__ void prefetch_index(const int* __restrict__ index_ptr)
  {
    HIPDMA_ASSERT(index_ptr != nullptr);
#ifdef DEBUG_CUDADMA
    m_idx_next_from = index_ptr;
#endif
    hipdma::detail::GridCursor c = m_grid.begin();
#pragma unroll
    for (int k = 0; k < MAX_LDS; ++k) {
      m_idx_next[k] = m_grid.live(k, c)
          ? (int)hipdma::detail::load_vec<unsigned, DMA_GLOBAL_LOAD, LOAD_CACHE_ALL>(index_ptr + c.row) : 0;
      m_grid.advance(c);
    }
  }

  // start_xfer_async() / execute_dma() for a transfer whose index_ptr went through prefetch_index() after the
  // previous transfer of this object was started (the words of later steps are still fetched here).
  template<bool DMA_GLOBAL_LOAD = false, int DMA_LOAD_QUAL = LOAD_CACHE_ALL, int DMA_STORE_QUAL = STORE_WRITE_BACK>
  __device__ __forceinline__ void start_xfer_async_prefetched(const int* __restrict__ index_ptr,
                                                              const void* __restrict__ src_ptr)
  { start_with<DMA_GLOBAL_LOAD, DMA_LOAD_QUAL, DMA_STORE_QUAL, true>(index_ptr, src_ptr); }

  template<bool DMA_GLOBAL_LOAD = false, int DMA_LOAD_QUAL = LOAD_CACHE_ALL, int DMA_STORE_QUAL = STORE_WRITE_BACK>
  __device__ __forceinline__ void execute_dma_prefetched(const int* __restrict__ index_ptr,
                                                         const void* __restrict__ src_ptr, void* __restrict__ dst_ptr)
  {
    start_with<DMA_GLOBAL_LOAD, DMA_LOAD_QUAL, DMA_STORE_QUAL, true>(index_ptr, src_ptr);
    wait_xfer_finish<DMA_GLOBAL_LOAD, DMA_LOAD_QUAL, DMA_STORE_QUAL>(dst_ptr);
  }

  template<bool DMA_GLOBAL_LOAD, int DMA_LOAD_QUAL, int DMA_STORE_QUAL>
  __device__ __forceinline__ void wait_xfer_finish(void* __restrict__ dst_ptr)
  {
    if constexpr (DO_SYNC) CudaDMA::wait_for_dma_start();
    if (use_direct<DMA_STORE_QUAL>()) {
      if constexpr (DMA_STORE_QUAL == STORE_LDS_DIRECT && GATHER) direct_all<DMA_LOAD_QUAL>((char*)dst_ptr);
    } else {
      hipdma::detail::GridCursor cur = m_grid.begin();
      store_step<DMA_STORE_QUAL>((char*)dst_ptr, 0, cur);
      for (int step = 1; step < m_grid.steps; ++step) {
        load_step<DMA_GLOBAL_LOAD, DMA_LOAD_QUAL>(step, cur);
        store_step<DMA_STORE_QUAL>((char*)dst_ptr, step, cur);
      }
    }
    if constexpr (DO_SYNC) CudaDMA::finish_async_dma();
  }

private:
  __device__ __forceinline__ static int threads_or_block(const int n) { return (n <= 0) ? int(blockDim.x) : n; }

  template<bool DMA_GLOBAL_LOAD, int DMA_LOAD_QUAL, int DMA_STORE_QUAL, bool PREFETCHED>
  __device__ __forceinline__ void start_with(const int* __restrict__ index_ptr, const void* __restrict__ src_ptr)
  {
    static_assert(DMA_STORE_QUAL != STORE_LDS_DIRECT || (GATHER && DMA_GLOBAL_LOAD),
                  "STORE_LDS_DIRECT needs a gather from a global source");
    static_assert(!hipdma::detail::store_is_swizzled(DMA_STORE_QUAL), "swizzled LDS rows are a CudaDMAStrided layout");
    HIPDMA_ASSERT(index_ptr != nullptr && (reinterpret_cast<uintptr_t>(src_ptr) % ALIGNMENT) == 0);
#ifdef DEBUG_CUDADMA
    if constexpr (PREFETCHED) HIPDMA_ASSERT(m_idx_next_from == index_ptr);   // the words on hand belong to this transfer
#endif
    m_index = index_ptr;
    m_src = (const char*)src_ptr;
    if (use_direct<DMA_STORE_QUAL>()) return;          // the direct form reads its index words when it issues its loads
    load_step<DMA_GLOBAL_LOAD, DMA_LOAD_QUAL, PREFETCHED>(0, m_grid.begin());
  }

  __device__ __forceinline__ void init(const int e, const int n, const int t, const int start, const int alt)
  {
    HIPDMA_ASSERT(e >= 0 && (e % 4) == 0 && n >= 0);
    HIPDMA_ASSERT(t > 0 && (t % HIPDMA_WAVE_SIZE) == 0);
    HIPDMA_ASSERT((alt % ALIGNMENT) == 0);
    m_grid.init(ALIGNMENT, MAX_LDS, e, n, t, int(threadIdx.x) - start);
    m_dense_stride = (alt > e) ? alt : e;
    // a *_prefetched() call that was not preceded by prefetch_index() then addresses record 0 instead of whatever
    // the registers held (the stores vanish from kernels that never use the prefetched calls)
#pragma unroll
    for (int k = 0; k < MAX_LDS; ++k) m_idx_next[k] = 0;
  }

  template<int STORE_QUAL>
  __device__ __forceinline__ bool use_direct() const
  {
    if constexpr (GATHER && STORE_QUAL == STORE_LDS_DIRECT && (ALIGNMENT == 16 || ALIGNMENT == 4))
      return (m_grid.last_bytes == ALIGNMENT) && ((m_grid.T % HIPDMA_WAVE_SIZE) == 0) &&
             ((m_grid.W >= HIPDMA_WAVE_SIZE) ||
              ((m_grid.W == m_grid.LPE) && (m_dense_stride == m_grid.E)));
    else
      return false;
  }

  // Index words travel as plain global/generic dword loads.
  template<bool GLOBAL_LOAD>
  __device__ __forceinline__ int load_index(const int row) const
  { return (int)hipdma::detail::load_vec<unsigned, GLOBAL_LOAD, LOAD_CACHE_ALL>(m_index + row); }

  // PREFETCHED (step 0 only): the index words are the ones prefetch_index() asked for.
  template<bool GLOBAL_LOAD, int LOAD_QUAL, bool PREFETCHED = false>
  __device__ __forceinline__ void load_step(const int step, hipdma::detail::GridCursor cur)
  {
    using namespace hipdma::detail;
    GridCursor c = cur;
#pragma unroll
    for (int k = 0; k < MAX_LDS; ++k) {
      if constexpr (PREFETCHED) m_idx[k] = m_idx_next[k];
      else m_idx[k] = m_grid.live(step * MAX_LDS + k, c) ? load_index<GLOBAL_LOAD>(c.row) : 0;
      m_grid.advance(c);
    }
    c = cur;
#pragma unroll
    for (int k = 0; k < MAX_LDS; ++k) {
      if (m_grid.live(step * MAX_LDS + k, c)) {
        // the indexed side takes a 64-bit offset: a table may exceed 2 GiB (the reference multiplies in int)
        const long long off = GATHER ? ((long long)m_idx[k] * m_grid.E + c.col * ALIGNMENT)
                                     : (long long)(c.row * m_dense_stride + c.col * ALIGNMENT);
        load_chunk<ALIGNMENT, ALIGNMENT, GLOBAL_LOAD, LOAD_QUAL>(m_buf[k], m_src + off,
                                                                 m_grid.chunk_bytes(ALIGNMENT, c));
      }
      m_grid.advance(c);
    }
  }

  template<int STORE_QUAL>
  __device__ __forceinline__ void store_step(char* dst, const int step, hipdma::detail::GridCursor& cur) const
  {
    using namespace hipdma::detail;
#pragma unroll
    for (int k = 0; k < MAX_LDS; ++k) {
      if (m_grid.live(step * MAX_LDS + k, cur)) {
        const long long off = GATHER ? (long long)(cur.row * m_dense_stride + cur.col * ALIGNMENT)
                                     : ((long long)m_idx[k] * m_grid.E + cur.col * ALIGNMENT);
        store_chunk<ALIGNMENT, ALIGNMENT, STORE_QUAL>(m_buf[k], dst + off, m_grid.chunk_bytes(ALIGNMENT, cur));
      }
      m_grid.advance(cur);
    }
  }

  template<int LOAD_QUAL>
  __device__ __forceinline__ void direct_all(char* dst)
  {
    using namespace hipdma::detail;
    const int lane = lane_id();
    GridCursor cur = m_grid.begin();
    for (int r0 = 0; r0 < m_grid.rounds; r0 += MAX_LDS) {
      GridCursor c = cur;
#pragma unroll
      for (int k = 0; k < MAX_LDS; ++k) {
        m_idx[k] = m_grid.live(r0 + k, c) ? load_index<true>(c.row) : 0;
        m_grid.advance(c);
      }
#pragma unroll
      for (int k = 0; k < MAX_LDS; ++k) {
        if (m_grid.live(r0 + k, cur)) {
          const int lds_off = cur.row * m_dense_stride + cur.col * ALIGNMENT;
          if constexpr (ALIGNMENT == 16 || ALIGNMENT == 4)
            load_to_lds<ALIGNMENT, LOAD_QUAL>(m_src + ((long long)m_idx[k] * m_grid.E + cur.col * ALIGNMENT),
                                   dst + (lds_off - lane * ALIGNMENT));
        }
        m_grid.advance(cur);
      }
    }
    wait_lds_direct();
  }

private:
  hipdma::detail::GridState m_grid;
  int m_dense_stride;
  const int* m_index;
  const char* m_src;
  int m_idx[MAX_LDS];
  int m_idx_next[MAX_LDS];      // prefetch_index(): index words of the first step of the next transfer
#ifdef DEBUG_CUDADMA
  const int* m_idx_next_from = nullptr;
#endif
  chunk_t m_buf[MAX_LDS];
};

// Host-side planner report (include/cudaDMAv2.h:9417-9698).
template<bool GATHER, bool DO_SYNC>
class CudaDMAIndirect<GATHER, DO_SYNC, 0, 0, 0, 0, 0> {
public:
  __host__ static void diagnose(const int ALIGNMENT, const int BYTES_PER_THREAD, const int BYTES_PER_ELMT,
                                const int DMA_THREADS, const int NUM_ELMTS, const bool FULL_TEMPLATE,
                                const bool verbose = false)
  {
    fprintf(stdout, "==== CudaDMAIndirect (%s): one index word per element, then the plan below ====\n",
            GATHER ? "gather" : "scatter");
    CudaDMAStrided<DO_SYNC, 0, 0, 0, 0, 0>::diagnose(ALIGNMENT, BYTES_PER_THREAD, BYTES_PER_ELMT, DMA_THREADS,
                                                       NUM_ELMTS, FULL_TEMPLATE, verbose);
  }
};
