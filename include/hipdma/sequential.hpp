// CudaDMASequential: contiguous block transfer, dst[0..B) = src[0..B).
//
// API contract: include/cudaDMAv2.h:1356-2971 (template parameters :1367,
// constructor forms :1848-1852, :2042-2044, :2265-2268, :2449-2450,
// :2663-2665, :2811; transfer methods :1460-1562; diagnose :1402-1458).
//
// Work split (wave64): the block is cut into chunks of ALIGNMENT bytes; chunk c
// belongs to DMA thread c % T, so one wavefront instruction touches 64
// consecutive chunks (1 KiB for ALIGNMENT 16).  A thread keeps at most
// BYTES_PER_THREAD/ALIGNMENT chunks in VGPRs; that many rounds make a step.
// start_xfer_async() issues the loads of step 0 and returns with them in
// flight, wait_xfer_finish() waits for the buffer, drains step 0 into it and
// runs the remaining steps load-then-store.  A tail of 4, 8 or 12 bytes is
// moved by the thread that owns the last chunk.
#pragma once

#include "mem.hpp"

namespace hipdma {

// Host/device description of how a sequential transfer is cut up.
struct SequentialPlan {
  int alignment, bytes_per_thread, bytes_per_elmt, dma_threads;
  int loads_per_step;    // chunks a thread holds in registers
  int step_bytes;        // bytes all threads move in one full step
  int full_steps;        // steps in which every thread moves loads_per_step full chunks
  int tail_bytes;        // bytes left for the last, predicated step
  int total_steps;
  __host__ __device__ constexpr SequentialPlan(int a, int bpt, int bpe, int t)
    : alignment(a), bytes_per_thread(bpt), bytes_per_elmt(bpe), dma_threads(t),
      loads_per_step(bpt / a), step_bytes(t * a * (bpt / a)),
      full_steps(step_bytes > 0 ? bpe / step_bytes : 0),
      tail_bytes(step_bytes > 0 ? bpe - (bpe / step_bytes) * step_bytes : 0),
      total_steps((step_bytes > 0 ? bpe / step_bytes : 0) +
                  ((step_bytes > 0 && (bpe % step_bytes) != 0) ? 1 : 0)) {}
  // Byte offset of the chunk DMA thread `tid` holds in register slot k during `step`.
  __host__ __device__ static constexpr int chunk_offset(int alignment, int max_lds, int threads, int tid, int step, int k)
  { return (tid + (step * max_lds + k) * threads) * alignment; }
};

}  // namespace hipdma

template<bool DO_SYNC = false, int ALIGNMENT = 0, int BYTES_PER_THREAD = 4 * ALIGNMENT,
         int BYTES_PER_ELMT = 0, int DMA_THREADS = 0>
class CudaDMASequential : public CudaDMA {
  static_assert(ALIGNMENT == 4 || ALIGNMENT == 8 || ALIGNMENT == 16, "ALIGNMENT must be 4, 8 or 16");
  static_assert((BYTES_PER_THREAD / ALIGNMENT) > 0, "BYTES_PER_THREAD must hold at least one chunk");
  static_assert((BYTES_PER_THREAD % ALIGNMENT) == 0, "BYTES_PER_THREAD must be a multiple of ALIGNMENT");
  static_assert((BYTES_PER_ELMT % 4) == 0, "sizes are multiples of 4 bytes");
  static constexpr int LEVEL = (BYTES_PER_ELMT == 0) ? 1 : (DMA_THREADS == 0) ? 2 : 3;
  static constexpr int MAX_LDS = BYTES_PER_THREAD / ALIGNMENT;
  typedef typename hipdma::detail::chunk_of<ALIGNMENT>::type chunk_t;
  template<bool C> using when = typename std::enable_if<C, int>::type;
public:
  // ---- warp-specialised constructors ----
  template<int L = LEVEL, bool S = DO_SYNC, when<(L == 1) && S> = 0>
  __device__ __forceinline__ CudaDMASequential(const int dmaID, const int num_dma_threads,
                                               const int num_compute_threads, const int dma_threadIdx_start,
                                               const int elmt_size_in_bytes)
    : CudaDMA(dmaID, num_dma_threads, num_compute_threads, dma_threadIdx_start)
  { init(elmt_size_in_bytes, num_dma_threads, dma_threadIdx_start); }

  template<int L = LEVEL, bool S = DO_SYNC, when<(L == 2) && S> = 0>
  __device__ __forceinline__ CudaDMASequential(const int dmaID, const int num_dma_threads,
                                               const int num_compute_threads, const int dma_threadIdx_start)
    : CudaDMA(dmaID, num_dma_threads, num_compute_threads, dma_threadIdx_start)
  { init(BYTES_PER_ELMT, num_dma_threads, dma_threadIdx_start); }

  template<int L = LEVEL, bool S = DO_SYNC, when<(L == 3) && S> = 0>
  __device__ __forceinline__ CudaDMASequential(const int dmaID, const int num_compute_threads,
                                               const int dma_threadIdx_start)
    : CudaDMA(dmaID, DMA_THREADS, num_compute_threads, dma_threadIdx_start)
  { init(BYTES_PER_ELMT, DMA_THREADS, dma_threadIdx_start); }

  // ---- constructors of the form that is not warp-specialised ----
  template<int L = LEVEL, bool S = DO_SYNC, when<(L == 1) && !S> = 0>
  __device__ __forceinline__ CudaDMASequential(const int elmt_size_in_bytes, const int num_dma_threads = 0,
                                               const int dma_threadIdx_start = 0)
    : CudaDMA(hipdma::detail::no_sync_t(), threads_or_block(num_dma_threads), dma_threadIdx_start)
  { init(elmt_size_in_bytes, threads_or_block(num_dma_threads), dma_threadIdx_start); }

  template<int L = LEVEL, bool S = DO_SYNC, when<(L == 2) && !S> = 0>
  __device__ __forceinline__ CudaDMASequential(const int num_dma_threads = 0, const int dma_threadIdx_start = 0)
    : CudaDMA(hipdma::detail::no_sync_t(), threads_or_block(num_dma_threads), dma_threadIdx_start)
  { init(BYTES_PER_ELMT, threads_or_block(num_dma_threads), dma_threadIdx_start); }

  template<int L = LEVEL, bool S = DO_SYNC, when<(L == 3) && !S> = 0>
  __device__ __forceinline__ CudaDMASequential(const int dma_threadIdx_start = 0)
    : CudaDMA(hipdma::detail::no_sync_t(), DMA_THREADS, dma_threadIdx_start)
  { init(BYTES_PER_ELMT, DMA_THREADS, dma_threadIdx_start); }

public:
  // ---- unqualified transfer methods: generic source, generic destination ----
  __device__ __forceinline__ void execute_dma(const void* __restrict__ src_ptr, void* __restrict__ dst_ptr)
  { execute_dma<false, LOAD_CACHE_ALL, STORE_WRITE_BACK>(src_ptr, dst_ptr); }
  __device__ __forceinline__ void start_xfer_async(const void* __restrict__ src_ptr)
  { start_xfer_async<false, LOAD_CACHE_ALL, STORE_WRITE_BACK>(src_ptr); }
  __device__ __forceinline__ void wait_xfer_finish(void* __restrict__ dst_ptr)
  { wait_xfer_finish<false, LOAD_CACHE_ALL, STORE_WRITE_BACK>(dst_ptr); }

  // ---- qualified on the source address space ----
  template<bool DMA_GLOBAL_LOAD>
  __device__ __forceinline__ void execute_dma(const void* __restrict__ src_ptr, void* __restrict__ dst_ptr)
  { execute_dma<DMA_GLOBAL_LOAD, LOAD_CACHE_ALL, STORE_WRITE_BACK>(src_ptr, dst_ptr); }
  template<bool DMA_GLOBAL_LOAD>
  __device__ __forceinline__ void start_xfer_async(const void* __restrict__ src_ptr)
  { start_xfer_async<DMA_GLOBAL_LOAD, LOAD_CACHE_ALL, STORE_WRITE_BACK>(src_ptr); }
  template<bool DMA_GLOBAL_LOAD>
  __device__ __forceinline__ void wait_xfer_finish(void* __restrict__ dst_ptr)
  { wait_xfer_finish<DMA_GLOBAL_LOAD, LOAD_CACHE_ALL, STORE_WRITE_BACK>(dst_ptr); }

  // ---- fully qualified ----
  template<bool DMA_GLOBAL_LOAD, int DMA_LOAD_QUAL, int DMA_STORE_QUAL>
  __device__ __forceinline__ void execute_dma(const void* __restrict__ src_ptr, void* __restrict__ dst_ptr)
  {
    start_xfer_async<DMA_GLOBAL_LOAD, DMA_LOAD_QUAL, DMA_STORE_QUAL>(src_ptr);
    wait_xfer_finish<DMA_GLOBAL_LOAD, DMA_LOAD_QUAL, DMA_STORE_QUAL>(dst_ptr);
  }

  template<bool DMA_GLOBAL_LOAD, int DMA_LOAD_QUAL, int DMA_STORE_QUAL>
  __device__ __forceinline__ void start_xfer_async(const void* __restrict__ src_ptr)
  {
    static_assert(!hipdma::detail::store_is_swizzled(DMA_STORE_QUAL), "swizzled LDS rows are a CudaDMAStrided layout");
    HIPDMA_ASSERT((reinterpret_cast<uintptr_t>(src_ptr) % ALIGNMENT) == 0);
    m_src = (const char*)src_ptr;
    if constexpr (DMA_STORE_QUAL != STORE_LDS_DIRECT)
      load_step<DMA_GLOBAL_LOAD, DMA_LOAD_QUAL>(0);
  }

  template<bool DMA_GLOBAL_LOAD, int DMA_LOAD_QUAL, int DMA_STORE_QUAL>
  __device__ __forceinline__ void wait_xfer_finish(void* __restrict__ dst_ptr)
  {
    if constexpr (DO_SYNC) CudaDMA::wait_for_dma_start();
    if constexpr (DMA_STORE_QUAL == STORE_LDS_DIRECT) {
      static_assert(DMA_STORE_QUAL != STORE_LDS_DIRECT || DMA_GLOBAL_LOAD,
                    "STORE_LDS_DIRECT needs a global source");
      direct_all<DMA_LOAD_QUAL>((char*)dst_ptr);
    } else {
      store_step<DMA_STORE_QUAL>((char*)dst_ptr, 0);
      for (int step = 1; step < m_total_steps; ++step) {
        load_step<DMA_GLOBAL_LOAD, DMA_LOAD_QUAL>(step);
        store_step<DMA_STORE_QUAL>((char*)dst_ptr, step);
      }
    }
    if constexpr (DO_SYNC) CudaDMA::finish_async_dma();
  }

private:
  __device__ __forceinline__ static int threads_or_block(const int n) { return (n <= 0) ? int(blockDim.x) : n; }

  __device__ __forceinline__ void init(const int bytes, const int threads, const int start)
  {
    HIPDMA_ASSERT(bytes >= 0 && (bytes % 4) == 0);
    HIPDMA_ASSERT(threads > 0 && (threads % HIPDMA_WAVE_SIZE) == 0);
    m_bytes = bytes;
    m_threads = threads;
    m_tid = int(threadIdx.x) - start;
    const int step_bytes = threads * BYTES_PER_THREAD;
    m_full_steps = bytes / step_bytes;
    m_total_steps = m_full_steps + (((bytes % step_bytes) != 0) ? 1 : 0);
  }

  // Byte offset of the chunk held in register slot k during `step`.
  __device__ __forceinline__ int chunk_offset(const int step, const int k) const
  { return hipdma::SequentialPlan::chunk_offset(ALIGNMENT, MAX_LDS, m_threads, m_tid, step, k); }

  template<bool GLOBAL_LOAD, int LOAD_QUAL>
  __device__ __forceinline__ void load_step(const int step)
  {
    using namespace hipdma::detail;
    if (step < m_full_steps) {
#pragma unroll
      for (int k = 0; k < MAX_LDS; ++k)
        m_buf[k] = load_vec<chunk_t, GLOBAL_LOAD, LOAD_QUAL>(m_src + chunk_offset(step, k));
    } else {
#pragma unroll
      for (int k = 0; k < MAX_LDS; ++k) {
        const int off = chunk_offset(step, k);
        const int rem = m_bytes - off;
        if (rem >= ALIGNMENT)
          m_buf[k] = load_vec<chunk_t, GLOBAL_LOAD, LOAD_QUAL>(m_src + off);
        else if (rem > 0)
          load_chunk<ALIGNMENT, 4, GLOBAL_LOAD, LOAD_QUAL>(m_buf[k], m_src + off, rem);
      }
    }
  }

  template<int STORE_QUAL>
  __device__ __forceinline__ void store_step(char* dst, const int step) const
  {
    using namespace hipdma::detail;
    if (step < m_full_steps) {
#pragma unroll
      for (int k = 0; k < MAX_LDS; ++k)
        store_vec<chunk_t, STORE_QUAL>(m_buf[k], dst + chunk_offset(step, k));
    } else {
#pragma unroll
      for (int k = 0; k < MAX_LDS; ++k) {
        const int off = chunk_offset(step, k);
        const int rem = m_bytes - off;
        if (rem >= ALIGNMENT)
          store_vec<chunk_t, STORE_QUAL>(m_buf[k], dst + off);
        else if (rem > 0)
          store_chunk<ALIGNMENT, 4, STORE_QUAL>(m_buf[k], dst + off, rem);
      }
    }
  }

  // Whole transfer without register staging.  Full chunks go through
  // global_load_lds; a ragged tail goes through one register chunk.
  template<int LOAD_QUAL>
  __device__ __forceinline__ void direct_all(char* dst)
  {
    using namespace hipdma::detail;
    static_assert(ALIGNMENT == 16 || ALIGNMENT == 4, "the direct path moves 4 or 16 bytes per lane");
    const int lane = lane_id();
    const int rounds = ceil_div(ceil_div(m_bytes, ALIGNMENT), m_threads);
    for (int r = 0; r < rounds; ++r) {
      const int off = (m_tid + r * m_threads) * ALIGNMENT;
      const int wave_off = off - lane * ALIGNMENT;
      const int rem = m_bytes - off;
      if (rem >= ALIGNMENT) {
        load_to_lds<ALIGNMENT, LOAD_QUAL>(m_src + off, dst + wave_off);
      } else if (rem > 0) {
        chunk_t tail;
        load_chunk<ALIGNMENT, 4, true, LOAD_QUAL>(tail, m_src + off, rem);
        store_chunk<ALIGNMENT, 4, STORE_LDS>(tail, dst + off, rem);
      }
    }
    wait_lds_direct();
  }

private:
  int m_bytes;
  int m_threads;
  int m_tid;
  int m_full_steps;
  int m_total_steps;
  const char* m_src;
  chunk_t m_buf[MAX_LDS];
};

// Host-side planner report (include/cudaDMAv2.h:1402-1458).
template<bool DO_SYNC>
class CudaDMASequential<DO_SYNC, 0, 0, 0, 0> {
public:
  __host__ static void diagnose(const int ALIGNMENT, const int BYTES_PER_THREAD, const int BYTES_PER_ELMT,
                                const int DMA_THREADS, const bool FULL_TEMPLATE, const bool verbose = false)
  {
    const hipdma::SequentialPlan p(ALIGNMENT, BYTES_PER_THREAD, BYTES_PER_ELMT, DMA_THREADS);
    fprintf(stdout, "==== CudaDMASequential plan (gfx950, 64-lane wavefronts) ====\n");
    fprintf(stdout, "  ALIGNMENT %d  BYTES_PER_THREAD %d  BYTES_PER_ELMT %d  DMA_THREADS %d (%d wavefronts)  %s\n",
            ALIGNMENT, BYTES_PER_THREAD, BYTES_PER_ELMT, DMA_THREADS,
            (DMA_THREADS + HIPDMA_WAVE_SIZE - 1) / HIPDMA_WAVE_SIZE,
            FULL_TEMPLATE ? "compile-time parameters" : "run-time parameters");
    fprintf(stdout, "  steps needed: %d (%d full + %d partial), %d bytes in flight per full step\n",
            p.total_steps, p.full_steps, p.total_steps - p.full_steps, p.step_bytes);
    if (p.total_steps <= 1) {
      fprintf(stdout, "  single step: every load is issued before the handshake wait.\n");
    } else {
      fprintf(stdout, "  multiple steps: later loads wait for earlier stores. To reach one step use\n");
      fprintf(stdout, "    DMA_THREADS >= %d at this BYTES_PER_THREAD, or BYTES_PER_THREAD >= %d at this DMA_THREADS\n",
              hipdma::detail::round_up(hipdma::detail::ceil_div(BYTES_PER_ELMT, BYTES_PER_THREAD), HIPDMA_WAVE_SIZE),
              hipdma::detail::round_up(hipdma::detail::ceil_div(BYTES_PER_ELMT, DMA_THREADS), ALIGNMENT));
      if (ALIGNMENT < 16)
        fprintf(stdout, "    or raise ALIGNMENT to 16 (dwordx4 moves) by padding the element\n");
    }
    if (verbose)
      fprintf(stdout, "  loads_per_step %d  step_bytes %d  full_steps %d  tail_bytes %d\n",
              p.loads_per_step, p.step_bytes, p.full_steps, p.tail_bytes);
    fflush(stdout);
  }
};
