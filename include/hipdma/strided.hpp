// CudaDMAStrided: 2-D transfer, dst[i*dst_stride + j] = src[i*src_stride + j]
// for i < NUM_ELMTS, j < BYTES_PER_ELMT.
//
// API contract: include/cudaDMAv2.h:2973-9368 (template parameters :3193-3194;
// warp-specialised constructors :5110-5163, :6298-6330, :7480-7510, :8610-8651;
// the other constructors :5556-5604, :6728-6760, :7877-7905, :8993-9030;
// diagnose :3208-3493).  The work split is the slot grid of grid.hpp.
#pragma once

#include "grid.hpp"

template<bool DO_SYNC = false, int ALIGNMENT = 0, int BYTES_PER_THREAD = 4 * ALIGNMENT,
         int BYTES_PER_ELMT = 0, int DMA_THREADS = 0, int NUM_ELMTS = 0>
class CudaDMAStrided : public CudaDMA {
  static_assert(ALIGNMENT == 4 || ALIGNMENT == 8 || ALIGNMENT == 16, "ALIGNMENT must be 4, 8 or 16");
  static_assert((BYTES_PER_THREAD / ALIGNMENT) > 0, "BYTES_PER_THREAD must hold at least one chunk");
  static_assert((BYTES_PER_THREAD % ALIGNMENT) == 0, "BYTES_PER_THREAD must be a multiple of ALIGNMENT");
  static_assert((BYTES_PER_ELMT % 4) == 0, "sizes are multiples of 4 bytes");
  static constexpr int LEVEL = (BYTES_PER_ELMT == 0) ? 1 : (DMA_THREADS == 0) ? 2 : (NUM_ELMTS == 0) ? 3 : 4;
  static constexpr int MAX_LDS = BYTES_PER_THREAD / ALIGNMENT;
  typedef typename hipdma::detail::chunk_of<ALIGNMENT>::type chunk_t;
  template<bool C> using when = typename std::enable_if<C, int>::type;
public:
  // ---- warp-specialised constructors: one stride for both sides, or src and dst strides ----
  template<int L = LEVEL, bool S = DO_SYNC, when<(L == 1) && S> = 0>
  __device__ __forceinline__ CudaDMAStrided(const int dmaID, const int num_dma_threads, const int num_compute_threads,
                                            const int dma_threadIdx_start, const int elmt_size_in_bytes,
                                            const int num_elements, const int elmt_stride)
    : CudaDMA(dmaID, num_dma_threads, num_compute_threads, dma_threadIdx_start)
  { init(elmt_size_in_bytes, num_elements, num_dma_threads, dma_threadIdx_start, elmt_stride, elmt_stride); }
  template<int L = LEVEL, bool S = DO_SYNC, when<(L == 1) && S> = 0>
  __device__ __forceinline__ CudaDMAStrided(const int dmaID, const int num_dma_threads, const int num_compute_threads,
                                            const int dma_threadIdx_start, const int elmt_size_in_bytes,
                                            const int num_elements, const int src_stride, const int dst_stride)
    : CudaDMA(dmaID, num_dma_threads, num_compute_threads, dma_threadIdx_start)
  { init(elmt_size_in_bytes, num_elements, num_dma_threads, dma_threadIdx_start, src_stride, dst_stride); }

  template<int L = LEVEL, bool S = DO_SYNC, when<(L == 2) && S> = 0>
  __device__ __forceinline__ CudaDMAStrided(const int dmaID, const int num_dma_threads, const int num_compute_threads,
                                            const int dma_threadIdx_start, const int num_elements,
                                            const int elmt_stride)
    : CudaDMA(dmaID, num_dma_threads, num_compute_threads, dma_threadIdx_start)
  { init(BYTES_PER_ELMT, num_elements, num_dma_threads, dma_threadIdx_start, elmt_stride, elmt_stride); }
  template<int L = LEVEL, bool S = DO_SYNC, when<(L == 2) && S> = 0>
  __device__ __forceinline__ CudaDMAStrided(const int dmaID, const int num_dma_threads, const int num_compute_threads,
                                            const int dma_threadIdx_start, const int num_elements,
                                            const int src_stride, const int dst_stride)
    : CudaDMA(dmaID, num_dma_threads, num_compute_threads, dma_threadIdx_start)
  { init(BYTES_PER_ELMT, num_elements, num_dma_threads, dma_threadIdx_start, src_stride, dst_stride); }

  template<int L = LEVEL, bool S = DO_SYNC, when<(L == 3) && S> = 0>
  __device__ __forceinline__ CudaDMAStrided(const int dmaID, const int num_compute_threads,
                                            const int dma_threadIdx_start, const int num_elements,
                                            const int elmt_stride)
    : CudaDMA(dmaID, DMA_THREADS, num_compute_threads, dma_threadIdx_start)
  { init(BYTES_PER_ELMT, num_elements, DMA_THREADS, dma_threadIdx_start, elmt_stride, elmt_stride); }
  template<int L = LEVEL, bool S = DO_SYNC, when<(L == 3) && S> = 0>
  __device__ __forceinline__ CudaDMAStrided(const int dmaID, const int num_compute_threads,
                                            const int dma_threadIdx_start, const int num_elements,
                                            const int src_stride, const int dst_stride)
    : CudaDMA(dmaID, DMA_THREADS, num_compute_threads, dma_threadIdx_start)
  { init(BYTES_PER_ELMT, num_elements, DMA_THREADS, dma_threadIdx_start, src_stride, dst_stride); }

  template<int L = LEVEL, bool S = DO_SYNC, when<(L == 4) && S> = 0>
  __device__ __forceinline__ CudaDMAStrided(const int dmaID, const int num_compute_threads,
                                            const int dma_threadIdx_start, const int elmt_stride)
    : CudaDMA(dmaID, DMA_THREADS, num_compute_threads, dma_threadIdx_start)
  { init(BYTES_PER_ELMT, NUM_ELMTS, DMA_THREADS, dma_threadIdx_start, elmt_stride, elmt_stride); }
  template<int L = LEVEL, bool S = DO_SYNC, when<(L == 4) && S> = 0>
  __device__ __forceinline__ CudaDMAStrided(const int dmaID, const int num_compute_threads,
                                            const int dma_threadIdx_start, const int src_stride,
                                            const int dst_stride)
    : CudaDMA(dmaID, DMA_THREADS, num_compute_threads, dma_threadIdx_start)
  { init(BYTES_PER_ELMT, NUM_ELMTS, DMA_THREADS, dma_threadIdx_start, src_stride, dst_stride); }

  // ---- constructors of the form that is not warp-specialised ----
  template<int L = LEVEL, bool S = DO_SYNC, when<(L == 1) && !S> = 0>
  __device__ __forceinline__ CudaDMAStrided(const int elmt_size_in_bytes, const int num_elements,
                                            const int elmt_stride)
    : CudaDMA(hipdma::detail::no_sync_t(), int(blockDim.x), 0)
  { init(elmt_size_in_bytes, num_elements, int(blockDim.x), 0, elmt_stride, elmt_stride); }
  template<int L = LEVEL, bool S = DO_SYNC, when<(L == 1) && !S> = 0>
  __device__ __forceinline__ CudaDMAStrided(const int elmt_size_in_bytes, const int num_elements,
                                            const int src_stride, const int dst_stride,
                                            const int num_dma_threads = 0, const int dma_threadIdx_start = 0)
    : CudaDMA(hipdma::detail::no_sync_t(), threads_or_block(num_dma_threads), dma_threadIdx_start)
  { init(elmt_size_in_bytes, num_elements, threads_or_block(num_dma_threads), dma_threadIdx_start, src_stride, dst_stride); }

  template<int L = LEVEL, bool S = DO_SYNC, when<(L == 2) && !S> = 0>
  __device__ __forceinline__ CudaDMAStrided(const int num_elements, const int elmt_stride)
    : CudaDMA(hipdma::detail::no_sync_t(), int(blockDim.x), 0)
  { init(BYTES_PER_ELMT, num_elements, int(blockDim.x), 0, elmt_stride, elmt_stride); }
  template<int L = LEVEL, bool S = DO_SYNC, when<(L == 2) && !S> = 0>
  __device__ __forceinline__ CudaDMAStrided(const int num_elements, const int src_stride, const int dst_stride,
                                            const int num_dma_threads = 0, const int dma_threadIdx_start = 0)
    : CudaDMA(hipdma::detail::no_sync_t(), threads_or_block(num_dma_threads), dma_threadIdx_start)
  { init(BYTES_PER_ELMT, num_elements, threads_or_block(num_dma_threads), dma_threadIdx_start, src_stride, dst_stride); }

  template<int L = LEVEL, bool S = DO_SYNC, when<(L == 3) && !S> = 0>
  __device__ __forceinline__ CudaDMAStrided(const int num_elements, const int elmt_stride)
    : CudaDMA(hipdma::detail::no_sync_t(), DMA_THREADS, 0)
  { init(BYTES_PER_ELMT, num_elements, DMA_THREADS, 0, elmt_stride, elmt_stride); }
  template<int L = LEVEL, bool S = DO_SYNC, when<(L == 3) && !S> = 0>
  __device__ __forceinline__ CudaDMAStrided(const int num_elements, const int src_stride, const int dst_stride,
                                            const int dma_threadIdx_start = 0)
    : CudaDMA(hipdma::detail::no_sync_t(), DMA_THREADS, dma_threadIdx_start)
  { init(BYTES_PER_ELMT, num_elements, DMA_THREADS, dma_threadIdx_start, src_stride, dst_stride); }

  template<int L = LEVEL, bool S = DO_SYNC, when<(L == 4) && !S> = 0>
  __device__ __forceinline__ CudaDMAStrided(const int elmt_stride)
    : CudaDMA(hipdma::detail::no_sync_t(), DMA_THREADS, 0)
  { init(BYTES_PER_ELMT, NUM_ELMTS, DMA_THREADS, 0, elmt_stride, elmt_stride); }
  template<int L = LEVEL, bool S = DO_SYNC, when<(L == 4) && !S> = 0>
  __device__ __forceinline__ CudaDMAStrided(const int src_stride, const int dst_stride,
                                            const int dma_threadIdx_start = 0)
    : CudaDMA(hipdma::detail::no_sync_t(), DMA_THREADS, dma_threadIdx_start)
  { init(BYTES_PER_ELMT, NUM_ELMTS, DMA_THREADS, dma_threadIdx_start, src_stride, dst_stride); }

public:
  __device__ __forceinline__ void execute_dma(const void* __restrict__ src_ptr, void* __restrict__ dst_ptr)
  { execute_dma<false, LOAD_CACHE_ALL, STORE_WRITE_BACK>(src_ptr, dst_ptr); }
  __device__ __forceinline__ void start_xfer_async(const void* __restrict__ src_ptr)
  { start_xfer_async<false, LOAD_CACHE_ALL, STORE_WRITE_BACK>(src_ptr); }
  __device__ __forceinline__ void wait_xfer_finish(void* __restrict__ dst_ptr)
  { wait_xfer_finish<false, LOAD_CACHE_ALL, STORE_WRITE_BACK>(dst_ptr); }

  template<bool DMA_GLOBAL_LOAD>
  __device__ __forceinline__ void execute_dma(const void* __restrict__ src_ptr, void* __restrict__ dst_ptr)
  { execute_dma<DMA_GLOBAL_LOAD, LOAD_CACHE_ALL, STORE_WRITE_BACK>(src_ptr, dst_ptr); }
  template<bool DMA_GLOBAL_LOAD>
  __device__ __forceinline__ void start_xfer_async(const void* __restrict__ src_ptr)
  { start_xfer_async<DMA_GLOBAL_LOAD, LOAD_CACHE_ALL, STORE_WRITE_BACK>(src_ptr); }
  template<bool DMA_GLOBAL_LOAD>
  __device__ __forceinline__ void wait_xfer_finish(void* __restrict__ dst_ptr)
  { wait_xfer_finish<DMA_GLOBAL_LOAD, LOAD_CACHE_ALL, STORE_WRITE_BACK>(dst_ptr); }

  template<bool DMA_GLOBAL_LOAD, int DMA_LOAD_QUAL, int DMA_STORE_QUAL>
  __device__ __forceinline__ void execute_dma(const void* __restrict__ src_ptr, void* __restrict__ dst_ptr)
  {
    start_xfer_async<DMA_GLOBAL_LOAD, DMA_LOAD_QUAL, DMA_STORE_QUAL>(src_ptr);
    wait_xfer_finish<DMA_GLOBAL_LOAD, DMA_LOAD_QUAL, DMA_STORE_QUAL>(dst_ptr);
  }

  template<bool DMA_GLOBAL_LOAD, int DMA_LOAD_QUAL, int DMA_STORE_QUAL>
  __device__ __forceinline__ void start_xfer_async(const void* __restrict__ src_ptr)
  {
    HIPDMA_ASSERT((reinterpret_cast<uintptr_t>(src_ptr) % ALIGNMENT) == 0);
    m_src = (const char*)src_ptr;
    if (use_direct<DMA_STORE_QUAL>()) return;
    load_step<DMA_GLOBAL_LOAD, DMA_LOAD_QUAL>(0, m_grid.begin());
  }

  template<bool DMA_GLOBAL_LOAD, int DMA_LOAD_QUAL, int DMA_STORE_QUAL>
  __device__ __forceinline__ void wait_xfer_finish(void* __restrict__ dst_ptr)
  {
    HIPDMA_ASSERT((reinterpret_cast<uintptr_t>(dst_ptr) % ALIGNMENT) == 0);
    HIPDMA_ASSERT(!hipdma::detail::store_is_swizzled(DMA_STORE_QUAL) || (m_grid.E % ALIGNMENT) == 0);
    if constexpr (DO_SYNC) CudaDMA::wait_for_dma_start();
    static_assert(!hipdma::detail::store_is_swizzled(DMA_STORE_QUAL) || (BYTES_PER_ELMT % ALIGNMENT) == 0,
                  "swizzled LDS rows must be whole chunks");
    if (use_direct<DMA_STORE_QUAL>()) {
      if constexpr (hipdma::detail::store_is_direct(DMA_STORE_QUAL)) {
        static_assert(!hipdma::detail::store_is_direct(DMA_STORE_QUAL) || DMA_GLOBAL_LOAD,
                      "STORE_LDS_DIRECT needs a global source");
        direct_all<hipdma::detail::store_is_swizzled(DMA_STORE_QUAL), DMA_LOAD_QUAL>((char*)dst_ptr);
      }
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

  // ---- direct-to-LDS transfers kept in flight (an addition of this library) ----
  // The two-phase calls cannot request a STORE_LDS_DIRECT transfer before the handshake says the
  // buffer is free, so with them a DMA wavefront has one direct transfer in flight at a time.  A
  // kernel that does its own hand-off (a sync-only object, src/examples usage of cudaDMACustom)
  // can keep several in flight: issue_direct() requests the whole transfer into a buffer the
  // caller knows to be free and returns; the loads of a wavefront land in issue order, so
  // hipdma::wait_direct_loads<YOUNGER>() waits for this transfer while the YOUNGER loads issued
  // after it (loads_per_thread() of each later transfer) stay in flight.  Needs the shape the
  // direct path needs (direct_ready()); neither call touches the handshake.
  template<int DMA_STORE_QUAL = STORE_LDS_DIRECT, int DMA_LOAD_QUAL = LOAD_CACHE_ALL>
  __device__ __forceinline__ void issue_direct(const void* __restrict__ src_ptr, void* __restrict__ dst_ptr)
  {
    static_assert(hipdma::detail::store_is_direct(DMA_STORE_QUAL), "issue_direct takes one of the STORE_LDS_DIRECT qualifiers");
    static_assert(ALIGNMENT == 16 || ALIGNMENT == 4, "global_load_lds moves 4 or 16 bytes per lane");
    HIPDMA_ASSERT(direct_ready());
    m_src = (const char*)src_ptr;
    issue_direct_rounds<hipdma::detail::store_is_swizzled(DMA_STORE_QUAL), false, DMA_LOAD_QUAL>((char*)dst_ptr);
  }
  // A part of the same transfer: the loads of rounds [first_round, first_round + num_rounds) of the
  // loads_per_thread() a thread issues for it, for callers that spread the loads of a transfer between other
  // instructions (a wavefront that also computes holds up its own work while it issues loads back to back:
  // the address unit takes a wavefront's 16-byte loads at one per sixteen cycles).
  // With WHOLE_ROWS the caller vouches for the shape the scalar-base loads need (the DMA threads cover whole rows,
  // a non-negative source stride, a round's rows within 4 GiB): only that form is compiled, and the few scalar
  // instructions of a load fit under one matrix instruction.
  template<int DMA_STORE_QUAL = STORE_LDS_DIRECT, bool WHOLE_ROWS = false, int DMA_LOAD_QUAL = LOAD_CACHE_ALL>
  __device__ __forceinline__ void issue_direct_part(const void* __restrict__ src_ptr, void* __restrict__ dst_ptr,
                                                    const int first_round, const int num_rounds)
  {
    static_assert(hipdma::detail::store_is_direct(DMA_STORE_QUAL), "issue_direct_part takes one of the STORE_LDS_DIRECT qualifiers");
    static_assert(ALIGNMENT == 16 || ALIGNMENT == 4, "global_load_lds moves 4 or 16 bytes per lane");
    HIPDMA_ASSERT(direct_ready());
    m_src = (const char*)src_ptr;
    issue_direct_rounds<hipdma::detail::store_is_swizzled(DMA_STORE_QUAL), WHOLE_ROWS, DMA_LOAD_QUAL>((char*)dst_ptr, first_round, first_round + num_rounds);
  }
  // True when this object's shape can use global_load_lds (whole chunks, whole wavefronts, rows of
  // at least a wavefront of chunks or unpadded power-of-two rows).
  __device__ __forceinline__ bool direct_ready() const { return use_direct<STORE_LDS_DIRECT>(); }
  // Loads each thread issues per transfer on the direct path (the unit of wait_direct_loads).
  __host__ __device__ static constexpr int loads_per_thread()
  { return hipdma::GridPlan(ALIGNMENT, BYTES_PER_THREAD, BYTES_PER_ELMT, DMA_THREADS, NUM_ELMTS).rounds; }

private:
  __device__ __forceinline__ static int threads_or_block(const int n) { return (n <= 0) ? int(blockDim.x) : n; }

  __device__ __forceinline__ void init(const int e, const int n, const int t, const int start,
                                       const int src_stride, const int dst_stride)
  {
    HIPDMA_ASSERT(e >= 0 && (e % 4) == 0 && n >= 0);
    HIPDMA_ASSERT(t > 0 && (t % HIPDMA_WAVE_SIZE) == 0);
    HIPDMA_ASSERT((src_stride % ALIGNMENT) == 0 && (dst_stride % ALIGNMENT) == 0);
    m_grid.init(ALIGNMENT, MAX_LDS, e, n, t, int(threadIdx.x) - start);
    m_src_stride = src_stride;
    m_dst_stride = dst_stride;
  }

  // The direct path needs the 64 lanes of a wavefront to land on 64 consecutive
  // chunks of LDS: rows at least one wavefront wide, or unpadded rows packed
  // back to back.  Otherwise the register path is taken.
  template<int STORE_QUAL>
  __device__ __forceinline__ bool use_direct() const
  {
    if constexpr (hipdma::detail::store_is_direct(STORE_QUAL) && (ALIGNMENT == 16 || ALIGNMENT == 4))
      return (m_grid.last_bytes == ALIGNMENT) && ((m_grid.T % HIPDMA_WAVE_SIZE) == 0) &&
             ((m_grid.W >= HIPDMA_WAVE_SIZE) ||
              ((m_grid.W == m_grid.LPE) && (m_dst_stride == m_grid.E)));
    else
      return false;
  }

  template<bool GLOBAL_LOAD, int LOAD_QUAL>
  __device__ __forceinline__ void load_step(const int step, hipdma::detail::GridCursor cur)
  {
    using namespace hipdma::detail;
    if constexpr (GLOBAL_LOAD) {
      // When a round moves every thread down whole rows (the threads cover whole rows: dcol == 0), the address
      // splits into a part that is the same for all threads and changes per load (round * drow rows down) and a
      // part per thread that never changes (its row and column of round 0).  Written that way the thread keeps
      // one offset instead of a 64-bit address per load in flight, and the per-load part is scalar arithmetic.
      if (m_grid.dcol == 0) {
        const long long lane_part = (long long)(m_grid.row0 * m_src_stride + m_grid.col0 * ALIGNMENT);
#pragma unroll
        for (int k = 0; k < MAX_LDS; ++k) {
          if (m_grid.live(step * MAX_LDS + k, cur)) {
            // the same value in every lane (object parameters are); saying so keeps it in scalar registers
            const long long rows_down = (long long)((step * MAX_LDS + k) * m_grid.drow) * (long long)m_src_stride;
            const long long uniform = (long long)(
                ((unsigned long long)__builtin_amdgcn_readfirstlane((unsigned)((unsigned long long)rows_down >> 32)) << 32) |
                (unsigned long long)__builtin_amdgcn_readfirstlane((unsigned)(unsigned long long)rows_down));
            load_chunk<ALIGNMENT, ALIGNMENT, GLOBAL_LOAD, LOAD_QUAL>(m_buf[k], m_src + uniform + lane_part,
                                                                     m_grid.chunk_bytes(ALIGNMENT, cur));
          }
          m_grid.advance(cur);
        }
        return;
      }
    }
#pragma unroll
    for (int k = 0; k < MAX_LDS; ++k) {
      if (m_grid.live(step * MAX_LDS + k, cur))
        load_chunk<ALIGNMENT, ALIGNMENT, GLOBAL_LOAD, LOAD_QUAL>(
            m_buf[k], m_src + cur.row * m_src_stride + cur.col * ALIGNMENT, m_grid.chunk_bytes(ALIGNMENT, cur));
      m_grid.advance(cur);
    }
  }

  // Drains the registers of `step` and leaves `cur` at the first slot of the next step.
  template<int STORE_QUAL>
  __device__ __forceinline__ void store_step(char* dst, const int step, hipdma::detail::GridCursor& cur) const
  {
    using namespace hipdma::detail;
#pragma unroll
    for (int k = 0; k < MAX_LDS; ++k) {
      if (m_grid.live(step * MAX_LDS + k, cur))
        store_chunk<ALIGNMENT, ALIGNMENT, STORE_QUAL>(
            m_buf[k], dst + cur.row * m_dst_stride + lds_col<store_is_swizzled(STORE_QUAL)>(cur) * ALIGNMENT,
            m_grid.chunk_bytes(ALIGNMENT, cur));
      m_grid.advance(cur);
    }
  }

  // Chunk position inside the LDS row for the chunk at cursor c.
  template<bool SWIZZLE>
  __device__ __forceinline__ int lds_col(const hipdma::detail::GridCursor& c) const
  {
    if constexpr (SWIZZLE) return hipdma::swizzled_chunk(c.row, c.col, m_grid.LPE, ALIGNMENT);
    else return c.col;
  }

  // Lane L of a wavefront always lands on LDS chunk (base + L); with SWIZZLE the lane
  // fetches the source chunk that belongs at its landing position instead.
  template<bool SWIZZLE, int LOAD_QUAL>
  __device__ __forceinline__ void direct_all(char* dst)
  {
    issue_direct_rounds<SWIZZLE, false, LOAD_QUAL>(dst);
    hipdma::detail::wait_lds_direct();
  }

  template<bool SWIZZLE, bool WHOLE_ROWS = false, int LOAD_QUAL = LOAD_CACHE_ALL>
  __device__ __forceinline__ void issue_direct_rounds(char* dst, const int first = 0, const int end = 0x7fffffff)
  {
    using namespace hipdma::detail;
    const int lane = lane_id();
    // When a round moves every thread down whole rows and a round's rows span less than 4 GiB of the
    // source, a load is written as "scalar base + 32-bit lane offset": the base (source, rows of the
    // round) and the LDS address are scalar arithmetic, the lane offsets do not change from one transfer
    // to the next, and no vector ALU instruction is left between two loads.  It matters next to compute
    // wavefronts that issue matrix instructions back to back: a vector ALU instruction of the DMA
    // wavefront then waits for a gap between those.
    const bool whole_rows = (m_grid.dcol == 0) && (m_src_stride >= 0) &&
        ((long long)m_grid.drow * (long long)m_src_stride + (long long)m_grid.W * ALIGNMENT <= 0xffffffffLL);
    if constexpr (WHOLE_ROWS) HIPDMA_ASSERT(whole_rows);
    if (WHOLE_ROWS || whole_rows) {
      const unsigned lane_row = (unsigned)(m_grid.row0 * m_src_stride);
      // The pointers, strides and rows per round are the same in every lane by the contract of the call;
      // the compiler cannot always tell, so they are pinned to scalar registers once per transfer.
      const char* const base = scalar_ptr(m_src);
      const long long round_src = (long long)(int)scalar_u32((unsigned)m_grid.drow) * (long long)(int)scalar_u32((unsigned)m_src_stride);
      const unsigned round_lds = scalar_u32((unsigned)(m_grid.drow * m_dst_stride));
      // where lane 0 of this wavefront lands in round 0 (lane L lands L chunks further on)
      const unsigned lds0 = scalar_u32((unsigned)(size_t)(HIPDMA_LDS_AS char*)dst) +
                            scalar_u32((unsigned)(m_grid.row0 * m_dst_stride + (m_grid.col0 - lane) * ALIGNMENT));
      GridCursor cur = m_grid.begin();
      for (int r = 0; r < m_grid.rounds; ++r) {
        if (r >= first && r < end && m_grid.live(r, cur)) {
          const unsigned lane_off = lane_row + (unsigned)(lds_col<SWIZZLE>(cur) * ALIGNMENT);
          if constexpr (ALIGNMENT == 16 || ALIGNMENT == 4)
            load_to_lds_scalar_base<ALIGNMENT, LOAD_QUAL>(base + r * round_src, lane_off, lds0 + r * round_lds);
        }
        m_grid.advance(cur);
      }
      return;
    }
    GridCursor cur = m_grid.begin();
    for (int r = 0; r < m_grid.rounds; ++r) {
      if (r >= first && r < end && m_grid.live(r, cur)) {
        const int lds_off = cur.row * m_dst_stride + cur.col * ALIGNMENT;
        if constexpr (ALIGNMENT == 16 || ALIGNMENT == 4)
          load_to_lds<ALIGNMENT, LOAD_QUAL>(m_src + cur.row * m_src_stride + lds_col<SWIZZLE>(cur) * ALIGNMENT,
                                 dst + (lds_off - lane * ALIGNMENT));
      }
      m_grid.advance(cur);
    }
  }

private:
  hipdma::detail::GridState m_grid;
  int m_src_stride;
  int m_dst_stride;
  const char* m_src;
  chunk_t m_buf[MAX_LDS];
};

namespace hipdma {
// Waits until every direct-to-LDS load of the calling wavefront except the YOUNGER most recent
// ones has landed (see CudaDMAStrided::issue_direct).
template<int YOUNGER>
__device__ __forceinline__ void wait_direct_loads() { detail::wait_lds_direct_but<YOUNGER>(); }
}  // namespace hipdma

// Host-side planner report (include/cudaDMAv2.h:3208-3493).
template<bool DO_SYNC>
class CudaDMAStrided<DO_SYNC, 0, 0, 0, 0, 0> {
public:
  __host__ static void diagnose(const int ALIGNMENT, const int BYTES_PER_THREAD, const int BYTES_PER_ELMT,
                                const int DMA_THREADS, const int NUM_ELMTS, const bool FULL_TEMPLATE,
                                const bool verbose = false)
  {
    const hipdma::GridPlan p(ALIGNMENT, BYTES_PER_THREAD, BYTES_PER_ELMT, DMA_THREADS, NUM_ELMTS);
    fprintf(stdout, "==== CudaDMAStrided plan (gfx950, 64-lane wavefronts) ====\n");
    fprintf(stdout, "  ALIGNMENT %d  BYTES_PER_THREAD %d  BYTES_PER_ELMT %d  DMA_THREADS %d (%d wavefronts)  NUM_ELMTS %d  %s\n",
            ALIGNMENT, BYTES_PER_THREAD, BYTES_PER_ELMT, DMA_THREADS,
            (DMA_THREADS + HIPDMA_WAVE_SIZE - 1) / HIPDMA_WAVE_SIZE, NUM_ELMTS,
            FULL_TEMPLATE ? "compile-time parameters" : "run-time parameters");
    if (p.slots_per_row <= HIPDMA_WAVE_SIZE)
      fprintf(stdout, "  layout: %d loads per element, %d lanes per element, %d elements per wavefront load\n",
              p.loads_per_elmt, p.slots_per_row, HIPDMA_WAVE_SIZE / p.slots_per_row);
    else
      fprintf(stdout, "  layout: %d loads per element, %d wavefront loads per element\n",
              p.loads_per_elmt, p.slots_per_row / HIPDMA_WAVE_SIZE);
    if (p.slots_per_row != p.loads_per_elmt)
      fprintf(stdout, "  %d of every %d lanes idle: element size is not a power-of-two (or 64x) number of loads\n",
              p.slots_per_row - p.loads_per_elmt, p.slots_per_row);
    fprintf(stdout, "  loads per thread: %d, registers hold %d -> %d step(s)\n", p.rounds, p.loads_per_step, p.total_steps);
    if (p.total_steps <= 1)
      fprintf(stdout, "  single step: every load is issued before the handshake wait.\n");
    else
      fprintf(stdout, "  multiple steps: to reach one step use BYTES_PER_THREAD >= %d or DMA_THREADS >= %d\n",
              p.rounds * ALIGNMENT,
              hipdma::detail::round_up(hipdma::detail::ceil_div(NUM_ELMTS * p.slots_per_row, p.loads_per_step), HIPDMA_WAVE_SIZE));
    if (verbose)
      fprintf(stdout, "  loads_per_elmt %d  slots_per_row %d  last_chunk_bytes %d  rounds %d  sure_rounds %d  total_steps %d\n",
              p.loads_per_elmt, p.slots_per_row, p.last_chunk_bytes, p.rounds, p.sure_rounds, p.total_steps);
    fflush(stdout);
  }
};
