// CudaDMAHalo: transfer of the ring of ghost cells around a dimx x dimy tile.
//
// The reference only has the older cudaDMAHalo<ELMT_TYPE,RADIUS,CORNERS,ALIGNMENT>
// (include/cudaDMA.h:3653-4156); this is the same transfer with the template
// parameters and the two-phase calls of the other objects, plus a class with
// the old name and constructor on top of it.  Behaviour followed:
//   * both origins point at the first interior cell of the tile
//     (src/tests/test_halo/cudaDMA_test_halo.cu:196-197);
//   * RADIUS rows above and RADIUS rows below the tile are moved, dimx cells
//     wide, or dimx + 2*RADIUS wide with CORNERS (include/cudaDMA.h:3616,3720-3727);
//   * RADIUS cells left and right of each of the dimy tile rows are moved
//     (include/cudaDMA.h:3746-3749);
//   * the source row pitch is `pitch` cells, the destination row pitch is
//     dimx + 2*RADIUS cells (include/cudaDMA.h:3718-3719) unless the constructor is
//     given a wider one (`dst_pitch`, an addition of this library: a consumer that
//     reads the plane down its columns picks the pitch that keeps those reads off
//     each other's LDS banks, as the strided classes let it with dst_stride);
//   * the interior is not touched (src/tests/test_halo/cudaDMA_test_halo.cu:91-164).
//
// Work split (wave64): two slot grids laid end to end and dealt round-robin to
// the DMA threads, thread t owning slots t, t+T, ...
//   rows : 2*RADIUS rows of ceil(row_bytes / XR) chunks, row padded to W1 slots
//   sides: 2*dimy strips of (RADIUS*BYTES_PER_ELMT / XS) chunks, strip padded to W2 slots
// ALIGNMENT is what both origins, both pitches in bytes, dimx*BYTES_PER_ELMT
// and 2*RADIUS*BYTES_PER_ELMT (hence the default destination pitch) are multiples of.
// Rows without corners start on such a boundary and move in chunks of XR =
// ALIGNMENT bytes; a strip, and a row with corners, starts RADIUS*BYTES_PER_ELMT
// bytes off one and moves in pieces of XS = the largest power of two (at most
// ALIGNMENT) dividing RADIUS*BYTES_PER_ELMT.
#pragma once

#include "grid.hpp"

namespace hipdma {
namespace detail {

// Where slot s of a halo transfer lives.  Offsets are bytes relative to the origins.
struct HaloSlot {
  bool live;
  bool is_row;     // row chunk (moved in XR pieces) or side chunk (XS pieces)
  int src_off, dst_off, nbytes;
};

// Geometry of one halo transfer; shared by the device object and the host-side checks.
template<int ALIGNMENT, int BYTES_PER_ELMT, int RADIUS, bool CORNERS>
struct HaloGeom {
  static constexpr int SIDE_BYTES = RADIUS * BYTES_PER_ELMT;
  static constexpr int XS = pow2_divisor(SIDE_BYTES, ALIGNMENT);   // side move size
  static constexpr int XR = CORNERS ? XS : ALIGNMENT;              // row move size
  static constexpr int LPS = SIDE_BYTES / XS;
  static constexpr int W2 = GridPlan::slots(LPS);
  int dimx_bytes, dimy, src_pitch, dst_pitch, row_bytes, lpr, w1, s1, total;

  // dst_pitch_cells <= 0 selects the reference's destination pitch, dimx + 2*RADIUS cells.
  __host__ __device__ __forceinline__ void init(const int dimx, const int dimy_, const int pitch,
                                                const int dst_pitch_cells = 0)
  {
    dimx_bytes = dimx * BYTES_PER_ELMT;
    dimy = dimy_;
    src_pitch = pitch * BYTES_PER_ELMT;
    dst_pitch = (dst_pitch_cells > 0 ? dst_pitch_cells : dimx + 2 * RADIUS) * BYTES_PER_ELMT;
    row_bytes = dimx_bytes + (CORNERS ? 2 * SIDE_BYTES : 0);
    lpr = ceil_div(row_bytes, XR);
    w1 = GridPlan::slots(lpr);
    s1 = round_up(2 * RADIUS * w1, HIPDMA_WAVE_SIZE);
    total = s1 + 2 * dimy * W2;
  }
  // What the slots [round*threads, (round+1)*threads) of one round are:
  //   0  all of them live row chunks, 1  all of them live side chunks, 2  a mix, or some idle.
  // With compile-time tile size and thread count this folds to a constant, which
  // turns the whole transfer into straight-line code: no per-lane predication,
  // so loads of later transfers can stay in flight across it.
  __host__ __device__ __forceinline__ int round_kind(const int round, const int threads) const
  {
    const int lo = round * threads, hi = lo + threads;
    if ((w1 == lpr) && (hi <= 2 * RADIUS * w1)) return 0;
    if ((W2 == LPS) && (lo >= s1) && (hi <= total)) return 1;
    return 2;
  }
  __host__ __device__ __forceinline__ HaloSlot decode(const int s) const
  {
    HaloSlot r;
    r.is_row = s < s1;
    if (r.is_row) {
      const int row = s / w1;
      const int c = s - row * w1;
      r.live = (row < 2 * RADIUS) && (c < lpr);
      const int y = (row < RADIUS) ? (row - RADIUS) : (dimy + row - RADIUS);
      const int x = c * XR - (CORNERS ? SIDE_BYTES : 0);
      r.nbytes = (c == lpr - 1) ? (row_bytes - c * XR) : XR;
      r.src_off = y * src_pitch + x;
      r.dst_off = y * dst_pitch + x;
    } else {
      const int s2 = s - s1;
      const int strip = s2 / W2;
      const int c = s2 - strip * W2;
      r.live = (strip < 2 * dimy) && (c < LPS);
      const int y = strip >> 1;
      const int x = ((strip & 1) ? dimx_bytes : -SIDE_BYTES) + c * XS;
      r.nbytes = XS;
      r.src_off = y * src_pitch + x;
      r.dst_off = y * dst_pitch + x;
    }
    return r;
  }
};

}  // namespace detail
}  // namespace hipdma

template<bool DO_SYNC = false, int ALIGNMENT = 0, int BYTES_PER_THREAD = 4 * ALIGNMENT, int BYTES_PER_ELMT = 0,
         int DMA_THREADS = 0, int RADIUS = 0, bool CORNERS = false, int DIMX = 0, int DIMY = 0>
class CudaDMAHalo : public CudaDMA {
  static_assert(ALIGNMENT == 4 || ALIGNMENT == 8 || ALIGNMENT == 16, "ALIGNMENT must be 4, 8 or 16");
  static_assert((BYTES_PER_THREAD / ALIGNMENT) > 0, "BYTES_PER_THREAD must hold at least one chunk");
  static_assert((BYTES_PER_THREAD % ALIGNMENT) == 0, "BYTES_PER_THREAD must be a multiple of ALIGNMENT");
  static_assert(BYTES_PER_ELMT > 0 && (BYTES_PER_ELMT % 4) == 0, "BYTES_PER_ELMT is the size of one cell");
  static_assert(RADIUS > 0, "RADIUS must be positive");
  static_assert((2 * RADIUS * BYTES_PER_ELMT) % ALIGNMENT == 0,
                "the destination pitch (dimx+2*RADIUS cells) must keep ALIGNMENT: lower ALIGNMENT");
  static_assert((DIMX == 0) == (DIMY == 0), "give both tile dimensions at compile time or neither");
  static constexpr int LEVEL = (DMA_THREADS == 0) ? 1 : (DIMX == 0) ? 2 : 3;
  static constexpr int MAX_LDS = BYTES_PER_THREAD / ALIGNMENT;
  typedef hipdma::detail::HaloGeom<ALIGNMENT, BYTES_PER_ELMT, RADIUS, CORNERS> geom_t;
  static constexpr int XS = geom_t::XS;
  static constexpr int XR = geom_t::XR;
  typedef typename hipdma::detail::chunk_of<ALIGNMENT>::type chunk_t;
  template<bool C> using when = typename std::enable_if<C, int>::type;
public:
  // ---- warp-specialised constructors; pitch is the source row pitch in cells ----
  template<int L = LEVEL, bool S = DO_SYNC, when<(L == 1) && S> = 0>
  __device__ __forceinline__ CudaDMAHalo(const int dmaID, const int num_dma_threads, const int num_compute_threads,
                                         const int dma_threadIdx_start, const int dimx, const int dimy,
                                         const int pitch, const int dst_pitch = 0)
    : CudaDMA(dmaID, num_dma_threads, num_compute_threads, dma_threadIdx_start)
  { init(num_dma_threads, dma_threadIdx_start, dimx, dimy, pitch, dst_pitch); }
  template<int L = LEVEL, bool S = DO_SYNC, when<(L == 2) && S> = 0>
  __device__ __forceinline__ CudaDMAHalo(const int dmaID, const int num_compute_threads,
                                         const int dma_threadIdx_start, const int dimx, const int dimy,
                                         const int pitch, const int dst_pitch = 0)
    : CudaDMA(dmaID, DMA_THREADS, num_compute_threads, dma_threadIdx_start)
  { init(DMA_THREADS, dma_threadIdx_start, dimx, dimy, pitch, dst_pitch); }
  template<int L = LEVEL, bool S = DO_SYNC, when<(L == 3) && S> = 0>
  __device__ __forceinline__ CudaDMAHalo(const int dmaID, const int num_compute_threads,
                                         const int dma_threadIdx_start, const int pitch, const int dst_pitch = 0)
    : CudaDMA(dmaID, DMA_THREADS, num_compute_threads, dma_threadIdx_start)
  { init(DMA_THREADS, dma_threadIdx_start, DIMX, DIMY, pitch, dst_pitch); }

  // ---- constructors of the form that is not warp-specialised ----
  template<int L = LEVEL, bool S = DO_SYNC, when<(L == 1) && !S> = 0>
  __device__ __forceinline__ CudaDMAHalo(const int dimx, const int dimy, const int pitch,
                                         const int num_dma_threads = 0, const int dma_threadIdx_start = 0,
                                         const int dst_pitch = 0)
    : CudaDMA(hipdma::detail::no_sync_t(), threads_or_block(num_dma_threads), dma_threadIdx_start)
  { init(threads_or_block(num_dma_threads), dma_threadIdx_start, dimx, dimy, pitch, dst_pitch); }
  template<int L = LEVEL, bool S = DO_SYNC, when<(L == 2) && !S> = 0>
  __device__ __forceinline__ CudaDMAHalo(const int dimx, const int dimy, const int pitch,
                                         const int dma_threadIdx_start = 0, const int dst_pitch = 0)
    : CudaDMA(hipdma::detail::no_sync_t(), DMA_THREADS, dma_threadIdx_start)
  { init(DMA_THREADS, dma_threadIdx_start, dimx, dimy, pitch, dst_pitch); }
  template<int L = LEVEL, bool S = DO_SYNC, when<(L == 3) && !S> = 0>
  __device__ __forceinline__ CudaDMAHalo(const int pitch, const int dma_threadIdx_start = 0, const int dst_pitch = 0)
    : CudaDMA(hipdma::detail::no_sync_t(), DMA_THREADS, dma_threadIdx_start)
  { init(DMA_THREADS, dma_threadIdx_start, DIMX, DIMY, pitch, dst_pitch); }

public:
  __device__ __forceinline__ void execute_dma(const void* __restrict__ src_origin, void* __restrict__ dst_origin)
  { execute_dma<false, LOAD_CACHE_ALL, STORE_WRITE_BACK>(src_origin, dst_origin); }
  __device__ __forceinline__ void start_xfer_async(const void* __restrict__ src_origin)
  { start_xfer_async<false, LOAD_CACHE_ALL, STORE_WRITE_BACK>(src_origin); }
  __device__ __forceinline__ void wait_xfer_finish(void* __restrict__ dst_origin)
  { wait_xfer_finish<false, LOAD_CACHE_ALL, STORE_WRITE_BACK>(dst_origin); }
  // Same transfer without the handshake (include/cudaDMA.h:3857-3860).
  __device__ __forceinline__ void execute_dma_no_sync(const void* __restrict__ src_origin, void* __restrict__ dst_origin)
  {
    start_xfer_async<false, LOAD_CACHE_ALL, STORE_WRITE_BACK>(src_origin);
    drain<false, LOAD_CACHE_ALL, STORE_WRITE_BACK>((char*)dst_origin);
  }

  template<bool DMA_GLOBAL_LOAD>
  __device__ __forceinline__ void execute_dma(const void* __restrict__ src_origin, void* __restrict__ dst_origin)
  { execute_dma<DMA_GLOBAL_LOAD, LOAD_CACHE_ALL, STORE_WRITE_BACK>(src_origin, dst_origin); }
  template<bool DMA_GLOBAL_LOAD>
  __device__ __forceinline__ void start_xfer_async(const void* __restrict__ src_origin)
  { start_xfer_async<DMA_GLOBAL_LOAD, LOAD_CACHE_ALL, STORE_WRITE_BACK>(src_origin); }
  template<bool DMA_GLOBAL_LOAD>
  __device__ __forceinline__ void wait_xfer_finish(void* __restrict__ dst_origin)
  { wait_xfer_finish<DMA_GLOBAL_LOAD, LOAD_CACHE_ALL, STORE_WRITE_BACK>(dst_origin); }

  template<bool DMA_GLOBAL_LOAD, int DMA_LOAD_QUAL, int DMA_STORE_QUAL>
  __device__ __forceinline__ void execute_dma(const void* __restrict__ src_origin, void* __restrict__ dst_origin)
  {
    start_xfer_async<DMA_GLOBAL_LOAD, DMA_LOAD_QUAL, DMA_STORE_QUAL>(src_origin);
    wait_xfer_finish<DMA_GLOBAL_LOAD, DMA_LOAD_QUAL, DMA_STORE_QUAL>(dst_origin);
  }
  template<bool DMA_GLOBAL_LOAD, int DMA_LOAD_QUAL, int DMA_STORE_QUAL>
  __device__ __forceinline__ void start_xfer_async(const void* __restrict__ src_origin)
  {
    static_assert(DMA_STORE_QUAL != STORE_LDS_DIRECT, "the halo ring is too ragged for the direct path");
    static_assert(!hipdma::detail::store_is_swizzled(DMA_STORE_QUAL), "swizzled LDS rows are a CudaDMAStrided layout");
    HIPDMA_ASSERT((reinterpret_cast<uintptr_t>(src_origin) % ALIGNMENT) == 0);
    m_src = (const char*)src_origin;
    pass<true, DMA_GLOBAL_LOAD, DMA_LOAD_QUAL, DMA_STORE_QUAL>(0, nullptr);
  }
  // Second half of a two-phase transfer without the handshake (the two-phase
  // counterpart of execute_dma_no_sync).
  template<bool DMA_GLOBAL_LOAD, int DMA_LOAD_QUAL, int DMA_STORE_QUAL>
  __device__ __forceinline__ void drain_no_sync(void* __restrict__ dst_origin)
  { drain<DMA_GLOBAL_LOAD, DMA_LOAD_QUAL, DMA_STORE_QUAL>((char*)dst_origin); }
  template<bool DMA_GLOBAL_LOAD, int DMA_LOAD_QUAL, int DMA_STORE_QUAL>
  __device__ __forceinline__ void wait_xfer_finish(void* __restrict__ dst_origin)
  {
    if constexpr (DO_SYNC) CudaDMA::wait_for_dma_start();
    drain<DMA_GLOBAL_LOAD, DMA_LOAD_QUAL, DMA_STORE_QUAL>((char*)dst_origin);
    if constexpr (DO_SYNC) CudaDMA::finish_async_dma();
  }

private:
  __device__ __forceinline__ static int threads_or_block(const int n) { return (n <= 0) ? int(blockDim.x) : n; }

  __device__ __forceinline__ void init(const int threads, const int start, const int dimx, const int dimy,
                                       const int pitch, const int dst_pitch)
  {
    using namespace hipdma::detail;
    HIPDMA_ASSERT(threads > 0 && (threads % HIPDMA_WAVE_SIZE) == 0);
    HIPDMA_ASSERT(dimx > 0 && dimy > 0 && pitch >= dimx + 2 * RADIUS);
    HIPDMA_ASSERT(((pitch * BYTES_PER_ELMT) % ALIGNMENT) == 0);
    HIPDMA_ASSERT(dst_pitch <= 0 || (dst_pitch >= dimx + 2 * RADIUS && ((dst_pitch * BYTES_PER_ELMT) % ALIGNMENT) == 0));
    m_tid = int(threadIdx.x) - start;
    m_threads = threads;
    m_geom.init(dimx, dimy, pitch, dst_pitch);
    m_steps = ceil_div(ceil_div(m_geom.total, threads), MAX_LDS);
  }

  template<bool GLOBAL_LOAD, int LOAD_QUAL, int STORE_QUAL>
  __device__ __forceinline__ void drain(char* dst)
  {
    pass<false, GLOBAL_LOAD, LOAD_QUAL, STORE_QUAL>(0, dst);
    for (int step = 1; step < m_steps; ++step) {
      pass<true, GLOBAL_LOAD, LOAD_QUAL, STORE_QUAL>(step, nullptr);
      pass<false, GLOBAL_LOAD, LOAD_QUAL, STORE_QUAL>(step, dst);
    }
  }

  // One sweep over the slots of `step`: loads into the registers or stores out of them.
  template<bool IS_LOAD, bool GLOBAL_LOAD, int LOAD_QUAL, int STORE_QUAL>
  __device__ __forceinline__ void pass(const int step, char* dst)
  {
    using namespace hipdma::detail;
#pragma unroll
    for (int k = 0; k < MAX_LDS; ++k) {
      const int round = step * MAX_LDS + k;
      const int kind = m_geom.round_kind(round, m_threads);
      const HaloSlot slot = m_geom.decode(m_tid + round * m_threads);
      if (kind == 0) {
        move<IS_LOAD, XR, GLOBAL_LOAD, LOAD_QUAL, STORE_QUAL>(k, slot, dst, slot.nbytes);
      } else if (kind == 1) {
        move<IS_LOAD, XS, GLOBAL_LOAD, LOAD_QUAL, STORE_QUAL>(k, slot, dst, XS);
      } else if (slot.live) {
        if (slot.is_row) move<IS_LOAD, XR, GLOBAL_LOAD, LOAD_QUAL, STORE_QUAL>(k, slot, dst, slot.nbytes);
        else move<IS_LOAD, XS, GLOBAL_LOAD, LOAD_QUAL, STORE_QUAL>(k, slot, dst, XS);
      }
    }
  }

  template<bool IS_LOAD, int PIECE, bool GLOBAL_LOAD, int LOAD_QUAL, int STORE_QUAL>
  __device__ __forceinline__ void move(const int k, const hipdma::detail::HaloSlot& slot, char* dst, const int nbytes)
  {
    using namespace hipdma::detail;
    if constexpr (IS_LOAD)
      load_chunk<ALIGNMENT, PIECE, GLOBAL_LOAD, LOAD_QUAL>(m_buf[k], m_src + slot.src_off, nbytes);
    else
      store_chunk<ALIGNMENT, PIECE, STORE_QUAL>(m_buf[k], dst + slot.dst_off, nbytes);
  }

private:
  int m_tid, m_threads;
  geom_t m_geom;
  int m_steps;
  const char* m_src;
  chunk_t m_buf[MAX_LDS];
};

// The older interface: cudaDMAHalo<ELMT_TYPE,RADIUS,CORNERS,ALIGNMENT> with its
// single warp-specialised constructor (include/cudaDMA.h:3653-3692) and four
// loads in flight per thread (include/cudaDMA.h:30-31).
template<typename ELMT_TYPE, int RADIUS, bool CORNERS, int ALIGNMENT>
class cudaDMAHalo : public CudaDMAHalo<true, ALIGNMENT, 4 * ALIGNMENT, int(sizeof(ELMT_TYPE)), 0, RADIUS, CORNERS> {
  typedef CudaDMAHalo<true, ALIGNMENT, 4 * ALIGNMENT, int(sizeof(ELMT_TYPE)), 0, RADIUS, CORNERS> base_t;
public:
  __device__ __forceinline__ cudaDMAHalo(const int dmaID, const int num_dma_threads, const int num_compute_threads,
                                         const int dma_threadIdx_start, const int dimx, const int dimy,
                                         const int pitch)
    : base_t(dmaID, num_dma_threads, num_compute_threads, dma_threadIdx_start, dimx, dimy, pitch) {}
};
