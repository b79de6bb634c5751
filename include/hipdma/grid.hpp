// Slot grid shared by CudaDMAStrided and CudaDMAIndirect.
//
// A transfer of N elements of E bytes is cut into chunks of ALIGNMENT bytes.
// Rows are padded to W chunk slots so that the 64 lanes of a wavefront never
// straddle a row in a way that breaks coalescing:
//     chunks per element  LPE = ceil(E / ALIGNMENT)
//     W = next power of two >= LPE          when LPE <= 64  (several rows per wavefront)
//     W = LPE rounded up to a multiple of 64 otherwise      (several wavefronts per row)
// The N*W slots are dealt round-robin: DMA thread t owns slots t, t+T, t+2T, ...
// Slot s is chunk (row s / W, column s % W); it is live when column < LPE and
// row < N.  This one rule replaces the split / big / full regimes of
// include/cudaDMAv2.h:2988-3191: small elements share a wavefront, large ones
// are swept by all wavefronts, and no wavefront is left idle while work remains
// (the aim of include/cudaDMAv2.h:8267-8288).
// A thread holds MAX_LDS = BYTES_PER_THREAD/ALIGNMENT chunks in VGPRs; that
// many consecutive slots of a thread form a step.
#pragma once

#include "mem.hpp"

namespace hipdma {

struct GridPlan {
  int alignment, bytes_per_thread, bytes_per_elmt, dma_threads, num_elmts;
  int loads_per_elmt;     // LPE
  int slots_per_row;      // W
  int last_chunk_bytes;   // bytes in the last chunk of a row (4..ALIGNMENT)
  int rows_per_round;     // rows that all threads touch with one load each (0 when a row needs several rounds)
  int rounds;             // loads per thread for the whole transfer (upper bound, predicated)
  int loads_per_step;     // MAX_LDS
  int total_steps;
  int sure_rounds;        // leading rounds in which every slot of every thread is live
  __host__ __device__ constexpr GridPlan(int a, int bpt, int bpe, int t, int n)
    : alignment(a), bytes_per_thread(bpt), bytes_per_elmt(bpe), dma_threads(t), num_elmts(n),
      loads_per_elmt(detail::ceil_div(bpe, a)),
      slots_per_row(slots(detail::ceil_div(bpe, a))),
      last_chunk_bytes(bpe - (detail::ceil_div(bpe, a) - 1) * a),
      rows_per_round(t / slots(detail::ceil_div(bpe, a))),
      rounds(t > 0 ? detail::ceil_div(n * slots(detail::ceil_div(bpe, a)), t) : 0),
      loads_per_step(bpt / a),
      total_steps(t > 0 ? detail::ceil_div(detail::ceil_div(n * slots(detail::ceil_div(bpe, a)), t), bpt / a) : 0),
      sure_rounds((t > 0 && slots(detail::ceil_div(bpe, a)) == detail::ceil_div(bpe, a))
                      ? (n * slots(detail::ceil_div(bpe, a))) / t : 0) {}
  __host__ __device__ static constexpr int slots(int lpe)
  {
    return lpe <= 0 ? 1 : (lpe <= HIPDMA_WAVE_SIZE ? detail::pow2_ceil(lpe) : detail::round_up(lpe, HIPDMA_WAVE_SIZE));
  }
};

namespace detail {

// Per-thread cursor over the slots of a GridPlan.
struct GridCursor {
  int row, col;
};

struct GridState {
  int E, N, T, W, LPE, last_bytes;
  int row0, col0;        // slot of this thread in round 0
  int drow, dcol;        // slot advance per round
  int rounds, steps, sure_rounds;

  __host__ __device__ __forceinline__ void init(const int alignment, const int max_lds, const int e, const int n,
                                       const int t, const int tid)
  {
    E = e; N = n; T = t;
    LPE = ceil_div(e, alignment);
    W = GridPlan::slots(LPE);
    last_bytes = e - (LPE - 1) * alignment;
    row0 = tid / W;
    col0 = tid - row0 * W;
    drow = t / W;
    dcol = t - drow * W;
    rounds = ceil_div(n * W, t);
    steps = ceil_div(rounds, max_lds);
    sure_rounds = (W == LPE) ? (n * W) / t : 0;
  }
  __host__ __device__ __forceinline__ GridCursor begin() const { return GridCursor{row0, col0}; }
  __host__ __device__ __forceinline__ void advance(GridCursor& c) const
  {
    c.row += drow;
    c.col += dcol;
    if (c.col >= W) { c.col -= W; c.row += 1; }
  }
  // Round `round` is live for this thread at cursor c.
  __host__ __device__ __forceinline__ bool live(const int round, const GridCursor& c) const
  { return (round < sure_rounds) || ((c.row < N) && (c.col < LPE)); }
  __host__ __device__ __forceinline__ int chunk_bytes(const int alignment, const GridCursor& c) const
  { return (c.col == LPE - 1) ? last_bytes : alignment; }
};

}  // namespace detail
}  // namespace hipdma
