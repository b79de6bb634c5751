// hipDMA: wavefront-specialised DMA objects for AMD CDNA4 (gfx950).
//
// This header holds what every DMA object shares: the cache-policy enums, the
// producer/consumer handshake that stands in for CUDA named barriers, and the
// CudaDMA base class.  API contract followed: include/cudaDMAv2.h:50-63
// (qualifier enums) and include/cudaDMAv2.h:1316-1353 (class CudaDMA).
//
// Handshake design.  CDNA has no counterpart of `bar.sync id,count` /
// `bar.arrive id,count`.  Each dmaID owns two monotonically increasing 32-bit
// words in LDS:
//     full   counts lanes that have called finish_async_dma()
//     empty  counts lanes that have called start_async_dma()
// A signalling wavefront elects one lane which adds the number of active lanes
// with a single ds_add_u32; a waiting wavefront keeps a private phase number
// and polls with ds_read_b32 + s_sleep until the word reaches
// phase * (threads in the signalling group).  The words only ever grow, so a
// signal that nobody waits for (the "drain" wait_for_dma_start of
// src/perf/sequential/perf_sequential.cu:139) is harmless either way.
// Ordering: a workgroup-scope release fence before the add, a workgroup-scope
// acquire fence after the poll, over every address space, which is what
// bar.sync / bar.arrive give CUDA code: global memory written by one side
// before its signal is seen by the other side after its wait (LDS -> global
// transfers, CudaDMAIndirect<false>, a source produced by the compute threads).
// On gfx950 the wavefronts of a workgroup share one vector L1 that serves their
// requests in issue order, so both fences come out as s_waitcnt lgkmcnt(0) and
// cost what an LDS-only fence costs; what they add is that the compiler keeps
// global accesses on their side of the hand-off.  HIPDMA_LDS_ONLY_FENCE
// restricts both fences to the LDS address space for kernels that hand over
// LDS contents only and want the compiler free to move global accesses across.
// The *_direct forms of the DMA-side calls carry no fence at all (see below).
//
// A wait that gives up (HIPDMA_SPIN_LIMIT) records it: hipdma::status_words()
// of the translation unit get the bit HIPDMA_STATUS_WAIT_GAVE_UP and a count,
// which the host reads with hipdma::read_status() once the stream is idle.
//
// Requirements that differ from the CUDA original:
//   * DMA and compute groups are made of whole 64-lane wavefronts:
//     dma_threadIdx_start must be a multiple of 64 (a wavefront must not hold
//     both roles) and calls must be wavefront-uniform.
//   * Every thread of the workgroup constructs every warp-specialised object
//     before the roles branch: the constructor zeroes the two words and
//     executes one s_barrier.
#pragma once

#include <hip/hip_runtime.h>
#include <cstdio>
#include <type_traits>

#define HIPDMA_WAVE_SIZE 64
#define HIPDMA_MAX_DMA_IDS 16

#ifndef HIPDMA_SPIN_SLEEP
#define HIPDMA_SPIN_SLEEP 1
#endif
// A wait gives up after this many polls (about a second) and lets the wavefront
// run on, so that unbalanced start_async_dma / execute_dma counts end in a
// finished kernel, wrong data and a recorded failure (HIPDMA_STATUS_WAIT_GAVE_UP)
// instead of a hung GPU.  0 = wait for ever: the semantics of the reference's
// named barriers (include/cudaDMAv2.h:65-75), for kernels whose stages between
// two hand-offs can legitimately take longer than that.
#ifndef HIPDMA_SPIN_LIMIT
#define HIPDMA_SPIN_LIMIT (1 << 24)
#endif

// Bits of status word 0 (hipdma::read_status).
#define HIPDMA_STATUS_OK            0u
#define HIPDMA_STATUS_WAIT_GAVE_UP  1u   // a handshake wait ran into HIPDMA_SPIN_LIMIT: the kernel's results are void

// DEBUG_CUDADMA (the reference's switch, include/cudaDMAv2.h:1564-1576) turns the
// preconditions the objects rely on into device-side asserts: thread groups made of whole
// wavefronts, dmaID in range, sizes in multiples of 4 bytes, pointers and strides aligned
// to ALIGNMENT.  Without it nothing is checked, as in the reference.
#ifdef DEBUG_CUDADMA
#include <cassert>
#define HIPDMA_ASSERT(cond) assert(cond)
#else
#define HIPDMA_ASSERT(cond) ((void)0)
#endif

// Load cache policies (names follow include/cudaDMAv2.h:50-56).  On gfx950:
//   LOAD_CACHE_ALL / LOAD_CACHE_GLOBAL  plain load
//   LOAD_CACHE_STREAMING / _LAST_USE    non-temporal load (nt bit)
//   LOAD_CACHE_VOLATILE                 volatile load (sc0 sc1)
enum CudaDMALoadQualifier {
  LOAD_CACHE_ALL,
  LOAD_CACHE_GLOBAL,
  LOAD_CACHE_STREAMING,
  LOAD_CACHE_LAST_USE,
  LOAD_CACHE_VOLATILE,
};

// Store cache policies (names follow include/cudaDMAv2.h:58-63) plus two
// additions that only exist here:
//   STORE_LDS         the destination is known to be LDS: ds_write_b128 instead
//                     of a generic-address store
//   STORE_LDS_DIRECT  the destination is LDS and the data never visits a VGPR:
//                     global_load_lds_dwordx4 writes it straight into LDS.
//                     Needs a global source; nothing can be issued before the
//                     buffer is free, so start_xfer_async() only records the
//                     source and wait_xfer_finish() issues the loads.
//   STORE_LDS_SWIZZLE / STORE_LDS_DIRECT_SWIZZLE  (CudaDMAStrided) the same two,
//                     with the ALIGNMENT-byte chunks of every LDS row permuted:
//                     chunk c of row r lands at chunk hipdma::swizzled_chunk(r, c, n, ALIGNMENT)
//                     of the row, n = chunks per row.  Unpadded power-of-two rows
//                     (which is what the direct path needs) can then be read down a
//                     column without bank conflicts.  Rows must be whole chunks.
enum CudaDMAStoreQualifier {
  STORE_WRITE_BACK,
  STORE_CACHE_GLOBAL,
  STORE_CACHE_STREAMING,
  STORE_CACHE_WRITE_THROUGH,
  STORE_LDS,
  STORE_LDS_DIRECT,
  STORE_LDS_SWIZZLE,
  STORE_LDS_DIRECT_SWIZZLE,
};

namespace hipdma {
namespace detail {

typedef __attribute__((address_space(3))) unsigned lds_word_t;

// Failure record of this translation unit's kernels: word 0 collects HIPDMA_STATUS_* bits, word 1
// counts the waits that gave up.  File scope and internal linkage: every translation unit that
// includes the header has its own pair (device code is linked per translation unit), read through
// hipdma::read_status() compiled in that same translation unit.
static __device__ __attribute__((used)) unsigned g_status_words[2];

// Cold path of a wait that ran into HIPDMA_SPIN_LIMIT.
__device__ __forceinline__ void record_wait_gave_up()
{
  // one lane per wavefront reports: the count is in wavefronts
  const int lane = (int)__builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u));
  if (lane == __builtin_ctzll(__builtin_amdgcn_ballot_w64(true))) {
    __hip_atomic_fetch_or(&g_status_words[0], HIPDMA_STATUS_WAIT_GAVE_UP, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __hip_atomic_fetch_add(&g_status_words[1], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
}

// Two words per dmaID.  A function-local __shared__ array: every kernel that
// constructs a warp-specialised object gets its own 128-byte copy and the
// user never has to pass LDS for it.
__device__ __forceinline__ lds_word_t* sync_words()
{
  __shared__ unsigned words[2 * HIPDMA_MAX_DMA_IDS];
  return (lds_word_t*)words;
}

__device__ __forceinline__ void release_lds()
{
#ifdef HIPDMA_LDS_ONLY_FENCE
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
#else
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
#endif
}

__device__ __forceinline__ void acquire_lds()
{
#ifdef HIPDMA_LDS_ONLY_FENCE
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
#else
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
#endif
}

// The lowest active lane of the calling wavefront adds the number of active lanes to `word`.
// The election is scalar work (s_ff1 on exec, exec narrowed to that lane around the ds_add, one
// v_mov for the count): a vector ALU instruction of a wavefront that shares its SIMD with
// wavefronts issuing matrix instructions back to back waits for a gap between those, so every
// one saved in a hand-off shortens it by tens of cycles (measured in the GEMM workload: a DMA
// wavefront with three vector ALU instructions per load issued a load every 175 cycles).
__device__ __forceinline__ void add_active_lanes(lds_word_t* word)
{
  const unsigned addr = (unsigned)(size_t)word;
  const unsigned count = (unsigned)__builtin_popcountll(__builtin_amdgcn_ballot_w64(true));
  unsigned long long saved;
  unsigned first;
  asm volatile("s_mov_b64 %0, exec\n\t"
               "s_ff1_i32_b64 %1, exec\n\t"
               "s_lshl_b64 exec, 1, %1\n\t"
               "ds_add_u32 %2, %3\n\t"
               "s_mov_b64 exec, %0"
               : "=&s"(saved), "=&s"(first) : "v"(addr), "v"(count) : "memory", "scc");     // s_lshl_b64 writes SCC
}

// All active lanes of the calling wavefront arrive at `word`.
__device__ __forceinline__ void signal_word(lds_word_t* word)
{
  release_lds();
  add_active_lanes(word);
}

// Block until `word` has reached `target` (wrap-around safe).  Every lane reads the same word with
// the same instruction, so the comparison and the loop are scalar.
__device__ __forceinline__ void wait_word(lds_word_t* word, unsigned target)
{
  const unsigned want = __builtin_amdgcn_readfirstlane(target);
#if HIPDMA_SPIN_LIMIT > 0
  int polls = 0;
  while ((int)(__builtin_amdgcn_readfirstlane(__hip_atomic_load(word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP)) - want) < 0) {
    if (++polls >= HIPDMA_SPIN_LIMIT) { record_wait_gave_up(); break; }
    __builtin_amdgcn_s_sleep(HIPDMA_SPIN_SLEEP);
  }
#else
  while ((int)(__builtin_amdgcn_readfirstlane(__hip_atomic_load(word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP)) - want) < 0)
    __builtin_amdgcn_s_sleep(HIPDMA_SPIN_SLEEP);
#endif
  acquire_lds();
}

// The same two operations for a DMA wavefront that keeps direct-to-LDS loads in flight across
// the hand-off.  The compiler counts a global_load_lds as an LDS write: any fence or LDS access
// it can see makes it wait for ALL outstanding ones (s_waitcnt vmcnt(0)), which would leave
// one transfer in flight at a time.  These versions keep the LDS word accesses out of its sight
// (inline assembly) and carry no fence; the caller orders things itself: it waits for the loads
// it reports with s_waitcnt vmcnt(N) before signalling, and it only issues loads into a buffer
// after the wait for that buffer has returned (a control dependence the hardware honours).
__device__ __forceinline__ void signal_word_unfenced(lds_word_t* word)
{
  add_active_lanes(word);
}

__device__ __forceinline__ void wait_word_unfenced(lds_word_t* word, unsigned target)
{
  const unsigned addr = (unsigned)(size_t)word;
  const unsigned want = __builtin_amdgcn_readfirstlane(target);
  unsigned seen;
  for (int polls = 0;;) {
    asm volatile("ds_read_b32 %0, %1\n\ts_waitcnt lgkmcnt(0)" : "=v"(seen) : "v"(addr) : "memory");
    if ((int)(__builtin_amdgcn_readfirstlane(seen) - want) >= 0) break;
#if HIPDMA_SPIN_LIMIT > 0
    if (++polls >= HIPDMA_SPIN_LIMIT) { record_wait_gave_up(); break; }
#endif
    __builtin_amdgcn_s_sleep(HIPDMA_SPIN_SLEEP);
  }
}

struct no_sync_t {};

__host__ __device__ constexpr int ceil_div(int a, int b) { return (a + b - 1) / b; }
__host__ __device__ constexpr int round_up(int a, int b) { return ceil_div(a, b) * b; }
__host__ __device__ constexpr int pow2_ceil(int v)
{
  int p = 1;
  while (p < v) p <<= 1;
  return p;
}
// Largest power of two that is <= cap and divides v (v > 0).
__host__ __device__ constexpr int pow2_divisor(int v, int cap)
{
  int p = cap;
  while (p > 1 && (v % p) != 0) p >>= 1;
  return p;
}

// The store qualifiers that only exist here, sorted into what they imply.
__host__ __device__ constexpr bool store_is_lds(int q)
{ return q == STORE_LDS || q == STORE_LDS_DIRECT || q == STORE_LDS_SWIZZLE || q == STORE_LDS_DIRECT_SWIZZLE; }
__host__ __device__ constexpr bool store_is_direct(int q) { return q == STORE_LDS_DIRECT || q == STORE_LDS_DIRECT_SWIZZLE; }
__host__ __device__ constexpr bool store_is_swizzled(int q) { return q == STORE_LDS_SWIZZLE || q == STORE_LDS_DIRECT_SWIZZLE; }

}  // namespace detail

// Host side of the failure record.  The address of this translation unit's words on the current device
// (hipGetSymbolAddress; every device holds its own copy), and a read of them: status[0] = HIPDMA_STATUS_* bits,
// status[1] = waits that gave up since the last clear.  read_status() waits for `stream` to drain, copies
// eight bytes and, with `clear`, writes zeros back; it allocates nothing.  Both must be compiled in the same
// translation unit as the kernels they report on.
static inline hipError_t status_words_address(unsigned** words)
{
  return hipGetSymbolAddress((void**)words, HIP_SYMBOL(detail::g_status_words));
}
static inline hipError_t read_status(unsigned status[2], hipStream_t stream = nullptr, bool clear = false)
{
  unsigned* words = nullptr;
  hipError_t e = status_words_address(&words);
  if (e != hipSuccess) return e;
  e = hipStreamSynchronize(stream);
  if (e != hipSuccess) return e;
  e = hipMemcpy(status, words, 2 * sizeof(unsigned), hipMemcpyDeviceToHost);
  if (e != hipSuccess || !clear) return e;
  const unsigned zeros[2] = {0u, 0u};
  return hipMemcpy(words, zeros, sizeof(zeros), hipMemcpyHostToDevice);
}

// The swizzled LDS layouts.  The LDS has 64 banks of 4 bytes: addresses 256 bytes apart share
// their banks.  For rows of `chunks_per_row` chunks of `chunk_bytes` bytes each:
//   P     = the largest power of two that divides chunks_per_row and is at most 256/chunk_bytes
//   shift = log2 of the rows that fit one 256-byte bank line, 256 / (P * chunk_bytes), at least 0
//   key(row) = the low log2(P) bits of (row >> shift), bit-reversed
// and chunk c of row r sits at chunk position c ^ key(r) of its row.  The permutation stays
// inside aligned groups of P chunks (so inside the row), is its own inverse, and serves the
// three ways a tile is read back: down a column (sixteen consecutive rows, one chunk each: the
// keys are a bijection), row fragments of narrow rows (rows sharing a bank line get different
// keys), and blocks of a few consecutive rows (bit reversal sends neighbouring rows to
// opposite ends of the bank line).
__host__ __device__ constexpr int swizzle_span(int chunks_per_row, int chunk_bytes)
{ return chunks_per_row > 0 ? detail::pow2_divisor(chunks_per_row, 256 / chunk_bytes) : 1; }
__host__ __device__ constexpr int swizzle_key(int row, int chunks_per_row, int chunk_bytes)
{
  const int span = swizzle_span(chunks_per_row, chunk_bytes);
  if (span <= 1) return 0;
  const int bits = __builtin_ctz((unsigned)span);
  const int rows_per_line = 256 / (span * chunk_bytes);                 // a power of two, or 0 for rows beyond 256 bytes
  const int shift = rows_per_line > 1 ? __builtin_ctz((unsigned)rows_per_line) : 0;
  return (int)(__builtin_bitreverse32((unsigned)(row >> shift)) >> (32 - bits));
}
// Where chunk `chunk` of row `row` sits inside its LDS row after a swizzled transfer
// (and, the permutation being an involution, which chunk sits at position `chunk`).
__host__ __device__ constexpr int swizzled_chunk(int row, int chunk, int chunks_per_row, int chunk_bytes = 16)
{ return chunk ^ swizzle_key(row, chunks_per_row, chunk_bytes); }

}  // namespace hipdma

// Base of every DMA object: role test and the empty/full handshake.
// Follows include/cudaDMAv2.h:1316-1353; wait_for_dma_start() and
// finish_async_dma() are public as in include/cudaDMA.h:838-846 because user
// kernels call them (src/perf/sequential/perf_sequential.cu:139,150).
class CudaDMA {
public:
  // Warp-specialised form.  Must be reached by every thread of the workgroup.
  __device__ __forceinline__ CudaDMA(const int dmaID,
                                     const int num_dma_threads,
                                     const int num_compute_threads,
                                     const int dma_threadIdx_start)
    : m_is_dma_thread((int(threadIdx.x) >= dma_threadIdx_start) &&
                      (int(threadIdx.x) < (dma_threadIdx_start + num_dma_threads))),
      m_has_sync(true),
      m_full(hipdma::detail::sync_words() + 2 * dmaID),
      m_empty(hipdma::detail::sync_words() + 2 * dmaID + 1),
      m_wait_unit(0),
      m_wait_target(0)
  {
    // A DMA thread waits on `empty` for the compute threads, a compute thread
    // waits on `full` for the DMA threads.
    HIPDMA_ASSERT(dmaID >= 0 && dmaID < HIPDMA_MAX_DMA_IDS);
    HIPDMA_ASSERT(num_dma_threads > 0 && (num_dma_threads % HIPDMA_WAVE_SIZE) == 0);
    HIPDMA_ASSERT((dma_threadIdx_start % HIPDMA_WAVE_SIZE) == 0);
    HIPDMA_ASSERT(num_compute_threads > 0);
    // the same in every lane (a wavefront holds one role): pinned to a scalar register, and with it the targets
    m_wait_unit = __builtin_amdgcn_readfirstlane(m_is_dma_thread ? unsigned(num_compute_threads) : unsigned(num_dma_threads));
    if (threadIdx.x == 0) {
      *m_full = 0u;
      *m_empty = 0u;
    }
    __syncthreads();
  }
protected:
  // Form used by objects that are not warp-specialised: no LDS words, no barrier.
  __device__ __forceinline__ CudaDMA(hipdma::detail::no_sync_t,
                                     const int num_dma_threads,
                                     const int dma_threadIdx_start)
    : m_is_dma_thread((int(threadIdx.x) >= dma_threadIdx_start) &&
                      (int(threadIdx.x) < (dma_threadIdx_start + num_dma_threads))),
      m_has_sync(false),
      m_full(nullptr),
      m_empty(nullptr),
      m_wait_unit(0),
      m_wait_target(0)
  {
  }
public:
  // Compute side: the buffer is free, the DMA wavefronts may overwrite it.  Does not block.
  __device__ __forceinline__ void start_async_dma(void) const
  {
    if (m_has_sync) hipdma::detail::signal_word(m_empty);
  }
  // Compute side: block until the DMA wavefronts have filled the buffer.
  __device__ __forceinline__ void wait_for_dma_finish(void) const
  {
    if (m_has_sync) {
      m_wait_target += m_wait_unit;
      hipdma::detail::wait_word(m_full, m_wait_target);
    }
  }
  // Compute side, the wait split in two so that the round trip to LDS can hide behind other
  // work: peek_dma_finish() reads the `full` word without blocking, wait_for_dma_finish(peeked)
  // later completes the wait (and only polls when the peeked value was not there yet).  An
  // addition of this library: with named barriers there is nothing to peek at.
  __device__ __forceinline__ unsigned peek_dma_finish(void) const
  {
    return m_has_sync ? __hip_atomic_load(m_full, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP) : 0u;
  }
  __device__ __forceinline__ void wait_for_dma_finish(const unsigned peeked) const
  {
    if (m_has_sync) {
      m_wait_target += m_wait_unit;
      // every lane peeked at the same word with the same instruction: a scalar comparison
      if ((int)(__builtin_amdgcn_readfirstlane(peeked) - __builtin_amdgcn_readfirstlane(m_wait_target)) < 0)
        hipdma::detail::wait_word(m_full, m_wait_target);
      else hipdma::detail::acquire_lds();
    }
  }
  __device__ __forceinline__ bool owns_this_thread(void) const { return m_is_dma_thread; }
  // DMA side: block until every compute thread has released the buffer.
  __device__ __forceinline__ void wait_for_dma_start(void) const
  {
    if (m_has_sync) {
      m_wait_target += m_wait_unit;
      hipdma::detail::wait_word(m_empty, m_wait_target);
    }
  }
  // DMA side: the buffer is full.  Does not block.
  __device__ __forceinline__ void finish_async_dma(void) const
  {
    if (m_has_sync) hipdma::detail::signal_word(m_full);
  }
  // DMA side, for wavefronts that keep direct-to-LDS loads (CudaDMAStrided::issue_direct) in
  // flight across the hand-off: the same two calls without a fence and without an LDS access the
  // compiler could see, because either would make it wait for every outstanding direct load.
  // The caller waits for the loads it reports (hipdma::wait_direct_loads<YOUNGER>()) before
  // finish_async_dma_direct(), and requests loads into a buffer only after
  // wait_for_dma_start_direct() for that buffer has returned.
  __device__ __forceinline__ void wait_for_dma_start_direct(void) const
  {
    if (m_has_sync) {
      m_wait_target += m_wait_unit;
      hipdma::detail::wait_word_unfenced(m_empty, m_wait_target);
    }
  }
  __device__ __forceinline__ void finish_async_dma_direct(void) const
  {
    if (m_has_sync) hipdma::detail::signal_word_unfenced(m_full);
  }
protected:
  const bool m_is_dma_thread;
  const bool m_has_sync;
  hipdma::detail::lds_word_t* const m_full;
  hipdma::detail::lds_word_t* const m_empty;
  unsigned m_wait_unit;
  mutable unsigned m_wait_target;
};

namespace hipdma {

// Barrier among a subset of the workgroup's wavefronts: what `bar.sync id,count`
// gives CUDA code that wants its compute warps to meet without the DMA warps.
// Uses the LDS word pair of slot `id` (shared numbering with dmaID: give it an
// id no DMA object of the kernel uses).  Every thread of the workgroup
// constructs it; only the `num_threads` participants call sync().
class GroupBarrier {
public:
  __device__ __forceinline__ GroupBarrier(const int id, const int num_threads)
    : m_word(detail::sync_words() + 2 * id), m_unit(unsigned(num_threads)), m_target(0)
  {
    if (threadIdx.x == 0) *m_word = 0u;
    __syncthreads();
  }
  __device__ __forceinline__ void sync()
  {
    m_target += m_unit;
    detail::signal_word(m_word);
    detail::wait_word(m_word, m_target);
  }
private:
  detail::lds_word_t* const m_word;
  const unsigned m_unit;
  unsigned m_target;
};

}  // namespace hipdma

// Sync-only object for hand-written transfer code (include/cudaDMA.h:4184-4208).
class cudaDMACustom : public CudaDMA {
public:
  __device__ __forceinline__ cudaDMACustom(const int dmaID,
                                           const int num_dma_threads,
                                           const int num_compute_threads,
                                           const int dma_threadIdx_start)
    : CudaDMA(dmaID, num_dma_threads, num_compute_threads, dma_threadIdx_start) {}
};
typedef cudaDMACustom CudaDMACustom;
