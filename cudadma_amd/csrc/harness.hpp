// Known-answer harness: registry of compiled DMA-object cases and the kernel
// skeleton they share.  One workgroup; warp-specialised cases run 64 compute
// threads [0,64) and DMA_THREADS DMA threads [64, 64+DMA_THREADS); the compute
// wavefront clears the LDS buffer, releases it, waits for the transfer and
// copies the whole buffer out (the shape of special_xfer_* in
// src/tests/test_sequential/cudaDMA_test_sequential_v2.cu:52-115).  The other
// cases run DMA_THREADS threads that all transfer, between two workgroup
// barriers (nonspec_xfer_*, same file).
#pragma once

#include "common.hpp"
#include "../../include/cudadma_amd_harness.h"
#include "../../include/hipDMA.h"
#include "status_word.hpp"

// The case lists are long and every case is a pair of kernels with a dozen call styles inlined: the Makefile
// compiles each harness source HARNESS_SHARDS times, piece HARNESS_SHARD taking every HARNESS_SHARDS-th case.
#ifndef HARNESS_SHARDS
#define HARNESS_SHARDS 1
#define HARNESS_SHARD 0
#endif

namespace harness {

constexpr int kComputeThreads = 64;

struct Args {
  const char* in;
  char* out;
  const int* index;
  int lds_bytes;
  int src_offset, dst_offset;
  int src_stride, dst_stride;
  int pitch;
  int call_style, two_phase;
  int reps, rep_src_bytes, rep_index_elmts;
  int reverse, out_bytes;
  // run-time copies of the template parameters, fed to the constructors of the lower levels
  int bytes_per_elmt, dma_threads, num_elmts, dimx, dimy;
  int dst_pitch;       // halo: destination row pitch in cells, 0 = dimx + 2*radius
};

typedef int (*launch_fn)(const Args&, hipStream_t);

struct Entry {
  cudadma_case_t desc;
  launch_fn launch;
  int order;
};

void register_case(const cudadma_case_t& desc, launch_fn fn, int order);

struct Registrar {
  Registrar(const cudadma_case_t& desc, launch_fn fn, int order) { register_case(desc, fn, order); }
};

// Transfer through the call style picked at run time.  XFER is a functor
// template<bool GL,int LQ,int SQ> with static run(obj, two_phase, ...).
template<typename Obj, typename... P>
__device__ __forceinline__ void do_transfer(Obj& dma, const int call_style, const int two_phase,
                                            const void* src, void* dst)
{
  if (call_style == CUDADMA_CALL_UNQUALIFIED) {
    if (two_phase) { dma.start_xfer_async(src); dma.wait_xfer_finish(dst); }
    else dma.execute_dma(src, dst);
  } else if (call_style == CUDADMA_CALL_GLOBAL) {
    if (two_phase) { dma.template start_xfer_async<true>(src); dma.template wait_xfer_finish<true>(dst); }
    else dma.template execute_dma<true>(src, dst);
  } else if (call_style == CUDADMA_CALL_QUALIFIED) {
    if (two_phase) {
      dma.template start_xfer_async<true, LOAD_CACHE_STREAMING, STORE_LDS>(src);
      dma.template wait_xfer_finish<true, LOAD_CACHE_STREAMING, STORE_LDS>(dst);
    } else dma.template execute_dma<true, LOAD_CACHE_STREAMING, STORE_LDS>(src, dst);
  }
}

template<int STORE_QUAL = STORE_LDS_DIRECT, typename Obj>
__device__ __forceinline__ void do_transfer_direct(Obj& dma, const int two_phase, const void* src, void* dst)
{
  if (two_phase) {
    dma.template start_xfer_async<true, LOAD_CACHE_ALL, STORE_QUAL>(src);
    dma.template wait_xfer_finish<true, LOAD_CACHE_ALL, STORE_QUAL>(dst);
  } else dma.template execute_dma<true, LOAD_CACHE_ALL, STORE_QUAL>(src, dst);
}

template<typename Obj>
__device__ __forceinline__ void do_transfer_indexed(Obj& dma, const int call_style, const int two_phase,
                                                    const int* index, const void* src, void* dst)
{
  if (call_style == CUDADMA_CALL_UNQUALIFIED) {
    if (two_phase) { dma.start_xfer_async(index, src); dma.wait_xfer_finish(dst); }
    else dma.execute_dma(index, src, dst);
  } else if (call_style == CUDADMA_CALL_GLOBAL) {
    if (two_phase) { dma.template start_xfer_async<true>(index, src); dma.template wait_xfer_finish<true>(dst); }
    else dma.template execute_dma<true>(index, src, dst);
  } else if (call_style == CUDADMA_CALL_QUALIFIED) {
    if (two_phase) {
      dma.template start_xfer_async<true, LOAD_CACHE_STREAMING, STORE_WRITE_BACK>(index, src);
      dma.template wait_xfer_finish<true, LOAD_CACHE_STREAMING, STORE_WRITE_BACK>(dst);
    } else dma.template execute_dma<true, LOAD_CACHE_STREAMING, STORE_WRITE_BACK>(index, src, dst);
  }
}

// The qualifier matrix (enums of include/cudaDMAv2.h:50-63; the reference's tests run an assortment of the
// combinations, src/tests/test_strided/cudaDMA_test_strided_v2.cu:693-812): every load qualifier once with a
// source known to be global and once with a generic source, every store qualifier of the reference at least
// twice, and the direct-to-LDS path with a load qualifier.  The kernels of these styles are instantiated
// apart from those of the first six (template parameter MATRIX of the case kernels) to keep each kernel small.
template<bool GL, int LQ, int SQ, typename Obj>
__device__ __forceinline__ void transfer_as(Obj& dma, const int two_phase, const void* src, void* dst)
{
  if (two_phase) {
    dma.template start_xfer_async<GL, LQ, SQ>(src);
    dma.template wait_xfer_finish<GL, LQ, SQ>(dst);
  } else dma.template execute_dma<GL, LQ, SQ>(src, dst);
}
template<bool GL, int LQ, int SQ, typename Obj>
__device__ __forceinline__ void transfer_indexed_as(Obj& dma, const int two_phase, const int* index, const void* src, void* dst)
{
  if (two_phase) {
    dma.template start_xfer_async<GL, LQ, SQ>(index, src);
    dma.template wait_xfer_finish<GL, LQ, SQ>(dst);
  } else dma.template execute_dma<GL, LQ, SQ>(index, src, dst);
}

// DIRECT: the object has a direct-to-LDS path for this case (otherwise the two direct styles are left out).
#define HARNESS_QUALIFIER_MATRIX(CALL, ...)                                                                              \
  switch (call_style) {                                                                                                  \
    case CUDADMA_CALL_Q_GLOBAL_CG:     CALL<true, LOAD_CACHE_GLOBAL, STORE_CACHE_GLOBAL>(__VA_ARGS__); break;            \
    case CUDADMA_CALL_Q_LASTUSE_CS:    CALL<true, LOAD_CACHE_LAST_USE, STORE_CACHE_STREAMING>(__VA_ARGS__); break;       \
    case CUDADMA_CALL_Q_VOLATILE_WT:   CALL<true, LOAD_CACHE_VOLATILE, STORE_CACHE_WRITE_THROUGH>(__VA_ARGS__); break;   \
    case CUDADMA_CALL_Q_STREAMING_WB:  CALL<true, LOAD_CACHE_STREAMING, STORE_WRITE_BACK>(__VA_ARGS__); break;           \
    case CUDADMA_CALL_QG_GLOBAL_CS:    CALL<false, LOAD_CACHE_GLOBAL, STORE_CACHE_STREAMING>(__VA_ARGS__); break;        \
    case CUDADMA_CALL_QG_STREAMING_WT: CALL<false, LOAD_CACHE_STREAMING, STORE_CACHE_WRITE_THROUGH>(__VA_ARGS__); break; \
    case CUDADMA_CALL_QG_LASTUSE_CG:   CALL<false, LOAD_CACHE_LAST_USE, STORE_CACHE_GLOBAL>(__VA_ARGS__); break;         \
    case CUDADMA_CALL_QG_VOLATILE_WB:  CALL<false, LOAD_CACHE_VOLATILE, STORE_WRITE_BACK>(__VA_ARGS__); break;           \
    default: break;                                                                                                      \
  }

template<bool DIRECT, typename Obj>
__device__ __forceinline__ void do_transfer_matrix(Obj& dma, const int call_style, const int two_phase,
                                                   const void* src, void* dst)
{
  HARNESS_QUALIFIER_MATRIX(transfer_as, dma, two_phase, src, dst)
  if constexpr (DIRECT) {
    if (call_style == CUDADMA_CALL_LDS_DIRECT_SC1) transfer_as<true, LOAD_CACHE_GLOBAL, STORE_LDS_DIRECT>(dma, two_phase, src, dst);
    else if (call_style == CUDADMA_CALL_LDS_DIRECT_NT) transfer_as<true, LOAD_CACHE_STREAMING, STORE_LDS_DIRECT>(dma, two_phase, src, dst);
  }
}
template<bool DIRECT, typename Obj>
__device__ __forceinline__ void do_transfer_indexed_matrix(Obj& dma, const int call_style, const int two_phase,
                                                           const int* index, const void* src, void* dst)
{
  HARNESS_QUALIFIER_MATRIX(transfer_indexed_as, dma, two_phase, index, src, dst)
  if constexpr (DIRECT) {
    if (call_style == CUDADMA_CALL_LDS_DIRECT_SC1)
      transfer_indexed_as<true, LOAD_CACHE_GLOBAL, STORE_LDS_DIRECT>(dma, two_phase, index, src, dst);
    else if (call_style == CUDADMA_CALL_LDS_DIRECT_NT)
      transfer_indexed_as<true, LOAD_CACHE_STREAMING, STORE_LDS_DIRECT>(dma, two_phase, index, src, dst);
  }
}

// The LDS buffer handling both kernel shapes share.
__device__ __forceinline__ void clear_lds(unsigned* buf, const int words, const int tid, const int nthreads)
{
  for (int i = tid; i < words; i += nthreads) buf[i] = 0u;
}
__device__ __forceinline__ void copy_out(const unsigned* buf, unsigned* out, const int words, const int tid,
                                         const int nthreads)
{
  for (int i = tid; i < words; i += nthreads) out[i] = buf[i];
}

__device__ __forceinline__ void fill_lds(unsigned* buf, const unsigned* in, const int words, const int tid,
                                         const int nthreads)
{
  for (int i = tid; i < words; i += nthreads) buf[i] = in[i];
}

// Body shared by every case.  `xfer(rep)` performs one transfer (DMA threads); it has exactly
// one call site per kernel shape so that it is inlined and the object stays in registers.
// Forward: the compute side clears LDS, releases it, waits for the transfer, copies LDS out.
// Reverse (LDS is the source): the compute side loads the image into LDS and waits until the DMA
// side has moved it out to global memory.  The objects issue their loads before the handshake
// wait (the source is assumed ready, as in the reference), so the compute side signals twice:
// the first signal says "the image is in LDS" and is consumed by an explicit
// wait_for_dma_start() ahead of the transfer, the second is the one the transfer itself waits for.
template<bool WS, typename Obj, typename Xfer>
__device__ __forceinline__ void run_body(Obj& dma, const Args& a, unsigned* lds, Xfer xfer)
{
  const int words = a.lds_bytes / 4;
  if constexpr (WS) {
    if (dma.owns_this_thread()) {
      for (int rep = 0; rep < a.reps; ++rep) {
        if (a.reverse) dma.wait_for_dma_start();
        xfer(rep);
      }
    } else if (threadIdx.x < kComputeThreads) {
      for (int rep = 0; rep < a.reps; ++rep) {
        if (a.reverse)
          fill_lds(lds, (const unsigned*)(a.in + (size_t)rep * a.rep_src_bytes), words, threadIdx.x, kComputeThreads);
        else
          clear_lds(lds, words, threadIdx.x, kComputeThreads);
        if (a.reverse) dma.start_async_dma();
        dma.start_async_dma();
        dma.wait_for_dma_finish();
        if (!a.reverse)
          copy_out(lds, (unsigned*)(a.out + (size_t)rep * a.lds_bytes), words, threadIdx.x, kComputeThreads);
      }
    }
  } else {
    for (int rep = 0; rep < a.reps; ++rep) {
      if (a.reverse)
        fill_lds(lds, (const unsigned*)(a.in + (size_t)rep * a.rep_src_bytes), words, threadIdx.x, blockDim.x);
      else
        clear_lds(lds, words, threadIdx.x, blockDim.x);
      __syncthreads();
      xfer(rep);
      __syncthreads();
      if (!a.reverse)
        copy_out(lds, (unsigned*)(a.out + (size_t)rep * a.lds_bytes), words, threadIdx.x, blockDim.x);
      __syncthreads();
    }
  }
}

inline bool is_matrix_style(const int call_style) { return call_style >= CUDADMA_CALL_Q_GLOBAL_CG && call_style <= CUDADMA_CALL_LDS_DIRECT_NT; }

// `kernel` runs the first six call styles, `matrix_kernel` the qualifier matrix.
template<typename Kernel>
int launch_case(Kernel kernel, Kernel matrix_kernel, const bool ws, const Args& a, hipStream_t stream)
{
  const int threads = ws ? (kComputeThreads + a.dma_threads) : a.dma_threads;
  hipLaunchKernelGGL(is_matrix_style(a.call_style) ? matrix_kernel : kernel, dim3(1), dim3(threads), (size_t)a.lds_bytes,
                     stream, a);
  CUDADMA_HIP_CHECK(hipGetLastError());
  return CUDADMA_OK;
}

}  // namespace harness
