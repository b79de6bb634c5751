// Read-bandwidth probe for CudaDMASequential with every parameter at run time: element
// size, DMA wavefronts, buffering style, transfers per workgroup and workgroups per compute
// unit.  The counterpart of src/perf/sequential/perf_sequential.cu:52-228, which bakes the
// same parameters in through params_directed.h and is recompiled per point by
// param_sweep.py:27-58.  As there, one compute wavefront stands for the consumer and the
// data is only brought into LDS; with `consume` set the compute wavefront also adds every
// 32-bit word it finds to a per-workgroup checksum so that a test can see the bytes arrive.
// The cache qualifier of the loads and the kind of store into LDS are template parameters of the
// objects' calls (include/cudaDMAv2.h:1460-1562); the entry point picks among the compiled combinations.
#include "workloads.hpp"

namespace {

constexpr int kCompute = 64;                 // one compute wavefront, as in the reference
constexpr int kBytesPerThread = 64;          // four dwordx4 in flight per DMA thread
static_assert(CUDADMA_LOAD_CACHE_ALL == LOAD_CACHE_ALL && CUDADMA_LOAD_CACHE_STREAMING == LOAD_CACHE_STREAMING &&
              CUDADMA_STORE_WRITE_BACK == STORE_WRITE_BACK && CUDADMA_STORE_LDS == STORE_LDS &&
              CUDADMA_STORE_LDS_DIRECT == STORE_LDS_DIRECT, "the C header restates the qualifier enums of the device header");

struct PerfArgs {
  const char* src;
  unsigned* sums;       // one word per workgroup (consume only)
  int elmt_bytes, dma_threads, loops, consume;
};

__device__ __forceinline__ unsigned sum_words(const char* buf, const int bytes, const int tid, const int nthreads)
{
  unsigned acc = 0;
  const unsigned* w = (const unsigned*)buf;
  for (int i = tid; i < bytes / 4; i += nthreads) acc += w[i];
  return acc;
}

__device__ __forceinline__ const char* wg_base(const PerfArgs& a)
{ return a.src + (size_t)blockIdx.x * a.elmt_bytes * a.loops; }

// No specialisation: every thread transfers, workgroup barriers around the use of the buffer.
template<int LQ, int SQ>
__global__ void perf_none(const PerfArgs a)
{
  typedef CudaDMASequential<false, 16, kBytesPerThread> all_dma_t;       // size and thread count at run time
  extern __shared__ __attribute__((aligned(16))) char lds[];
  all_dma_t dma(a.elmt_bytes);
  const char* p = wg_base(a);
  unsigned acc = 0;
  for (int i = 0; i < a.loops; ++i) {
    dma.template execute_dma<true, LQ, SQ>(p, lds);
    __syncthreads();
    if (a.consume) acc += sum_words(lds, a.elmt_bytes, threadIdx.x, blockDim.x);
    p += a.elmt_bytes;
    __syncthreads();
  }
  if (a.consume) atomicAdd(a.sums + blockIdx.x, acc);
}

template<int LQ, int SQ>
__global__ void perf_single(const PerfArgs a)
{
  typedef CudaDMASequential<true, 16, kBytesPerThread> ws_dma_t;       // size and thread count at run time
  extern __shared__ __attribute__((aligned(16))) char lds[];
  ws_dma_t dma(0, a.dma_threads, kCompute, kCompute, a.elmt_bytes);
  if (dma.owns_this_thread()) {
    const char* p = wg_base(a);
    for (int i = 0; i < a.loops; ++i) {
      dma.template execute_dma<true, LQ, SQ>(p, lds);
      p += a.elmt_bytes;
    }
  } else {
    unsigned acc = 0;
    for (int i = 0; i < a.loops; ++i) {
      dma.start_async_dma();
      dma.wait_for_dma_finish();
      if (a.consume) acc += sum_words(lds, a.elmt_bytes, threadIdx.x, kCompute);
    }
    if (a.consume) atomicAdd(a.sums + blockIdx.x, acc);
  }
}

// Two buffers, two objects on disjoint DMA wavefronts; transfer i goes through buffer i & 1.
template<int LQ, int SQ>
__global__ void perf_double(const PerfArgs a)
{
  typedef CudaDMASequential<true, 16, kBytesPerThread> ws_dma_t;       // size and thread count at run time
  extern __shared__ __attribute__((aligned(16))) char lds[];
  char* buf0 = lds;
  char* buf1 = lds + hipdma::detail::round_up(a.elmt_bytes, 16);
  ws_dma_t dma0(0, a.dma_threads, kCompute, kCompute, a.elmt_bytes);
  ws_dma_t dma1(1, a.dma_threads, kCompute, kCompute + a.dma_threads, a.elmt_bytes);
  if (dma0.owns_this_thread()) {
    const char* p = wg_base(a);
    for (int i = 0; i < a.loops; i += 2) dma0.template execute_dma<true, LQ, SQ>(p + (size_t)i * a.elmt_bytes, buf0);
  } else if (dma1.owns_this_thread()) {
    const char* p = wg_base(a);
    for (int i = 1; i < a.loops; i += 2) dma1.template execute_dma<true, LQ, SQ>(p + (size_t)i * a.elmt_bytes, buf1);
  } else {
    unsigned acc = 0;
    dma0.start_async_dma();
    dma1.start_async_dma();
    for (int i = 0; i < a.loops; i += 2) {
      dma0.wait_for_dma_finish();
      if (a.consume) acc += sum_words(buf0, a.elmt_bytes, threadIdx.x, kCompute);
      if (i + 2 < a.loops) dma0.start_async_dma();
      if (i + 1 < a.loops) {
        dma1.wait_for_dma_finish();
        if (a.consume) acc += sum_words(buf1, a.elmt_bytes, threadIdx.x, kCompute);
        if (i + 3 < a.loops) dma1.start_async_dma();
      }
    }
    if (a.consume) atomicAdd(a.sums + blockIdx.x, acc);
  }
}

// Two buffers, two objects on the SAME DMA wavefronts, kept busy with the two-phase calls.
template<int LQ, int SQ>
__global__ void perf_manual(const PerfArgs a)
{
  typedef CudaDMASequential<true, 16, kBytesPerThread> ws_dma_t;       // size and thread count at run time
  extern __shared__ __attribute__((aligned(16))) char lds[];
  char* buf0 = lds;
  char* buf1 = lds + hipdma::detail::round_up(a.elmt_bytes, 16);
  ws_dma_t dma0(0, a.dma_threads, kCompute, kCompute, a.elmt_bytes);
  ws_dma_t dma1(1, a.dma_threads, kCompute, kCompute, a.elmt_bytes);
  if (dma0.owns_this_thread()) {
    const char* p = wg_base(a);
    const int last = a.loops - 1;
    // transfers past the end re-request the last element so that no load sits behind a branch
    dma0.template start_xfer_async<true, LQ, SQ>(p);
    dma1.template start_xfer_async<true, LQ, SQ>(p + (size_t)(1 < last ? 1 : last) * a.elmt_bytes);
    for (int i = 0; i < a.loops; i += 2) {
      dma0.template wait_xfer_finish<true, LQ, SQ>(buf0);
      dma0.template start_xfer_async<true, LQ, SQ>(p + (size_t)(i + 2 < last ? i + 2 : last) * a.elmt_bytes);
      if (i + 1 < a.loops) {
        dma1.template wait_xfer_finish<true, LQ, SQ>(buf1);
        dma1.template start_xfer_async<true, LQ, SQ>(p + (size_t)(i + 3 < last ? i + 3 : last) * a.elmt_bytes);
      }
    }
  } else {
    unsigned acc = 0;
    dma0.start_async_dma();
    dma1.start_async_dma();
    for (int i = 0; i < a.loops; i += 2) {
      dma0.wait_for_dma_finish();
      if (a.consume) acc += sum_words(buf0, a.elmt_bytes, threadIdx.x, kCompute);
      if (i + 2 < a.loops) dma0.start_async_dma();
      if (i + 1 < a.loops) {
        dma1.wait_for_dma_finish();
        if (a.consume) acc += sum_words(buf1, a.elmt_bytes, threadIdx.x, kCompute);
        if (i + 3 < a.loops) dma1.start_async_dma();
      }
    }
    if (a.consume) atomicAdd(a.sums + blockIdx.x, acc);
  }
}

typedef void (*perf_kernel_t)(const PerfArgs);
struct PerfEntry { int load_qualifier, store_qualifier; perf_kernel_t kernels[4]; };
#define PERF_ENTRY(LQ, SQ) {LQ, SQ, {perf_none<LQ, SQ>, perf_single<LQ, SQ>, perf_double<LQ, SQ>, perf_manual<LQ, SQ>}}
// STORE_WRITE_BACK: a generic store as in the reference's probe (execute_dma<true>); STORE_LDS: ds_write_b128;
// STORE_LDS_DIRECT: global_load_lds, no register staging
const PerfEntry kPerfEntries[] = {PERF_ENTRY(LOAD_CACHE_ALL, STORE_WRITE_BACK), PERF_ENTRY(LOAD_CACHE_ALL, STORE_LDS),
                                  PERF_ENTRY(LOAD_CACHE_ALL, STORE_LDS_DIRECT), PERF_ENTRY(LOAD_CACHE_STREAMING, STORE_WRITE_BACK),
                                  PERF_ENTRY(LOAD_CACHE_STREAMING, STORE_LDS), PERF_ENTRY(LOAD_CACHE_STREAMING, STORE_LDS_DIRECT)};
#undef PERF_ENTRY

}  // namespace

extern "C" long long cudadma_perf_sequential(const void* d_src, size_t src_bytes, unsigned* d_sums, int elmt_bytes,
                                             int dma_wavefronts, int buffering, int loop_iters, int workgroups,
                                             int load_qualifier, int store_qualifier, void* stream)
{
  auto fail = [](int code) { return (long long)code; };
  if (elmt_bytes < 16 || (elmt_bytes % 16) != 0 || elmt_bytes > 24 * 1024) {
    cudadma_host::set_error("elmt_bytes (%d) must be a multiple of 16 between 16 and 24576", elmt_bytes);
    return fail(CUDADMA_EINVAL);
  }
  if (dma_wavefronts < 1 || dma_wavefronts > 7 || loop_iters < 1 || workgroups < 1) {
    cudadma_host::set_error("dma_wavefronts 1..7, loop_iters >= 1, workgroups >= 1 (got %d, %d, %d)", dma_wavefronts, loop_iters,
                            workgroups);
    return fail(CUDADMA_EINVAL);
  }
  if (buffering < CUDADMA_BUFFERING_NONE || buffering > CUDADMA_BUFFERING_MANUAL) {
    cudadma_host::set_error("unknown buffering %d", buffering);
    return fail(CUDADMA_ERANGE);
  }
  const PerfEntry* e = nullptr;
  for (const PerfEntry& c : kPerfEntries)
    if (c.load_qualifier == load_qualifier && c.store_qualifier == store_qualifier)
      e = &c;
  if (e == nullptr) {
    cudadma_host::set_error("the probe is compiled for load qualifiers LOAD_CACHE_ALL (%d) and LOAD_CACHE_STREAMING (%d), store qualifiers "
                            "STORE_WRITE_BACK (%d), STORE_LDS (%d) and STORE_LDS_DIRECT (%d) (got %d, %d)",
                            (int)LOAD_CACHE_ALL, (int)LOAD_CACHE_STREAMING, (int)STORE_WRITE_BACK, (int)STORE_LDS, (int)STORE_LDS_DIRECT,
                            load_qualifier, store_qualifier);
    return fail(CUDADMA_ERANGE);
  }
  const long long total = (long long)workgroups * elmt_bytes * loop_iters;
  if (d_src == nullptr || !cudadma_host::aligned_to(d_src, 16) || (unsigned long long)total > src_bytes) {
    cudadma_host::set_error("d_src must be 16-byte aligned and hold workgroups * elmt_bytes * loop_iters = %lld bytes", total);
    return fail(CUDADMA_EINVAL);
  }
  const int dma_threads = dma_wavefronts * 64;
  const bool two = buffering == CUDADMA_BUFFERING_DOUBLE || buffering == CUDADMA_BUFFERING_MANUAL;
  const size_t lds = (size_t)(two ? 2 : 1) * hipdma::detail::round_up(elmt_bytes, 16);
  PerfArgs a = {(const char*)d_src, d_sums, elmt_bytes, dma_threads, loop_iters, d_sums != nullptr ? 1 : 0};
  hipStream_t s = (hipStream_t)stream;
  const int threads = buffering == CUDADMA_BUFFERING_NONE ? dma_threads
                    : buffering == CUDADMA_BUFFERING_DOUBLE ? kCompute + 2 * dma_threads : kCompute + dma_threads;
  hipLaunchKernelGGL(e->kernels[buffering], dim3(workgroups), dim3(threads), lds, s, a);
  if (hipGetLastError() != hipSuccess) {
    cudadma_host::set_error("launch of the sequential probe failed");
    return fail(CUDADMA_ELAUNCH);
  }
  return total;
}
