// Self-test of the split wait (peek_dma_finish + wait_for_dma_finish(peeked)); kept apart from
// the bounded-wait test, which lowers the poll limit for its whole translation unit.
#include "common.hpp"
#include "../../include/cudadma_amd_harness.h"
#include "../../include/hipDMA.h"
#include "status_word.hpp"

namespace {

// The split wait: the compute wavefront peeks at the `full` word, does something else, and
// completes the wait with the peeked value.  Every phase the DMA wavefront writes a new
// pattern into the buffer; the compute wavefront must see exactly that pattern whether or
// not the peek had already found the buffer full.
__global__ void __launch_bounds__(128) split_wait(int* out, const int phases)
{
  __shared__ int buf[64];
  cudaDMACustom dma(1, 64, 64, 64);
  if (dma.owns_this_thread()) {
    for (int p = 0; p < phases; ++p) {
      dma.wait_for_dma_start();
      if (p & 1) __builtin_amdgcn_s_sleep(16);         // late on odd phases, so both branches of the wait run
      buf[threadIdx.x - 64] = p * 64 + int(threadIdx.x) - 64;
      dma.finish_async_dma();
    }
  } else {
    int wrong = 0, early = 0;
    for (int p = 0; p < phases; ++p) {
      dma.start_async_dma();
      if (!(p & 1)) __builtin_amdgcn_s_sleep(16);      // give the DMA side a head start on even phases
      const unsigned peeked = dma.peek_dma_finish();
      early += (int)(peeked - 64u * (unsigned)(p + 1)) >= 0 ? 1 : 0;
      dma.wait_for_dma_finish(peeked);
      wrong += (buf[threadIdx.x] != p * 64 + int(threadIdx.x)) ? 1 : 0;
    }
    atomicAdd(out, wrong);
    if (threadIdx.x == 0) out[1] = early;
  }
}

}  // namespace

extern "C" int cudadma_selftest_split_wait(int* d_out, int phases, void* stream)
{
  CUDADMA_REQUIRE(d_out != nullptr && phases > 0, "d_out is NULL or phases is not positive");
  hipLaunchKernelGGL(split_wait, dim3(1), dim3(128), 0, (hipStream_t)stream, d_out, phases);
  CUDADMA_HIP_CHECK(hipGetLastError());
  return CUDADMA_OK;
}

