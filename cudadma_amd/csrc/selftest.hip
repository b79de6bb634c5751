// Failure handling of the handshake: a wait that can never be satisfied must end.
// This translation unit lowers the poll limit so that the condition is forced from the
// host side and every wavefront still exits normally.
#define HIPDMA_SPIN_LIMIT 256
#include "common.hpp"
#include "../../include/cudadma_amd_harness.h"
#include "../../include/hipDMA.h"
#include "status_word.hpp"

namespace {

// 64 compute threads and 64 DMA threads that never signal each other.
__global__ void __launch_bounds__(128) unmatched_waits(int* flags)
{
  cudaDMACustom dma(0, 64, 64, 64);
  if (dma.owns_this_thread()) {
    dma.wait_for_dma_start();          // nobody calls start_async_dma()
    if (threadIdx.x == 64) flags[0] = 1;
  } else {
    dma.wait_for_dma_finish();         // nobody calls finish_async_dma()
    if (threadIdx.x == 0) flags[1] = 1;
  }
}

}  // namespace

extern "C" int cudadma_selftest_bounded_wait(int* d_flags, void* stream)
{
  CUDADMA_REQUIRE(d_flags != nullptr, "d_flags is NULL");
  hipLaunchKernelGGL(unmatched_waits, dim3(1), dim3(128), 0, (hipStream_t)stream, d_flags);
  CUDADMA_HIP_CHECK(hipGetLastError());
  return CUDADMA_OK;
}
