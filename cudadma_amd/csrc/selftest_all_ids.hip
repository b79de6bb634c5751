// Self-test of the handshake words of all sixteen dmaIDs: sixteen sync-only objects guard sixteen LDS
// slots, the DMA wavefronts may run up to sixteen phases ahead of the compute wavefront, and every
// slot must hold exactly the token of its phase when the compute side gets to it.  A word shared
// between two ids, or a lost count, shows up as a wrong token (the bounded wait turns a hang into one).
#include "common.hpp"
#include "../../include/cudadma_amd_harness.h"
#include "../../include/hipDMA.h"
#include "status_word.hpp"

namespace {

constexpr int kIds = HIPDMA_MAX_DMA_IDS;
constexpr int kComputeThreads = 64;
constexpr int kDmaThreads = 128;

__global__ void __launch_bounds__(kComputeThreads + kDmaThreads) all_ids(int* out, const int phases)
{
  __shared__ int slot[kIds][kDmaThreads];
#define HIPDMA_GUARD(I) cudaDMACustom(I, kDmaThreads, kComputeThreads, kComputeThreads)
  cudaDMACustom guard[kIds] = {HIPDMA_GUARD(0), HIPDMA_GUARD(1), HIPDMA_GUARD(2), HIPDMA_GUARD(3), HIPDMA_GUARD(4), HIPDMA_GUARD(5),
                               HIPDMA_GUARD(6), HIPDMA_GUARD(7), HIPDMA_GUARD(8), HIPDMA_GUARD(9), HIPDMA_GUARD(10), HIPDMA_GUARD(11),
                               HIPDMA_GUARD(12), HIPDMA_GUARD(13), HIPDMA_GUARD(14), HIPDMA_GUARD(15)};
#undef HIPDMA_GUARD
  static_assert(kIds == 16, "the list above names sixteen objects");
  if (guard[0].owns_this_thread()) {
    const int t = int(threadIdx.x) - kComputeThreads;
    for (int p = 0; p < phases; ++p) {
      const cudaDMACustom& g = guard[p % kIds];
      g.wait_for_dma_start();
      slot[p % kIds][t] = p * 1024 + t;
      g.finish_async_dma();
    }
  } else {
    int wrong = 0;
    for (int i = 0; i < kIds; ++i) guard[i].start_async_dma();       // all sixteen slots are free
    for (int p = 0; p < phases; ++p) {
      const cudaDMACustom& g = guard[p % kIds];
      if ((p % 5) == 0) __builtin_amdgcn_s_sleep(32);                  // let the DMA side get ahead now and then
      g.wait_for_dma_finish();
      wrong += (slot[p % kIds][threadIdx.x] != p * 1024 + int(threadIdx.x)) ? 1 : 0;
      wrong += (slot[p % kIds][threadIdx.x + 64] != p * 1024 + int(threadIdx.x) + 64) ? 1 : 0;
      g.start_async_dma();
    }
    atomicAdd(out, wrong);
  }
}

}  // namespace

extern "C" int cudadma_selftest_all_ids(int* d_out, int phases, void* stream)
{
  CUDADMA_REQUIRE(d_out != nullptr && phases > 0, "d_out is NULL or phases is not positive");
  hipLaunchKernelGGL(all_ids, dim3(1), dim3(kComputeThreads + kDmaThreads), 0, (hipStream_t)stream, d_out, phases);
  CUDADMA_HIP_CHECK(hipGetLastError());
  return CUDADMA_OK;
}
