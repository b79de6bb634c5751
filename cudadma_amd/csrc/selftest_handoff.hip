// Global-memory hand-off across the handshake with the header's default (all address spaces) fences.
#define HANDOFF_ENTRY cudadma_selftest_global_handoff
#include "selftest_handoff.inc"

// ---- the same self-test for callers that cannot allocate device memory ----------------------------------
// cudadma_selftest_global_handoff() takes its 16 KiB of staging memory from the caller.  This entry point keeps them
// in a file-scope device array instead, so a caller under graph capture, in a serving loop or in a harness that forbids
// hipMalloc can run the self-test with nothing but the word for the result.  In host code the array's name is only a
// stand-in: the address on each device comes from hipGetSymbolAddress, once per device, and that pointer is what the
// kernel receives.
#include <mutex>

namespace {

constexpr int kNoAllocMaxDevices = 64;
static __device__ __align__(256) unsigned scratch[2 * kHandoffWords];   // 16 KiB on every device the library runs on
unsigned* g_scratch_ptr[kNoAllocMaxDevices];                             // address of `scratch` on each device
std::mutex g_scratch_mutex;

// The device's copy of `scratch`, looked up on the first call with that device current.
int scratch_on_current_device(unsigned** out)
{
  int dev = 0;
  CUDADMA_HIP_CHECK(hipGetDevice(&dev));
  CUDADMA_REQUIRE(dev >= 0 && dev < kNoAllocMaxDevices, "device %d is beyond the %d this entry point keeps staging memory for",
                  dev, kNoAllocMaxDevices);
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (g_scratch_ptr[dev] == nullptr) {
    unsigned* p = nullptr;
    CUDADMA_HIP_CHECK(hipGetSymbolAddress((void**)&p, HIP_SYMBOL(scratch)));
    CUDADMA_REQUIRE(p != nullptr, "hipGetSymbolAddress returned no address for the staging array");
    g_scratch_ptr[dev] = p;
  }
  *out = g_scratch_ptr[dev];
  return CUDADMA_OK;
}

}  // namespace

extern "C" int cudadma_selftest_global_handoff_noalloc(int* d_wrong, int phases, void* stream)
{
  CUDADMA_REQUIRE(d_wrong != nullptr && phases > 0, "NULL pointer or phases not positive");
  CUDADMA_REQUIRE(phases <= CUDADMA_NOALLOC_MAX_PHASES, "phases = %d is beyond the %d this entry point accepts", phases,
                  CUDADMA_NOALLOC_MAX_PHASES);
  unsigned* staging = nullptr;
  const int rc = scratch_on_current_device(&staging);
  if (rc != CUDADMA_OK) return rc;
  // Nothing in the array has to start at zero: every phase writes its 8 KiB of source before the DMA wavefronts read them
  // and the destination half is only read after the transfer of the same phase has signalled.
  hipLaunchKernelGGL(global_handoff, dim3(1), dim3(64 + kHandoffDmaThreads), 0, (hipStream_t)stream, staging,
                     staging + kHandoffWords, d_wrong, phases);
  CUDADMA_HIP_CHECK(hipGetLastError());
  return CUDADMA_OK;
}
