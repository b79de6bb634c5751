// Error text and device queries of libcudadma_amd.so.
#include "common.hpp"

namespace cudadma_host {

static thread_local char g_error[512] = "";

void set_error(const char* fmt, ...)
{
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
}

}  // namespace cudadma_host

extern "C" const char* cudadma_last_error(void) { return cudadma_host::g_error; }

extern "C" int cudadma_device_cus(void)
{
  int dev = 0;
  CUDADMA_HIP_CHECK(hipGetDevice(&dev));
  hipDeviceProp_t prop;
  CUDADMA_HIP_CHECK(hipGetDeviceProperties(&prop, dev));
  return prop.multiProcessorCount;
}
