// Error text and device queries of libcudadma_amd.so.
#include "common.hpp"
#include <mutex>
#include <vector>

namespace cudadma_host {

static thread_local char g_error[512] = "";
constexpr int kMaxDevices = 64;

void set_error(const char* fmt, ...)
{
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
}

struct StatusSource {
  status_address_fn address;
  const char* file;
  unsigned* words[kMaxDevices];     // this unit's words on each device, looked up once per device
};

static std::vector<StatusSource>& status_sources()
{
  static std::vector<StatusSource> v;
  return v;
}
static std::mutex g_status_mutex;   // constant-initialised: usable by registrars that run before this unit's own initialisers

// Called from static initialisers: of this library at load time, and of any library loaded later that instantiates
// DMA objects (the harness), possibly while another thread is inside cudadma_device_status().
void register_status_source(status_address_fn fn, const char* file)
{
  StatusSource s{};
  s.address = fn;
  s.file = file;
  std::lock_guard<std::mutex> lock(g_status_mutex);
  status_sources().push_back(s);
}

}  // namespace cudadma_host

extern "C" int cudadma_device_status(unsigned* status_bits, unsigned* waits_given_up, int clear, void* stream)
{
  using namespace cudadma_host;
  int dev = 0;
  CUDADMA_HIP_CHECK(hipGetDevice(&dev));
  CUDADMA_REQUIRE(dev >= 0 && dev < kMaxDevices, "device %d is beyond the %d this library keeps records for", dev, kMaxDevices);
  std::lock_guard<std::mutex> lock(g_status_mutex);
  for (StatusSource& s : status_sources())
    if (s.words[dev] == nullptr) CUDADMA_HIP_CHECK(s.address(&s.words[dev]));
  CUDADMA_HIP_CHECK(hipStreamSynchronize((hipStream_t)stream));
  unsigned bits = 0, count = 0;
  const unsigned zeros[2] = {0u, 0u};
  for (StatusSource& s : status_sources()) {
    unsigned w[2] = {0u, 0u};
    CUDADMA_HIP_CHECK(hipMemcpy(w, s.words[dev], sizeof(w), hipMemcpyDeviceToHost));
    bits |= w[0];
    count += w[1];
    if (clear && (w[0] != 0u || w[1] != 0u))
      CUDADMA_HIP_CHECK(hipMemcpy(s.words[dev], zeros, sizeof(zeros), hipMemcpyHostToDevice));
  }
  if (status_bits != nullptr) *status_bits = bits;
  if (waits_given_up != nullptr) *waits_given_up = count;
  return CUDADMA_OK;
}

extern "C" int cudadma_device_status_sources(void)
{
  std::lock_guard<std::mutex> lock(cudadma_host::g_status_mutex);
  return (int)cudadma_host::status_sources().size();
}

extern "C" const char* cudadma_last_error(void) { return cudadma_host::g_error; }

extern "C" int cudadma_device_cus(void)
{
  int dev = 0;
  CUDADMA_HIP_CHECK(hipGetDevice(&dev));
  hipDeviceProp_t prop;
  CUDADMA_HIP_CHECK(hipGetDeviceProperties(&prop, dev));
  return prop.multiProcessorCount;
}
