// Shared host-side plumbing of libcudadma_amd.so: error text, HIP checks.
#pragma once

#include <hip/hip_runtime.h>
#include <cstdarg>
#include <cstdio>
#include "../../include/cudadma_amd.h"

namespace cudadma_host {

void set_error(const char* fmt, ...);

#define CUDADMA_HIP_CHECK(expr)                                                          \
  do {                                                                                   \
    hipError_t e_ = (expr);                                                              \
    if (e_ != hipSuccess) {                                                              \
      cudadma_host::set_error("%s failed: %s", #expr, hipGetErrorString(e_));            \
      return CUDADMA_ELAUNCH;                                                            \
    }                                                                                    \
  } while (0)

#define CUDADMA_REQUIRE(cond, ...)                                                       \
  do {                                                                                   \
    if (!(cond)) {                                                                       \
      cudadma_host::set_error(__VA_ARGS__);                                              \
      return CUDADMA_EINVAL;                                                             \
    }                                                                                    \
  } while (0)

inline bool aligned_to(const void* p, size_t a) { return (reinterpret_cast<uintptr_t>(p) % a) == 0; }

// The failure record of the DMA objects (hipdma::status_words_address in include/hipdma/base.hpp) exists once
// per translation unit; status_word.hpp registers each unit's accessor here so that cudadma_device_status()
// can read them all.  Called from static initialisers only.
typedef hipError_t (*status_address_fn)(unsigned** words);
void register_status_source(status_address_fn fn, const char* file);
struct StatusRegistrar {
  StatusRegistrar(status_address_fn fn, const char* file) { register_status_source(fn, file); }
};

}  // namespace cudadma_host
