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

}  // namespace cudadma_host
