// Shared pieces of the benchmark workloads: persistent-grid sizing, the variant
// tables and the seeded input generators' hash.
#pragma once

#include "common.hpp"
#include "../../include/hipDMA.h"
#include "status_word.hpp"

namespace workloads {

// Workgroups to launch for a persistent kernel: CUs x (knob or the kernel's
// default), never more than there are work items.
int persistent_grid(long long work_items, int default_wg_per_cu);
// Compute units of the current device, queried once.
int device_cus();

// Value of a named knob, or `fallback` while it is unset (0).
int tuning(const char* name, int fallback);

struct VariantInfo {
  const char* name;
};

__host__ __device__ inline unsigned long long splitmix64(unsigned long long x)
{
  unsigned long long z = x + 0x9E3779B97F4A7C15ull;
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  return z ^ (z >> 31);
}
__host__ __device__ inline unsigned hash32(unsigned long long seed, unsigned long long i)
{
  return (unsigned)(splitmix64(seed + i) >> 32);
}

typedef hipdma::detail::u32x4_t vec4_t;

}  // namespace workloads
