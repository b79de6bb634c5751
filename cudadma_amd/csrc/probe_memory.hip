// Streaming yardsticks without LDS and without a DMA object: what read-only, write-only and copy-shaped
// kernels reach on this part at a given launch shape, and the vendor's own device-to-device copy.  The benchmark
// reports them next to the DMA patterns, on the same buffers; the reference has nothing of the kind (its sweep
// scripts, src/perf/sequential/param_sweep.py:27-58, only vary its own kernels).
#include "workloads.hpp"

namespace {
using workloads::vec4_t;

constexpr int kThreads = 256;

template<bool NONTEMPORAL>
__global__ void __launch_bounds__(kThreads)
probe_read(const vec4_t* __restrict__ in, vec4_t* __restrict__ sink, const size_t n_vec)
{
  auto ld = [](const vec4_t* p) __attribute__((always_inline)) {
    if constexpr (NONTEMPORAL) return __builtin_nontemporal_load(p);
    else return *p;
  };
  vec4_t acc = {0u, 0u, 0u, 0u};
  const size_t stride = (size_t)gridDim.x * kThreads;
  size_t i = (size_t)blockIdx.x * kThreads + threadIdx.x;
  // four loads in flight per lane
  for (; i + 3 * stride < n_vec; i += 4 * stride) {
    const vec4_t a = ld(in + i), b = ld(in + i + stride), c = ld(in + i + 2 * stride), d = ld(in + i + 3 * stride);
    acc ^= a ^ b ^ c ^ d;
  }
  for (; i < n_vec; i += stride) acc ^= ld(in + i);
  // never true for the benchmark data (finite floats); keeps the loads alive
  if ((acc.x & acc.y & acc.z & acc.w) == 0xffffffffu && sink != nullptr) sink[threadIdx.x] = acc;
}

template<bool NONTEMPORAL>
__global__ void __launch_bounds__(kThreads)
probe_write(vec4_t* __restrict__ out, const size_t n_vec)
{
  const vec4_t one = {0x3f800000u, 0x3f800000u, 0x3f800000u, 0x3f800000u};
  const size_t stride = (size_t)gridDim.x * kThreads;
  for (size_t i = (size_t)blockIdx.x * kThreads + threadIdx.x; i < n_vec; i += stride) {
    if constexpr (NONTEMPORAL) __builtin_nontemporal_store(one, out + i);
    else out[i] = one;
  }
}

template<bool NONTEMPORAL>
__global__ void __launch_bounds__(kThreads)
probe_copy(const vec4_t* __restrict__ in, vec4_t* __restrict__ out, const size_t n_vec)
{
  const size_t stride = (size_t)gridDim.x * kThreads;
  for (size_t i = (size_t)blockIdx.x * kThreads + threadIdx.x; i < n_vec; i += stride) {
    if constexpr (NONTEMPORAL) __builtin_nontemporal_store(__builtin_nontemporal_load(in + i), out + i);
    else out[i] = in[i];
  }
}

__global__ void __launch_bounds__(64)
probe_clock(unsigned long long* __restrict__ ticks, const int iterations)
{
  float x = 1.0f + 1e-7f * threadIdx.x;
  const unsigned long long t0 = __builtin_readcyclecounter();           // s_memtime: shader clock
  const unsigned long long r0 = __builtin_amdgcn_s_memrealtime();       // constant 100 MHz
  for (int i = 0; i < iterations; ++i) x = __builtin_fmaf(x, 1.0000001f, 1e-9f);
  asm volatile("" :: "v"(x));                                           // the chain has to be finished before the second reading
  const unsigned long long t1 = __builtin_readcyclecounter();
  const unsigned long long r1 = __builtin_amdgcn_s_memrealtime();
  if (threadIdx.x == 0) {
    ticks[0] = t1 - t0;
    ticks[1] = r1 - r0;
  }
}

}  // namespace

extern "C" int cudadma_probe_clock(uint64_t* d_ticks, int iterations, void* stream)
{
  CUDADMA_REQUIRE(d_ticks != nullptr && cudadma_host::aligned_to(d_ticks, 8), "d_ticks must be an 8-byte aligned device pointer");
  CUDADMA_REQUIRE(iterations > 0, "iterations must be positive");
  hipLaunchKernelGGL(probe_clock, dim3(1), dim3(64), 0, (hipStream_t)stream, (unsigned long long*)d_ticks, iterations);
  CUDADMA_HIP_CHECK(hipGetLastError());
  return CUDADMA_OK;
}

extern "C" long long cudadma_probe_memory(int mode, const void* d_src, void* d_dst, size_t bytes, int workgroups,
                                          void* stream)
{
  if (mode < 0 || mode >= CUDADMA_PROBE_MODES) {
    cudadma_host::set_error("no probe mode %d", mode);
    return CUDADMA_ERANGE;
  }
  CUDADMA_REQUIRE(bytes > 0 && (bytes % 16) == 0, "bytes must be a positive multiple of 16");
  const bool reads = mode != CUDADMA_PROBE_WRITE && mode != CUDADMA_PROBE_WRITE_NONTEMPORAL;
  const bool writes = mode != CUDADMA_PROBE_READ && mode != CUDADMA_PROBE_READ_NONTEMPORAL;
  CUDADMA_REQUIRE((!reads || d_src != nullptr) && (!writes || d_dst != nullptr), "NULL pointer");
  CUDADMA_REQUIRE((!reads || cudadma_host::aligned_to(d_src, 16)) && (!writes || cudadma_host::aligned_to(d_dst, 16)),
                  "pointers must be 16-byte aligned");
  hipStream_t s = (hipStream_t)stream;
  if (mode == CUDADMA_PROBE_VENDOR_COPY) {
    // the runtime picks the launch shape (or a copy engine) itself
    CUDADMA_HIP_CHECK(hipMemcpyDtoDAsync((hipDeviceptr_t)d_dst, (hipDeviceptr_t)const_cast<void*>(d_src), bytes, s));
    return (long long)(2 * bytes);
  }
  CUDADMA_REQUIRE(workgroups > 0 && workgroups <= 65536, "workgroups must lie in 1..65536");
  const dim3 grid((unsigned)workgroups), block(kThreads);
  const size_t n_vec = bytes / 16;
  switch (mode) {
    case CUDADMA_PROBE_READ: hipLaunchKernelGGL(probe_read<false>, grid, block, 0, s, (const vec4_t*)d_src, (vec4_t*)d_dst, n_vec); break;
    case CUDADMA_PROBE_READ_NONTEMPORAL: hipLaunchKernelGGL(probe_read<true>, grid, block, 0, s, (const vec4_t*)d_src, (vec4_t*)d_dst, n_vec); break;
    case CUDADMA_PROBE_WRITE: hipLaunchKernelGGL(probe_write<false>, grid, block, 0, s, (vec4_t*)d_dst, n_vec); break;
    case CUDADMA_PROBE_WRITE_NONTEMPORAL: hipLaunchKernelGGL(probe_write<true>, grid, block, 0, s, (vec4_t*)d_dst, n_vec); break;
    case CUDADMA_PROBE_COPY: hipLaunchKernelGGL(probe_copy<false>, grid, block, 0, s, (const vec4_t*)d_src, (vec4_t*)d_dst, n_vec); break;
    default: hipLaunchKernelGGL(probe_copy<true>, grid, block, 0, s, (const vec4_t*)d_src, (vec4_t*)d_dst, n_vec); break;
  }
  CUDADMA_HIP_CHECK(hipGetLastError());
  return (long long)((reads ? bytes : 0) + (writes ? bytes : 0));
}
