// Config 1: tiled copy through LDS with CudaDMASequential, plus the seeded
// input generators and the plain copy used as the bandwidth yardstick.
// Kernel shapes follow src/perf/sequential/perf_sequential.cu:52-223
// (non_specialized / single_buffer / double_buffer / manual_buffer), with a
// consumer that really writes the tile back instead of a dead branch.
#include "workloads.hpp"

namespace {
using workloads::vec4_t;

constexpr int kTileBytes = 16 * 1024;
constexpr int kDmaThreads = 128;
constexpr int kComputeThreads = 128;
constexpr int kTileVecs = kTileBytes / 16;
constexpr int kVecsPerConsumer = kTileVecs / kComputeThreads;   // 8 ds_read_b128 per compute thread
constexpr size_t kCacheAssistedBytes = 192u << 20;             // read + written bytes that still sit in the 256 MB Infinity Cache

// Consumer: LDS tile -> registers, release the buffer, registers -> global (STREAM: non-temporal stores).
template<bool STREAM = false, typename Dma>
__device__ __forceinline__ void drain_tile(const vec4_t* lds_tile, vec4_t* __restrict__ out_tile, const Dma& dma)
{
  vec4_t v[kVecsPerConsumer];
#pragma unroll
  for (int k = 0; k < kVecsPerConsumer; ++k) v[k] = lds_tile[threadIdx.x + k * kComputeThreads];
  dma.start_async_dma();
#pragma unroll
  for (int k = 0; k < kVecsPerConsumer; ++k) {
    if constexpr (STREAM) __builtin_nontemporal_store(v[k], out_tile + threadIdx.x + k * kComputeThreads);
    else out_tile[threadIdx.x + k * kComputeThreads] = v[k];
  }
}

// variants 0 and 3: one DMA group, two objects, two-phase calls
template<int STORE_QUAL>
__global__ void __launch_bounds__(kDmaThreads + kComputeThreads)
copy_manual_double(const char* __restrict__ in, char* __restrict__ out, const int num_tiles)
{
  __shared__ __attribute__((aligned(16))) vec4_t buf0[kTileVecs];
  __shared__ __attribute__((aligned(16))) vec4_t buf1[kTileVecs];
  typedef CudaDMASequential<true, 16, kTileBytes / kDmaThreads, kTileBytes, kDmaThreads> dma_t;
  dma_t dma0(0, kComputeThreads, kComputeThreads);
  dma_t dma1(1, kComputeThreads, kComputeThreads);
  const int stride = gridDim.x;
  if (dma0.owns_this_thread()) {
    int t = blockIdx.x;
    if (t + 3 * stride < num_tiles) {
      // Steady state with no branch around any load, entered from a prologue that has none either:
      // the wait for one object's tile then leaves the other object's loads in flight.
      dma0.template start_xfer_async<true, LOAD_CACHE_ALL, STORE_QUAL>(in + (size_t)t * kTileBytes);
      dma1.template start_xfer_async<true, LOAD_CACHE_ALL, STORE_QUAL>(in + (size_t)(t + stride) * kTileBytes);
      do {
        dma0.template wait_xfer_finish<true, LOAD_CACHE_ALL, STORE_QUAL>(buf0);
        dma0.template start_xfer_async<true, LOAD_CACHE_ALL, STORE_QUAL>(in + (size_t)(t + 2 * stride) * kTileBytes);
        dma1.template wait_xfer_finish<true, LOAD_CACHE_ALL, STORE_QUAL>(buf1);
        dma1.template start_xfer_async<true, LOAD_CACHE_ALL, STORE_QUAL>(in + (size_t)(t + 3 * stride) * kTileBytes);
        t += 2 * stride;
      } while (t + 3 * stride < num_tiles);
    } else {
      if (t < num_tiles) dma0.template start_xfer_async<true, LOAD_CACHE_ALL, STORE_QUAL>(in + (size_t)t * kTileBytes);
      if (t + stride < num_tiles)
        dma1.template start_xfer_async<true, LOAD_CACHE_ALL, STORE_QUAL>(in + (size_t)(t + stride) * kTileBytes);
    }
    // the last tiles of this workgroup
    for (; t < num_tiles; t += 2 * stride) {
      dma0.template wait_xfer_finish<true, LOAD_CACHE_ALL, STORE_QUAL>(buf0);
      if (t + 2 * stride < num_tiles)
        dma0.template start_xfer_async<true, LOAD_CACHE_ALL, STORE_QUAL>(in + (size_t)(t + 2 * stride) * kTileBytes);
      if (t + stride < num_tiles) {
        dma1.template wait_xfer_finish<true, LOAD_CACHE_ALL, STORE_QUAL>(buf1);
        if (t + 3 * stride < num_tiles)
          dma1.template start_xfer_async<true, LOAD_CACHE_ALL, STORE_QUAL>(in + (size_t)(t + 3 * stride) * kTileBytes);
      }
    }
  } else {
    dma0.start_async_dma();
    dma1.start_async_dma();
    for (int t = blockIdx.x; t < num_tiles; t += 2 * stride) {
      dma0.wait_for_dma_finish();
      drain_tile(buf0, (vec4_t*)(out + (size_t)t * kTileBytes), dma0);
      if (t + stride < num_tiles) {
        dma1.wait_for_dma_finish();
        drain_tile(buf1, (vec4_t*)(out + (size_t)(t + stride) * kTileBytes), dma1);
      }
    }
  }
}

// variant 1: one object, one buffer.  execute_dma requests a tile into the DMA wavefronts' registers before it
// waits for the buffer, so the double buffer is the LDS tile plus those registers.  STREAM (used for working sets
// beyond the Infinity Cache): streaming loads and non-temporal stores, neither side is read again.
// CHUNKED: a workgroup takes a contiguous run of tiles instead of every gridDim.x-th one.  The tiles in flight at one
// time are then spread over the whole buffer instead of forming one window that moves through it, and the speed
// no longer depends on how source and destination lie relative to each other (with the moving window, a 1 GiB
// copy ran between 0.350 and 0.440 ms depending on the distance between the two buffers modulo 64 MiB: reads and
// writes of the same window meet in the same memory channels and banks).
template<bool STREAM, bool CHUNKED = false>
__global__ void __launch_bounds__(kDmaThreads + kComputeThreads)
copy_single(const char* __restrict__ in, char* __restrict__ out, const int num_tiles)
{
  __shared__ __attribute__((aligned(16))) vec4_t buf[kTileVecs];
  CudaDMASequential<true, 16, kTileBytes / kDmaThreads, kTileBytes, kDmaThreads> dma(0, kComputeThreads, kComputeThreads);
  constexpr int kLoad = STREAM ? LOAD_CACHE_STREAMING : LOAD_CACHE_ALL;
  const int per = (num_tiles + (int)gridDim.x - 1) / (int)gridDim.x;
  const int first = CHUNKED ? (int)blockIdx.x * per : (int)blockIdx.x;
  const int step = CHUNKED ? 1 : (int)gridDim.x;
  const int end = CHUNKED ? ((first + per < num_tiles) ? first + per : num_tiles) : num_tiles;
  if (dma.owns_this_thread()) {
    for (int t = first; t < end; t += step)
      dma.template execute_dma<true, kLoad, STORE_LDS>(in + (size_t)t * kTileBytes, buf);
  } else {
    dma.start_async_dma();
    for (int t = first; t < end; t += step) {
      dma.wait_for_dma_finish();
      drain_tile<STREAM>(buf, (vec4_t*)(out + (size_t)t * kTileBytes), dma);
    }
  }
}

// variant 2: two DMA groups of one wavefront, each with its own object and buffer
__global__ void __launch_bounds__(kDmaThreads + kComputeThreads)
copy_double(const char* __restrict__ in, char* __restrict__ out, const int num_tiles)
{
  __shared__ __attribute__((aligned(16))) vec4_t buf0[kTileVecs];
  __shared__ __attribute__((aligned(16))) vec4_t buf1[kTileVecs];
  constexpr int kGroup = kDmaThreads / 2;
  typedef CudaDMASequential<true, 16, kTileBytes / kGroup / 2, kTileBytes, kGroup> dma_t;   // two steps of 128 B
  dma_t dma0(0, kComputeThreads, kComputeThreads);
  dma_t dma1(1, kComputeThreads, kComputeThreads + kGroup);
  const int stride = gridDim.x;
  if (dma0.owns_this_thread()) {
    for (int t = blockIdx.x; t < num_tiles; t += 2 * stride)
      dma0.template execute_dma<true, LOAD_CACHE_ALL, STORE_LDS>(in + (size_t)t * kTileBytes, buf0);
  } else if (dma1.owns_this_thread()) {
    for (int t = blockIdx.x + stride; t < num_tiles; t += 2 * stride)
      dma1.template execute_dma<true, LOAD_CACHE_ALL, STORE_LDS>(in + (size_t)t * kTileBytes, buf1);
  } else {
    dma0.start_async_dma();
    dma1.start_async_dma();
    for (int t = blockIdx.x; t < num_tiles; t += 2 * stride) {
      dma0.wait_for_dma_finish();
      drain_tile(buf0, (vec4_t*)(out + (size_t)t * kTileBytes), dma0);
      if (t + stride < num_tiles) {
        dma1.wait_for_dma_finish();
        drain_tile(buf1, (vec4_t*)(out + (size_t)(t + stride) * kTileBytes), dma1);
      }
    }
  }
}

// variant 4: the form that is not warp-specialised (non_specialized, perf_sequential.cu:52-76)
__global__ void __launch_bounds__(kDmaThreads + kComputeThreads)
copy_not_specialized(const char* __restrict__ in, char* __restrict__ out, const int num_tiles)
{
  __shared__ __attribute__((aligned(16))) vec4_t buf[kTileVecs];
  constexpr int kThreads = kDmaThreads + kComputeThreads;
  CudaDMASequential<false, 16, kTileBytes / kThreads, kTileBytes, kThreads> dma;
  for (int t = blockIdx.x; t < num_tiles; t += gridDim.x) {
    dma.template execute_dma<true, LOAD_CACHE_ALL, STORE_LDS>(in + (size_t)t * kTileBytes, buf);
    __syncthreads();
    vec4_t v[kTileVecs / kThreads];
#pragma unroll
    for (int k = 0; k < kTileVecs / kThreads; ++k) v[k] = buf[threadIdx.x + k * kThreads];
    __syncthreads();
    vec4_t* o = (vec4_t*)(out + (size_t)t * kTileBytes);
#pragma unroll
    for (int k = 0; k < kTileVecs / kThreads; ++k) o[threadIdx.x + k * kThreads] = v[k];
  }
}

__global__ void __launch_bounds__(256)
plain_copy_kernel(const vec4_t* __restrict__ in, vec4_t* __restrict__ out, const size_t n_vec)
{
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  // four independent loads in flight per lane
  for (; i + 3 * stride < n_vec; i += 4 * stride) {
    const vec4_t a = in[i], b = in[i + stride], c = in[i + 2 * stride], d = in[i + 3 * stride];
    out[i] = a; out[i + stride] = b; out[i + 2 * stride] = c; out[i + 3 * stride] = d;
  }
  for (; i < n_vec; i += stride) out[i] = in[i];
}

__global__ void __launch_bounds__(256)
fill_uniform_kernel(float* __restrict__ dst, const size_t n, const unsigned long long seed)
{
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride)
    dst[i] = (float)(workloads::hash32(seed, i) >> 8) * (1.0f / 8388608.0f) - 1.0f;
}

// normal(0,1) by Box-Muller on two hashes, in double precision, rounded to float and then to bf16 (nearest even):
// the operations of the host statement in the same order.  Double-precision log, cos and sqrt may differ from the
// host library's in their last bit; after the two roundings a difference survives in about one of 2^40 values.
__global__ void __launch_bounds__(256)
fill_normal_bf16_kernel(unsigned short* __restrict__ dst, const size_t n, const unsigned long long seed)
{
#pragma clang fp contract(off)
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
    const double u1 = ((double)(workloads::hash32(seed, 2ull * i) >> 8) + 1.0) / 16777216.0;
    const double u2 = (double)(workloads::hash32(seed, 2ull * i + 1ull) >> 8) / 16777216.0;
    const float v = (float)(sqrt(-2.0 * log(u1)) * cos(6.283185307179586476925286766559 * u2));
    unsigned u = __float_as_uint(v);
    u += 0x7fffu + ((u >> 16) & 1u);          // the value is finite: u1 > 0
    dst[i] = (unsigned short)(u >> 16);
  }
}

__global__ void __launch_bounds__(256)
fill_indices_kernel(int* __restrict__ dst, const size_t n, const unsigned n_records, const unsigned long long seed)
{
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
    size_t j = i;
    const unsigned r = workloads::hash32(seed ^ 0x5bd1e995u, i);
    if (i > 1024 && (r % 10u) == 0u) j = i - 1u - ((r / 10u) % 1024u);
    dst[i] = (int)(workloads::hash32(seed, j) % n_records);
  }
}

__global__ void __launch_bounds__(256)
fill_permutation_kernel(int* __restrict__ dst, const int log2_n, const unsigned long long k0,
                        const unsigned long long k1)
{
  const unsigned long long n = 1ull << log2_n, mask = n - 1;
  const int h = (log2_n + 1) / 2;
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
    unsigned long long x = i;
    x = (x * ((k0 & 0xffffffffull) | 1ull) + (k0 >> 32)) & mask;
    x ^= x >> h;
    x = (x * ((k1 & 0xffffffffull) | 1ull) + (k1 >> 32)) & mask;
    x ^= x >> h;
    x = (x * 0x9E3779B1ull) & mask;
    dst[i] = (int)x;
  }
}

}  // namespace

extern "C" int cudadma_fill_permutation(int32_t* d_dst, int log2_n, uint64_t seed, void* stream)
{
  CUDADMA_REQUIRE(log2_n >= 1 && log2_n <= 31, "log2_n (%d) must lie in 1..31", log2_n);
  CUDADMA_REQUIRE(d_dst != nullptr, "d_dst is NULL");
  const size_t n = (size_t)1 << log2_n;
  const int grid = workloads::persistent_grid((long long)((n + 255) / 256), 8);
  hipLaunchKernelGGL(fill_permutation_kernel, dim3(grid), dim3(256), 0, (hipStream_t)stream, d_dst, log2_n,
                     workloads::splitmix64(seed), workloads::splitmix64(seed + 1));
  CUDADMA_HIP_CHECK(hipGetLastError());
  return CUDADMA_OK;
}

extern "C" int cudadma_fill_uniform(float* d_dst, size_t n, uint64_t seed, void* stream)
{
  CUDADMA_REQUIRE(d_dst != nullptr || n == 0, "d_dst is NULL");
  if (n == 0) return CUDADMA_OK;
  const int grid = workloads::persistent_grid((long long)((n + 255) / 256), 8);
  hipLaunchKernelGGL(fill_uniform_kernel, dim3(grid), dim3(256), 0, (hipStream_t)stream, d_dst, n,
                     (unsigned long long)seed);
  CUDADMA_HIP_CHECK(hipGetLastError());
  return CUDADMA_OK;
}

extern "C" int cudadma_fill_normal_bf16(uint16_t* d_dst, size_t n, uint64_t seed, void* stream)
{
  CUDADMA_REQUIRE(d_dst != nullptr || n == 0, "d_dst is NULL");
  if (n == 0) return CUDADMA_OK;
  const int grid = workloads::persistent_grid((long long)((n + 255) / 256), 8);
  hipLaunchKernelGGL(fill_normal_bf16_kernel, dim3(grid), dim3(256), 0, (hipStream_t)stream, d_dst, n,
                     (unsigned long long)seed);
  CUDADMA_HIP_CHECK(hipGetLastError());
  return CUDADMA_OK;
}

extern "C" int cudadma_fill_indices(int32_t* d_dst, size_t n, uint32_t n_records, uint64_t seed, void* stream)
{
  CUDADMA_REQUIRE(d_dst != nullptr || n == 0, "d_dst is NULL");
  CUDADMA_REQUIRE(n_records > 0, "n_records must be positive");
  if (n == 0) return CUDADMA_OK;
  const int grid = workloads::persistent_grid((long long)((n + 255) / 256), 8);
  hipLaunchKernelGGL(fill_indices_kernel, dim3(grid), dim3(256), 0, (hipStream_t)stream, d_dst, n, n_records,
                     (unsigned long long)seed);
  CUDADMA_HIP_CHECK(hipGetLastError());
  return CUDADMA_OK;
}

extern "C" int cudadma_plain_copy(const void* d_src, void* d_dst, size_t bytes, void* stream)
{
  CUDADMA_REQUIRE((bytes % 16) == 0, "bytes must be a multiple of 16");
  if (bytes == 0) return CUDADMA_OK;
  CUDADMA_REQUIRE(d_src != nullptr && d_dst != nullptr, "NULL pointer");
  CUDADMA_REQUIRE(cudadma_host::aligned_to(d_src, 16) && cudadma_host::aligned_to(d_dst, 16), "pointers must be 16-byte aligned");
  const size_t n_vec = bytes / 16;
  const int grid = workloads::persistent_grid((long long)((n_vec + 255) / 256), 8);
  hipLaunchKernelGGL(plain_copy_kernel, dim3(grid), dim3(256), 0, (hipStream_t)stream, (const vec4_t*)d_src,
                     (vec4_t*)d_dst, n_vec);
  CUDADMA_HIP_CHECK(hipGetLastError());
  return CUDADMA_OK;
}

extern "C" int cudadma_sequential_copy(const float* d_in, float* d_out, size_t bytes, int variant, void* stream)
{
  CUDADMA_REQUIRE((bytes % kTileBytes) == 0, "bytes (%zu) must be a multiple of the 16 KiB tile", bytes);
  CUDADMA_REQUIRE(bytes / kTileBytes <= 0x7fffffff, "too many tiles");
  if (variant < 0 || variant >= cudadma_num_variants(CUDADMA_WORKLOAD_SEQUENTIAL)) {
    cudadma_host::set_error("sequential copy has no variant %d", variant);
    return CUDADMA_ERANGE;
  }
  if (bytes == 0) return CUDADMA_OK;
  CUDADMA_REQUIRE(d_in != nullptr && d_out != nullptr, "NULL pointer");
  CUDADMA_REQUIRE(cudadma_host::aligned_to(d_in, 16) && cudadma_host::aligned_to(d_out, 16), "pointers must be 16-byte aligned");
  const int tiles = (int)(bytes / kTileBytes);
  const char* in = (const char*)d_in;
  char* out = (char*)d_out;
  hipStream_t s = (hipStream_t)stream;
  const dim3 block(kDmaThreads + kComputeThreads);
  switch (variant) {
    case 0:
      // Two operating points, as for every read + write stream on this part: a working set that the 256 MB Infinity
      // Cache holds from launch to launch wants many tiles in flight (two LDS tiles, four workgroups per compute unit);
      // beyond it the memory system serves a short queue better (one LDS tile, two workgroups per compute unit,
      // streaming loads and non-temporal stores: 1 GiB in 0.353 ms against 0.408 ms).
      if (2 * bytes <= kCacheAssistedBytes)
        hipLaunchKernelGGL(copy_manual_double<STORE_LDS>, dim3(workloads::persistent_grid(tiles, 4)), block, 0, s, in, out, tiles);
      else
        hipLaunchKernelGGL(copy_single<true>, dim3(workloads::persistent_grid(tiles, 2)), block, 0, s, in, out, tiles);
      break;
    case 1: hipLaunchKernelGGL(copy_single<false>, dim3(workloads::persistent_grid(tiles, 8)), block, 0, s, in, out, tiles); break;
    case 5: hipLaunchKernelGGL(copy_single<true>, dim3(workloads::persistent_grid(tiles, 2)), block, 0, s, in, out, tiles); break;
    case 6: hipLaunchKernelGGL((copy_single<true, true>), dim3(workloads::persistent_grid(tiles, 2)), block, 0, s, in, out, tiles); break;
    case 2: hipLaunchKernelGGL(copy_double, dim3(workloads::persistent_grid(tiles, 4)), block, 0, s, in, out, tiles); break;
    case 3: hipLaunchKernelGGL(copy_manual_double<STORE_LDS_DIRECT>, dim3(workloads::persistent_grid(tiles, 4)), block, 0, s, in, out, tiles); break;
    default: hipLaunchKernelGGL(copy_not_specialized, dim3(workloads::persistent_grid(tiles, 8)), block, 0, s, in, out, tiles); break;
  }
  CUDADMA_HIP_CHECK(hipGetLastError());
  return CUDADMA_OK;
}
