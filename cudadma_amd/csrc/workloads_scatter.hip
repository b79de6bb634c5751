// Scatter of 128-byte records, the transfer direction the other workloads do not time:
//   table[idx[i]] = records[i]
// The compute wavefronts are the producers here: they bring a tile of 32 dense records
// into an LDS buffer and hand it over; the DMA wavefronts move it LDS -> global with
// CudaDMAIndirect<false> (addressing of include/cudaDMAv2.h:10199-10217, generic loads as
// in :107-114 since the source is not global memory).  The hand-over is the base class's
// own pair of calls (include/cudaDMAv2.h:1329-1347) on a cudaDMACustom guard per buffer,
// read the other way round: start_async_dma() says "the buffer is full",
// wait_for_dma_finish() says "it has been drained".  Kernel shapes as in the gather
// workload (src/tests/test_indirect/cudaDMA_test_indirect_v2.cu:52-120 made persistent).
#include "workloads.hpp"

namespace {
using workloads::vec4_t;

constexpr int kRecBytes = 128;
constexpr int kRecsPerTile = 32;
constexpr int kTileBytes = kRecBytes * kRecsPerTile;     // 4 KiB
constexpr int kDmaThreads = 128;
constexpr int kComputeThreads = 128;
constexpr int kBytesPerThread = kTileBytes / kDmaThreads;   // 32: two dwordx4 per DMA thread, one step

typedef CudaDMAIndirect<false, false, 16, kBytesPerThread, kRecBytes, kDmaThreads, kRecsPerTile> scatter_t;

// The dense tile `tile` in two dwordx4 per compute thread.
struct TileRegs {
  vec4_t v[2];
  __device__ __forceinline__ void load(const float* __restrict__ records, const long long tile)
  {
    const vec4_t* src = (const vec4_t*)(records + tile * (kTileBytes / 4));
    v[0] = __builtin_nontemporal_load(src + threadIdx.x);
    v[1] = __builtin_nontemporal_load(src + threadIdx.x + kComputeThreads);
  }
  __device__ __forceinline__ void put(char* lds_tile) const
  {
    vec4_t* dst = (vec4_t*)lds_tile;
    dst[threadIdx.x] = v[0];
    dst[threadIdx.x + kComputeThreads] = v[1];
  }
};

// STAGES buffers, each with its guard; the DMA wavefronts drain them in turn.  (Requesting the index words of the
// next tile ahead of the current tile's stores, prefetch_index between the two phases, changes nothing here at
// any number of workgroups: 36.6 / 62.6 / 66.8 / 66.5 % of 8 TB/s at one to four per compute unit either way.)
template<int STAGES>
__global__ void __launch_bounds__(kDmaThreads + kComputeThreads)
scatter_manual(const float* __restrict__ records, const int* __restrict__ idx, float* __restrict__ table,
               const long long num_tiles)
{
  __shared__ __attribute__((aligned(16))) char buf[STAGES][kTileBytes];
  cudaDMACustom g0(0, kDmaThreads, kComputeThreads, kComputeThreads);
  cudaDMACustom g1(1, kDmaThreads, kComputeThreads, kComputeThreads);
  cudaDMACustom g2(2, kDmaThreads, kComputeThreads, kComputeThreads);
  cudaDMACustom g3(3, kDmaThreads, kComputeThreads, kComputeThreads);
  scatter_t dma(0, kComputeThreads);
  const long long stride = gridDim.x;
  const long long first = blockIdx.x;
#define HIPDMA_FOR_STAGES(...)                                                           \
  { constexpr int s = 0; cudaDMACustom& g = g0; __VA_ARGS__ }                            \
  if constexpr (STAGES > 1) { constexpr int s = 1; cudaDMACustom& g = g1; __VA_ARGS__ }  \
  if constexpr (STAGES > 2) { constexpr int s = 2; cudaDMACustom& g = g2; __VA_ARGS__ }  \
  if constexpr (STAGES > 3) { constexpr int s = 3; cudaDMACustom& g = g3; __VA_ARGS__ }
  if (g0.owns_this_thread()) {
    for (long long t = first; t < num_tiles; t += STAGES * stride) {
      HIPDMA_FOR_STAGES({
        const long long tt = t + s * stride;
        if (tt < num_tiles) {
          g.wait_for_dma_start();                       // the producers have filled buf[s]
          dma.template execute_dma<false, LOAD_CACHE_ALL, STORE_CACHE_STREAMING>(idx + tt * kRecsPerTile, buf[s], table);
          g.finish_async_dma();                         // its contents are in registers or on their way
        }
      })
    }
  } else {
    TileRegs cur;
    cur.load(records, first);
    bool refill = false;
    for (long long t = first; t < num_tiles; t += STAGES * stride) {
      HIPDMA_FOR_STAGES({
        const long long tt = t + s * stride;
        if (tt < num_tiles) {
          if (refill) g.wait_for_dma_finish();          // the previous tile in buf[s] has been drained
          cur.put(buf[s]);
          g.start_async_dma();
          if (tt + stride < num_tiles) cur.load(records, tt + stride);
        }
      })
      refill = true;
    }
    // every hand-over is answered before the producers leave
    HIPDMA_FOR_STAGES({ if (first + s * stride < num_tiles) g.wait_for_dma_finish(); })
  }
#undef HIPDMA_FOR_STAGES
}

// No DMA wavefronts: all four wavefronts bring the tile into LDS, meet, and all four
// scatter it with an object that is not warp-specialised
// (src/examples/stencil/non_warp_specialized_single_buffer.h:47-57).
__global__ void __launch_bounds__(kDmaThreads + kComputeThreads)
scatter_not_specialized(const float* __restrict__ records, const int* __restrict__ idx, float* __restrict__ table,
                        const long long num_tiles)
{
  constexpr int kThreads = kDmaThreads + kComputeThreads;
  __shared__ __attribute__((aligned(16))) char buf[kTileBytes];
  CudaDMAIndirect<false, false, 16, kTileBytes / kThreads, kRecBytes, kThreads, kRecsPerTile> dma;
  for (long long t = blockIdx.x; t < num_tiles; t += gridDim.x) {
    const vec4_t v = __builtin_nontemporal_load((const vec4_t*)(records + t * (kTileBytes / 4)) + threadIdx.x);
    ((vec4_t*)buf)[threadIdx.x] = v;
    __syncthreads();
    dma.template execute_dma<false, LOAD_CACHE_ALL, STORE_WRITE_BACK>(idx + t * kRecsPerTile, buf, table);
    __syncthreads();
  }
}

}  // namespace

extern "C" int cudadma_scatter_copy(const float* d_records, const int32_t* d_idx, float* d_table, size_t n_records,
                                    size_t n_idx, int variant, void* stream)
{
  CUDADMA_REQUIRE((n_idx % kRecsPerTile) == 0, "n_idx (%zu) must be a multiple of %d", n_idx, kRecsPerTile);
  CUDADMA_REQUIRE(n_records > 0 && n_records <= 0x7fffffffull, "the table (%zu records) is indexed with int record numbers", n_records);
  if (variant < 0 || variant >= cudadma_num_variants(CUDADMA_WORKLOAD_SCATTER)) {
    cudadma_host::set_error("scatter has no variant %d", variant);
    return CUDADMA_ERANGE;
  }
  if (n_idx == 0) return CUDADMA_OK;
  CUDADMA_REQUIRE(d_records != nullptr && d_idx != nullptr && d_table != nullptr, "NULL pointer");
  CUDADMA_REQUIRE(cudadma_host::aligned_to(d_records, 16) && cudadma_host::aligned_to(d_table, 16), "pointers must be 16-byte aligned");
  const long long tiles = (long long)(n_idx / kRecsPerTile);
  hipStream_t s = (hipStream_t)stream;
  const dim3 block(kDmaThreads + kComputeThreads);
  // workgroups per compute unit: four where several tiles are buffered, eight where one is
  const dim3 few(workloads::persistent_grid(tiles, 4)), many(workloads::persistent_grid(tiles, 8));
  switch (variant) {
    case 0: hipLaunchKernelGGL(scatter_manual<4>, few, block, 0, s, d_records, d_idx, d_table, tiles); break;
    case 1: hipLaunchKernelGGL(scatter_manual<1>, many, block, 0, s, d_records, d_idx, d_table, tiles); break;
    case 2: hipLaunchKernelGGL(scatter_manual<2>, few, block, 0, s, d_records, d_idx, d_table, tiles); break;
    default: hipLaunchKernelGGL(scatter_not_specialized, many, block, 0, s, d_records, d_idx, d_table, tiles); break;
  }
  CUDADMA_HIP_CHECK(hipGetLastError());
  return CUDADMA_OK;
}
