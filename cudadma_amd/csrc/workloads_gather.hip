// Config 3: indirect gather of 128-byte records with CudaDMAIndirect, 32 records
// per LDS tile.  Shapes follow the warp-specialised kernels of
// src/tests/test_indirect/cudaDMA_test_indirect_v2.cu:52-120, made persistent
// and multi-buffered as src/examples/stencil/warp_specialized_manual_buffer.h:54-71.
// Two consumers:
//   copy   out[i] = table[idx[i]]                       (checks every moved byte)
//   rowsum out[t][j] = sum_r tile[r][j], r ascending     (the reported workload)
#include "workloads.hpp"

namespace {
using workloads::vec4_t;

constexpr int kRecBytes = 128;
constexpr int kRecFloats = kRecBytes / 4;
constexpr int kRecsPerTile = 32;
constexpr int kTileBytes = kRecBytes * kRecsPerTile;     // 4 KiB
constexpr int kDmaThreads = 128;
constexpr int kComputeThreads = 128;
constexpr int kBytesPerThread = kTileBytes / kDmaThreads;   // 32: two dwordx4 per DMA thread, one step

typedef CudaDMAIndirect<true, true, 16, kBytesPerThread, kRecBytes, kDmaThreads, kRecsPerTile> dma_t;

struct CopyConsumer {
  static constexpr bool kWritesEveryRecord = true;
  static __device__ __forceinline__ void run(const char* lds_tile, float* __restrict__ out, const long long tile,
                                             const dma_t& dma)
  {
    vec4_t v[2];
    const vec4_t* src = (const vec4_t*)lds_tile;
    v[0] = src[threadIdx.x];
    v[1] = src[threadIdx.x + kComputeThreads];
    dma.start_async_dma();
    vec4_t* dst = (vec4_t*)(out + tile * (kTileBytes / 4));
    dst[threadIdx.x] = v[0];
    dst[threadIdx.x + kComputeThreads] = v[1];
  }
};

struct RowsumConsumer {
  static constexpr bool kWritesEveryRecord = false;
  static __device__ __forceinline__ void run(const char* lds_tile, float* __restrict__ out, const long long tile,
                                             const dma_t& dma)
  {
    // 32 sums per tile: the first 32 compute threads each add one word of every record, record 0 first
    const float* t = (const float*)lds_tile;
    float acc = 0.0f;
    if (threadIdx.x < kRecFloats) {
      acc = t[threadIdx.x];
#pragma unroll
      for (int r = 1; r < kRecsPerTile; ++r) acc = acc + t[r * kRecFloats + threadIdx.x];
    }
    dma.start_async_dma();
    if (threadIdx.x < kRecFloats) out[tile * kRecFloats + threadIdx.x] = acc;
  }
};

// STAGES objects share the DMA threads; each has its own 4 KiB buffer.  With PREFETCH the index words of an
// object's next tile are requested right after its current tile (prefetch_index), one turn of the ring before
// they are used: the transfer that uses them then waits only for loads older than they are, and the elements of
// the other STAGES - 1 objects stay in flight across it.  Without it every start_xfer_async fetches its own index
// words and, a wavefront's loads returning in order, waits until nothing of the thread is in flight any more.
template<typename Consumer, int STAGES, bool PREFETCH = false>
__global__ void __launch_bounds__(kDmaThreads + kComputeThreads)
gather_manual(const float* __restrict__ table, const int* __restrict__ idx, float* __restrict__ out,
              const long long num_tiles)
{
  __shared__ __attribute__((aligned(16))) char buf[STAGES][kTileBytes];
  dma_t dma0(0, kComputeThreads, kComputeThreads);
  dma_t dma1(1, kComputeThreads, kComputeThreads);
  dma_t dma2(2, kComputeThreads, kComputeThreads);
  dma_t dma3(3, kComputeThreads, kComputeThreads);
  const long long stride = gridDim.x;
  const long long first = blockIdx.x;
#define HIPDMA_FOR_STAGES(...)                                                    \
  { constexpr int s = 0; dma_t& d = dma0; __VA_ARGS__ }                           \
  if constexpr (STAGES > 1) { constexpr int s = 1; dma_t& d = dma1; __VA_ARGS__ } \
  if constexpr (STAGES > 2) { constexpr int s = 2; dma_t& d = dma2; __VA_ARGS__ } \
  if constexpr (STAGES > 3) { constexpr int s = 3; dma_t& d = dma3; __VA_ARGS__ }
  if (dma0.owns_this_thread()) {
    long long t = first;
    if (t + (2 * STAGES - 1) * stride < num_tiles) {
      // Steady state with no branch around any load, entered from a prologue that has none either:
      // waiting for one stage then leaves the loads of the other stages in flight.
      if constexpr (PREFETCH) {
        // a prefetch beyond the last tile reads the last tile's words instead (never used): no branch
        const long long last = num_tiles - 1;
        HIPDMA_FOR_STAGES({ d.template prefetch_index<true>(idx + (t + s * stride) * kRecsPerTile); })
        HIPDMA_FOR_STAGES({
          d.template start_xfer_async_prefetched<true, LOAD_CACHE_ALL, STORE_LDS>(idx + (t + s * stride) * kRecsPerTile, table);
          d.template prefetch_index<true>(idx + (t + (s + STAGES) * stride) * kRecsPerTile);
        })
        do {
          HIPDMA_FOR_STAGES({
            d.template wait_xfer_finish<true, LOAD_CACHE_ALL, STORE_LDS>(buf[s]);
            d.template start_xfer_async_prefetched<true, LOAD_CACHE_ALL, STORE_LDS>(idx + (t + (s + STAGES) * stride) * kRecsPerTile, table);
            const long long ahead = t + (s + 2 * STAGES) * stride;
            d.template prefetch_index<true>(idx + (ahead < last ? ahead : last) * kRecsPerTile);
          })
          t += STAGES * stride;
        } while (t + (2 * STAGES - 1) * stride < num_tiles);
      } else {
        HIPDMA_FOR_STAGES({
          d.template start_xfer_async<true, LOAD_CACHE_ALL, STORE_LDS>(idx + (t + s * stride) * kRecsPerTile, table);
        })
        do {
          HIPDMA_FOR_STAGES({
            d.template wait_xfer_finish<true, LOAD_CACHE_ALL, STORE_LDS>(buf[s]);
            d.template start_xfer_async<true, LOAD_CACHE_ALL, STORE_LDS>(idx + (t + (s + STAGES) * stride) * kRecsPerTile, table);
          })
          t += STAGES * stride;
        } while (t + (2 * STAGES - 1) * stride < num_tiles);
      }
    } else {
      HIPDMA_FOR_STAGES({
        const long long tt = t + s * stride;
        if (tt < num_tiles) d.template start_xfer_async<true, LOAD_CACHE_ALL, STORE_LDS>(idx + tt * kRecsPerTile, table);
      })
    }
    // the last tiles of this workgroup
    for (; t < num_tiles; t += STAGES * stride) {
      HIPDMA_FOR_STAGES({
        const long long tt = t + s * stride;
        if (tt < num_tiles) {
          d.template wait_xfer_finish<true, LOAD_CACHE_ALL, STORE_LDS>(buf[s]);
          const long long nx = tt + STAGES * stride;
          if (nx < num_tiles) d.template start_xfer_async<true, LOAD_CACHE_ALL, STORE_LDS>(idx + nx * kRecsPerTile, table);
        }
      })
    }
  } else {
    HIPDMA_FOR_STAGES({ d.start_async_dma(); })
    for (long long t = first; t < num_tiles; t += STAGES * stride) {
      HIPDMA_FOR_STAGES({
        const long long tt = t + s * stride;
        if (tt < num_tiles) {
          d.wait_for_dma_finish();
          Consumer::run(buf[s], out, tt, d);
        }
      })
    }
  }
#undef HIPDMA_FOR_STAGES
}

template<typename Consumer>
__global__ void __launch_bounds__(kDmaThreads + kComputeThreads)
gather_single(const float* __restrict__ table, const int* __restrict__ idx, float* __restrict__ out,
              const long long num_tiles)
{
  __shared__ __attribute__((aligned(16))) char buf[kTileBytes];
  dma_t dma(0, kComputeThreads, kComputeThreads);
  if (dma.owns_this_thread()) {
    for (long long t = blockIdx.x; t < num_tiles; t += gridDim.x)
      dma.template execute_dma<true, LOAD_CACHE_ALL, STORE_LDS>(idx + t * kRecsPerTile, table, buf);
  } else {
    dma.start_async_dma();
    for (long long t = blockIdx.x; t < num_tiles; t += gridDim.x) {
      dma.wait_for_dma_finish();
      Consumer::run(buf, out, t, dma);
    }
  }
}

template<typename Consumer>
int launch_gather(const float* d_table, const int32_t* d_idx, float* d_out, size_t n_records, size_t n_idx,
                  int variant, void* stream)
{
  CUDADMA_REQUIRE((n_idx % kRecsPerTile) == 0, "n_idx (%zu) must be a multiple of %d", n_idx, kRecsPerTile);
  CUDADMA_REQUIRE(n_records > 0 && n_records <= 0x7fffffffull, "the table (%zu records) is indexed with int record numbers", n_records);
  if (variant < 0 || variant >= cudadma_num_variants(CUDADMA_WORKLOAD_GATHER)) {
    cudadma_host::set_error("gather has no variant %d", variant);
    return CUDADMA_ERANGE;
  }
  if (n_idx == 0) return CUDADMA_OK;
  CUDADMA_REQUIRE(d_table != nullptr && d_idx != nullptr && d_out != nullptr, "NULL pointer");
  CUDADMA_REQUIRE(cudadma_host::aligned_to(d_table, 16) && cudadma_host::aligned_to(d_out, 16), "pointers must be 16-byte aligned");
  const long long tiles = (long long)(n_idx / kRecsPerTile);
  hipStream_t s = (hipStream_t)stream;
  const dim3 block(kDmaThreads + kComputeThreads);
  // Workgroups per compute unit.  Objects that fetch their own index words drain the DMA wavefronts at every
  // transfer and need many workgroups to cover that (six with several objects, eight with one).  With the index
  // words requested ahead two objects and three workgroups are enough (0.634 ms on the configuration's 512 MiB
  // table, which the caches help to serve); a table several times the Infinity Cache wants four (0.724 ms against
  // 0.775 ms without the prefetch on 1.875 GiB).
  // The copy consumer writes as much as it reads and wants a shorter queue still: two (74.6 % on the 512 MiB table,
  // 69.5 % on 1.875 GiB, against 74.0 / 68.2 with three).
  const int ahead_wgs = Consumer::kWritesEveryRecord ? 2 : n_records * (size_t)kRecBytes <= (1ull << 30) ? 3 : 4;
  auto grid = [&](const int per_cu) { return dim3((unsigned)workloads::persistent_grid(tiles, per_cu)); };
  switch (variant) {
    case 0:
    case 6: hipLaunchKernelGGL((gather_manual<Consumer, 2, true>), grid(ahead_wgs), block, 0, s, d_table, d_idx, d_out, tiles); break;
    case 1: hipLaunchKernelGGL(gather_single<Consumer>, grid(8), block, 0, s, d_table, d_idx, d_out, tiles); break;
    case 2: hipLaunchKernelGGL((gather_manual<Consumer, 2>), grid(6), block, 0, s, d_table, d_idx, d_out, tiles); break;
    case 3: hipLaunchKernelGGL((gather_manual<Consumer, 4>), grid(6), block, 0, s, d_table, d_idx, d_out, tiles); break;
    case 4: hipLaunchKernelGGL((gather_manual<Consumer, 4, true>), grid(ahead_wgs), block, 0, s, d_table, d_idx, d_out, tiles); break;
    default: hipLaunchKernelGGL((gather_manual<Consumer, 3, true>), grid(ahead_wgs), block, 0, s, d_table, d_idx, d_out, tiles); break;
  }
  CUDADMA_HIP_CHECK(hipGetLastError());
  return CUDADMA_OK;
}

}  // namespace

extern "C" int cudadma_gather_copy(const float* d_table, const int32_t* d_idx, float* d_out, size_t n_records,
                                   size_t n_idx, int variant, void* stream)
{ return launch_gather<CopyConsumer>(d_table, d_idx, d_out, n_records, n_idx, variant, stream); }

extern "C" int cudadma_gather_rowsum(const float* d_table, const int32_t* d_idx, float* d_out, size_t n_records,
                                     size_t n_idx, int variant, void* stream)
{ return launch_gather<RowsumConsumer>(d_table, d_idx, d_out, n_records, n_idx, variant, stream); }
