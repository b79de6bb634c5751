// Config 4: 8th-order, 25-point star stencil over a 3-D grid, 32x32 tiles
// marched along z.  The buffering idioms are those of
// src/examples/stencil/warp_specialized_double_buffer.h:25-106 and
// src/examples/stencil/non_warp_specialized_single_buffer.h:34-58; the ring of
// ghost cells comes through CudaDMAHalo (include/cudaDMA.h:3653-4156), the
// stencil itself is the textbook one, not stencil_math.h.
//
// Per output plane z a compute thread owns four cells of the tile.  Their z
// neighbours live in a 9-deep register queue fed by one coalesced global load
// per cell and plane; the centre plane is shared through LDS: the interior is
// written by the compute threads themselves, the 4-wide ring around it by the
// DMA wavefront.  Two LDS planes alternate so the ring of plane z+1 lands
// while plane z is being computed.
#include "workloads.hpp"

namespace {

constexpr int kR = 4;
constexpr int kTX = 32, kTY = 32;
constexpr int kPitch = kTX + 2 * kR;                 // 40 floats per LDS row
constexpr int kPlaneFloats = kPitch * (kTY + 2 * kR);
constexpr int kComputeThreads = 256;
constexpr int kDmaThreads = 64;
constexpr int kCells = kTX * kTY / kComputeThreads;   // 4 cells per compute thread
constexpr int kRowsPerPass = kComputeThreads / kTX;   // 8

// ring of a 32x32 float tile: 8 rows x 8 chunks + 64 strips x 1 chunk = 128 chunks of 16 B = 2 per DMA thread
typedef CudaDMAHalo<true, 16, 32, 4, kDmaThreads, kR, false, kTX, kTY> halo_ws_t;
typedef CudaDMAHalo<false, 16, 16, 4, kComputeThreads, kR, false, kTX, kTY> halo_all_t;

struct Coeffs {
  float c0, c1, c2, c3, c4;
};

// One cell: same operations in the same order as the host statement, no fused multiply-add.
__device__ __forceinline__ float stencil_cell(const float* __restrict__ plane, const int lx, const int ly,
                                              const float (&q)[2 * kR + 1], const Coeffs& k)
{
#pragma clang fp contract(off)
  const float* c = plane + (ly + kR) * kPitch + (lx + kR);
  const float cr[5] = {0.0f, k.c1, k.c2, k.c3, k.c4};
  float acc = k.c0 * q[kR];
#pragma unroll
  for (int r = 1; r <= kR; ++r) {
    const float sx = c[-r] + c[r];
    const float sy = c[-r * kPitch] + c[r * kPitch];
    const float sz = q[kR - r] + q[kR + r];
    acc += cr[r] * ((sx + sy) + sz);
  }
  return acc;
}

struct TileWork {
  const float* in_origin;   // first interior cell of the tile in padded plane 0 of the z-chunk
  float* out_origin;        // first cell of the tile in output plane z0
  int planes;               // output planes in this chunk
};

__device__ __forceinline__ TileWork tile_work(const float* in, float* out, const int nx, const int ny, const int nz,
                                              const int zchunk)
{
  const int tiles_x = nx / kTX, tiles_y = ny / kTY;
  int b = blockIdx.x;
  const int tx = b % tiles_x; b /= tiles_x;
  const int ty = b % tiles_y; b /= tiles_y;
  const int z0 = b * zchunk;
  const size_t px = (size_t)nx + 2 * kR, py = (size_t)ny + 2 * kR;
  TileWork w;
  w.in_origin = in + ((size_t)z0 * py + (size_t)(ty * kTY + kR)) * px + (size_t)(tx * kTX + kR);
  w.out_origin = out + ((size_t)z0 * ny + (size_t)ty * kTY) * nx + (size_t)tx * kTX;
  w.planes = (nz - z0 < zchunk) ? (nz - z0) : zchunk;
  return w;
}

__global__ void __launch_bounds__(kComputeThreads + kDmaThreads)
stencil_warp_specialized(const float* __restrict__ in, float* __restrict__ out, const int nx, const int ny,
                         const int nz, const int zchunk, const Coeffs k)
{
  __shared__ __attribute__((aligned(16))) float plane[2][kPlaneFloats];
  const int px = nx + 2 * kR;
  const size_t in_plane = (size_t)px * (size_t)(ny + 2 * kR);
  const size_t out_plane = (size_t)nx * ny;
  halo_ws_t halo0(0, kComputeThreads, kComputeThreads, px);
  halo_ws_t halo1(1, kComputeThreads, kComputeThreads, px);
  hipdma::GroupBarrier compute_barrier(2, kComputeThreads);
  const TileWork w = tile_work(in, out, nx, ny, nz, zchunk);
  float* lds_origin0 = &plane[0][kR * kPitch + kR];
  float* lds_origin1 = &plane[1][kR * kPitch + kR];

  if (halo0.owns_this_thread()) {
    // centre plane of output plane z is padded plane z + kR
    const float* src = w.in_origin + (size_t)kR * in_plane;
    for (int z = 0; z < w.planes; z += 2) {
      halo0.template execute_dma<true, LOAD_CACHE_ALL, STORE_LDS>(src, lds_origin0);
      src += in_plane;
      if (z + 1 < w.planes) halo1.template execute_dma<true, LOAD_CACHE_ALL, STORE_LDS>(src, lds_origin1);
      src += in_plane;
    }
  } else {
    const int lx = threadIdx.x % kTX;
    const int ly = threadIdx.x / kTX;
    float q[kCells][2 * kR + 1];
    const float* col = w.in_origin + (size_t)ly * px + lx;
#pragma unroll
    for (int i = 0; i < kCells; ++i)
#pragma unroll
      for (int p = 0; p < 2 * kR; ++p) q[i][p + 1] = col[(size_t)p * in_plane + (size_t)(i * kRowsPerPass) * px];
    halo0.start_async_dma();
    halo1.start_async_dma();
    // interior of the first centre plane
#pragma unroll
    for (int i = 0; i < kCells; ++i) lds_origin0[(ly + i * kRowsPerPass) * kPitch + lx] = q[i][kR + 1];
    const float* next = col + (size_t)(2 * kR) * in_plane;
    float* o = w.out_origin + (size_t)ly * nx + lx;

    auto one_plane = [&](const float* cur_plane, float* other_origin, const halo_ws_t& cur_halo, const bool last) {
      // slide the queue and fetch the newest plane
#pragma unroll
      for (int i = 0; i < kCells; ++i) {
#pragma unroll
        for (int p = 0; p < 2 * kR; ++p) q[i][p] = q[i][p + 1];
        q[i][2 * kR] = next[(size_t)(i * kRowsPerPass) * px];
      }
      next += in_plane;
      cur_halo.wait_for_dma_finish();
      compute_barrier.sync();
      float r[kCells];
#pragma unroll
      for (int i = 0; i < kCells; ++i) r[i] = stencil_cell(cur_plane, lx, ly + i * kRowsPerPass, q[i], k);
      cur_halo.start_async_dma();
      if (!last) {
#pragma unroll
        for (int i = 0; i < kCells; ++i) other_origin[(ly + i * kRowsPerPass) * kPitch + lx] = q[i][kR + 1];
      }
#pragma unroll
      for (int i = 0; i < kCells; ++i) o[(size_t)(i * kRowsPerPass) * nx] = r[i];
      o += out_plane;
    };
    for (int z = 0; z < w.planes; z += 2) {
      one_plane(plane[0], lds_origin1, halo0, z + 1 >= w.planes);
      if (z + 1 < w.planes) one_plane(plane[1], lds_origin0, halo1, z + 2 >= w.planes);
    }
  }
}

__global__ void __launch_bounds__(kComputeThreads)
stencil_not_specialized(const float* __restrict__ in, float* __restrict__ out, const int nx, const int ny,
                        const int nz, const int zchunk, const Coeffs k)
{
  __shared__ __attribute__((aligned(16))) float plane[kPlaneFloats];
  const int px = nx + 2 * kR;
  const size_t in_plane = (size_t)px * (size_t)(ny + 2 * kR);
  const size_t out_plane = (size_t)nx * ny;
  halo_all_t halo(px);
  const TileWork w = tile_work(in, out, nx, ny, nz, zchunk);
  float* lds_origin = &plane[kR * kPitch + kR];
  const int lx = threadIdx.x % kTX;
  const int ly = threadIdx.x / kTX;
  float q[kCells][2 * kR + 1];
  const float* col = w.in_origin + (size_t)ly * px + lx;
#pragma unroll
  for (int i = 0; i < kCells; ++i)
#pragma unroll
    for (int p = 0; p < 2 * kR; ++p) q[i][p + 1] = col[(size_t)p * in_plane + (size_t)(i * kRowsPerPass) * px];
  const float* next = col + (size_t)(2 * kR) * in_plane;
  const float* ring_src = w.in_origin + (size_t)kR * in_plane;
  float* o = w.out_origin + (size_t)ly * nx + lx;
  for (int z = 0; z < w.planes; ++z) {
#pragma unroll
    for (int i = 0; i < kCells; ++i) {
#pragma unroll
      for (int p = 0; p < 2 * kR; ++p) q[i][p] = q[i][p + 1];
      q[i][2 * kR] = next[(size_t)(i * kRowsPerPass) * px];
    }
    next += in_plane;
    halo.template execute_dma<true, LOAD_CACHE_ALL, STORE_LDS>(ring_src, lds_origin);
    ring_src += in_plane;
#pragma unroll
    for (int i = 0; i < kCells; ++i) lds_origin[(ly + i * kRowsPerPass) * kPitch + lx] = q[i][kR];
    __syncthreads();
#pragma unroll
    for (int i = 0; i < kCells; ++i)
      o[(size_t)(i * kRowsPerPass) * nx] = stencil_cell(plane, lx, ly + i * kRowsPerPass, q[i], k);
    o += out_plane;
    __syncthreads();
  }
}

}  // namespace

extern "C" int cudadma_halo_stencil(const float* d_in, float* d_out, int nx, int ny, int nz, int variant, void* stream)
{
  CUDADMA_REQUIRE(nx > 0 && ny > 0 && nz > 0, "grid dimensions must be positive");
  CUDADMA_REQUIRE((nx % kTX) == 0 && (ny % kTY) == 0, "nx and ny must be multiples of 32");
  if (variant < 0 || variant >= cudadma_num_variants(CUDADMA_WORKLOAD_HALO)) {
    cudadma_host::set_error("halo stencil has no variant %d", variant);
    return CUDADMA_ERANGE;
  }
  CUDADMA_REQUIRE(d_in != nullptr && d_out != nullptr, "NULL pointer");
  CUDADMA_REQUIRE(cudadma_host::aligned_to(d_in, 16) && cudadma_host::aligned_to(d_out, 16), "pointers must be 16-byte aligned");
  const Coeffs k = {(float)(3.0 * (-205.0 / 72.0)), (float)(8.0 / 5.0), (float)(-1.0 / 5.0), (float)(8.0 / 315.0),
                    (float)(-1.0 / 560.0)};
  // z is cut into chunks so that a 512^3 grid yields a few thousand workgroups instead of 256
  int zchunk = 64;
  if (zchunk > nz) zchunk = nz;
  const int chunks = (nz + zchunk - 1) / zchunk;
  const long long grid = (long long)(nx / kTX) * (ny / kTY) * chunks;
  CUDADMA_REQUIRE(grid <= 0x7fffffffLL, "grid too large");
  hipStream_t s = (hipStream_t)stream;
  if (variant == 0)
    hipLaunchKernelGGL(stencil_warp_specialized, dim3((unsigned)grid), dim3(kComputeThreads + kDmaThreads), 0, s,
                       d_in, d_out, nx, ny, nz, zchunk, k);
  else
    hipLaunchKernelGGL(stencil_not_specialized, dim3((unsigned)grid), dim3(kComputeThreads), 0, s,
                       d_in, d_out, nx, ny, nz, zchunk, k);
  CUDADMA_HIP_CHECK(hipGetLastError());
  return CUDADMA_OK;
}
