// Config 2: out = in^T for an n x n float matrix.  CudaDMAStrided pulls tiles of
// 64 rows x 256 B (source stride n*4 bytes) into LDS; the compute wavefronts
// write each tile transposed.  The nearest reference analogue is the
// matrix-tile load of src/examples/sgemv/sgemv_dma.cu:329-388.
//
// LDS layout: rows are padded to 272 B (17 chunks of 16 B).  A compute lane owns
// one tile row and reads it with ds_read_b128; lane L reads 16-byte unit
// 17*L + j, so eight consecutive lanes hit eight different units modulo 8 and no
// banks collide.  The tile column c then leaves as one global_store_dword per
// wavefront: 64 lanes x 4 B = 256 contiguous bytes of output row c.
#include "workloads.hpp"

namespace {
using workloads::vec4_t;

constexpr int kTile = 64;                       // rows and columns of a tile
constexpr int kRowBytes = kTile * 4;            // 256
constexpr int kDmaThreads = 128;
constexpr int kComputeThreads = 128;
constexpr int kBytesPerThread = kTile * kRowBytes / kDmaThreads;   // 128: the whole tile in one step

// Tile order: the matrix is cut into bands of `band` tile rows; inside a band
// the tile row index runs fastest, then the tile column.  The workgroups
// resident at one time therefore read runs of (resident / band) * 256 B of the
// source rows and write runs of band * 256 B of the output rows.
constexpr int kDefaultBand = 16;

__device__ __forceinline__ void tile_coords(const int t, const int tiles_per_side, const int band_rows, int& ty, int& tx)
{
  const int band = t / (band_rows * tiles_per_side);
  const int in_band = t - band * (band_rows * tiles_per_side);
  tx = in_band / band_rows;
  ty = band * band_rows + (in_band - tx * band_rows);
}

template<int LDS_ROW_BYTES, typename Dma>
__device__ __forceinline__ void write_tile_transposed(const char* lds_tile, float* __restrict__ out, const int n,
                                                      const int ty, const int tx, const Dma& dma)
{
  // compute thread: lane = tile row, wavefront w handles tile columns [32w, 32w+32)
  const int lane = threadIdx.x & 63;
  const int w = threadIdx.x >> 6;
  vec4_t v[8];
  const vec4_t* row = (const vec4_t*)(lds_tile + lane * LDS_ROW_BYTES) + w * 8;
#pragma unroll
  for (int j = 0; j < 8; ++j) v[j] = row[j];
  dma.start_async_dma();
  // element (r = lane, c) of the tile goes to out[(tx*64 + c) * n + ty*64 + r]
  float* o = out + (size_t)(tx * kTile + w * 32) * n + (size_t)ty * kTile + lane;
#pragma unroll
  for (int j = 0; j < 8; ++j) {
#pragma unroll
    for (int k = 0; k < 4; ++k)
      o[(size_t)(4 * j + k) * n] = __uint_as_float(v[j][k]);
  }
}

template<int LDS_ROW_BYTES>
__global__ void __launch_bounds__(kDmaThreads + kComputeThreads)
transpose_manual_double(const float* __restrict__ in, float* __restrict__ out, const int n, const int num_tiles,
                        const int band)
{
  __shared__ __attribute__((aligned(16))) char buf0[kTile * LDS_ROW_BYTES];
  __shared__ __attribute__((aligned(16))) char buf1[kTile * LDS_ROW_BYTES];
  typedef CudaDMAStrided<true, 16, kBytesPerThread, kRowBytes, kDmaThreads, kTile> dma_t;
  dma_t dma0(0, kComputeThreads, kComputeThreads, n * 4, LDS_ROW_BYTES);
  dma_t dma1(1, kComputeThreads, kComputeThreads, n * 4, LDS_ROW_BYTES);
  const int tiles_per_side = n / kTile;
  const int stride = gridDim.x;
  auto src_of = [&](const int t) {
    int ty, tx;
    tile_coords(t, tiles_per_side, band, ty, tx);
    return (const void*)(in + (size_t)ty * kTile * n + (size_t)tx * kTile);
  };
  if (dma0.owns_this_thread()) {
    int t = blockIdx.x;
    if (t < num_tiles) dma0.template start_xfer_async<true, LOAD_CACHE_ALL, STORE_LDS>(src_of(t));
    if (t + stride < num_tiles) dma1.template start_xfer_async<true, LOAD_CACHE_ALL, STORE_LDS>(src_of(t + stride));
    for (; t < num_tiles; t += 2 * stride) {
      dma0.template wait_xfer_finish<true, LOAD_CACHE_ALL, STORE_LDS>(buf0);
      if (t + 2 * stride < num_tiles) dma0.template start_xfer_async<true, LOAD_CACHE_ALL, STORE_LDS>(src_of(t + 2 * stride));
      if (t + stride < num_tiles) {
        dma1.template wait_xfer_finish<true, LOAD_CACHE_ALL, STORE_LDS>(buf1);
        if (t + 3 * stride < num_tiles) dma1.template start_xfer_async<true, LOAD_CACHE_ALL, STORE_LDS>(src_of(t + 3 * stride));
      }
    }
  } else {
    dma0.start_async_dma();
    dma1.start_async_dma();
    for (int t = blockIdx.x; t < num_tiles; t += 2 * stride) {
      int ty, tx;
      tile_coords(t, tiles_per_side, band, ty, tx);
      dma0.wait_for_dma_finish();
      write_tile_transposed<LDS_ROW_BYTES>(buf0, out, n, ty, tx, dma0);
      if (t + stride < num_tiles) {
        tile_coords(t + stride, tiles_per_side, band, ty, tx);
        dma1.wait_for_dma_finish();
        write_tile_transposed<LDS_ROW_BYTES>(buf1, out, n, ty, tx, dma1);
      }
    }
  }
}

__global__ void __launch_bounds__(kDmaThreads + kComputeThreads)
transpose_single(const float* __restrict__ in, float* __restrict__ out, const int n, const int num_tiles, const int band)
{
  constexpr int kLdsRow = 272;
  __shared__ __attribute__((aligned(16))) char buf[kTile * kLdsRow];
  CudaDMAStrided<true, 16, kBytesPerThread, kRowBytes, kDmaThreads, kTile>
      dma(0, kComputeThreads, kComputeThreads, n * 4, kLdsRow);
  const int tiles_per_side = n / kTile;
  if (dma.owns_this_thread()) {
    for (int t = blockIdx.x; t < num_tiles; t += gridDim.x) {
      int ty, tx;
      tile_coords(t, tiles_per_side, band, ty, tx);
      dma.template execute_dma<true, LOAD_CACHE_ALL, STORE_LDS>(in + (size_t)ty * kTile * n + (size_t)tx * kTile, buf);
    }
  } else {
    dma.start_async_dma();
    for (int t = blockIdx.x; t < num_tiles; t += gridDim.x) {
      int ty, tx;
      tile_coords(t, tiles_per_side, band, ty, tx);
      dma.wait_for_dma_finish();
      write_tile_transposed<kLdsRow>(buf, out, n, ty, tx, dma);
    }
  }
}

}  // namespace

extern "C" int cudadma_strided_transpose(const float* d_in, float* d_out, int n, int variant, void* stream)
{
  CUDADMA_REQUIRE(n >= 0 && (n % kTile) == 0, "n (%d) must be a multiple of %d", n, kTile);
  int band = workloads::tuning("transpose_band", kDefaultBand);
  while (band > 1 && (n / kTile) % band != 0) band /= 2;      // bands must tile the matrix
  CUDADMA_REQUIRE((long long)n * 4 <= 0x7fffffffLL, "row pitch must fit an int");
  if (variant < 0 || variant >= cudadma_num_variants(CUDADMA_WORKLOAD_STRIDED)) {
    cudadma_host::set_error("strided transpose has no variant %d", variant);
    return CUDADMA_ERANGE;
  }
  if (n == 0) return CUDADMA_OK;
  CUDADMA_REQUIRE(d_in != nullptr && d_out != nullptr && d_in != d_out, "NULL or aliased pointers");
  CUDADMA_REQUIRE(cudadma_host::aligned_to(d_in, 16) && cudadma_host::aligned_to(d_out, 16), "pointers must be 16-byte aligned");
  const int tiles = (n / kTile) * (n / kTile);
  hipStream_t s = (hipStream_t)stream;
  const dim3 block(kDmaThreads + kComputeThreads);
  switch (variant) {
    case 0: hipLaunchKernelGGL(transpose_manual_double<272>, dim3(workloads::persistent_grid(tiles, 4)), block, 0, s, d_in, d_out, n, tiles, band); break;
    case 1: hipLaunchKernelGGL(transpose_single, dim3(workloads::persistent_grid(tiles, 8)), block, 0, s, d_in, d_out, n, tiles, band); break;
    default: hipLaunchKernelGGL(transpose_manual_double<256>, dim3(workloads::persistent_grid(tiles, 4)), block, 0, s, d_in, d_out, n, tiles, band); break;
  }
  CUDADMA_HIP_CHECK(hipGetLastError());
  return CUDADMA_OK;
}
