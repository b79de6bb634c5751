// The five buffering styles of the reference's 2-D stencil example on the wave64
// objects: every z slice of a padded float2 volume is cut into TILE_X x TILE_Y
// tiles, the tile plus its halo is brought into LDS by CudaDMAStrided (one
// strided element per tile row) and TILE_X*TILE_Y compute threads each average
// a cross of neighbours.
//
// What the reference's example does: src/examples/stencil/
//   warp_specialized_single_buffer.h:26-87, warp_specialized_double_buffer.h:26-107,
//   warp_specialized_manual_buffer.h:26-114, non_warp_specialized_single_buffer.h:26-61,
//   non_warp_specialized_double_buffer.h:24-91, arithmetic stencil_math.h:27-87,
//   launch geometry cudaDMA_stencil2D.cu:99-204.
// Kernel arguments keep the reference's meaning: `offset` is the element index of
// interior point (0,0,0), `row_stride` and `slice_stride` are in elements, the grid
// is (DIM_X/TILE_X, DIM_Y/TILE_Y) workgroups and each marches `z_steps` slices.
// The buffered kernels with two buffers need an even z_steps, as the reference's do.
#pragma once

#include "../../../include/cudaDMAv2.h"

namespace examples {

// The cross average.  REACH neighbours are summed on each of the four arms and the
// sum is divided by 4*RADIUS+1.  The reference's loops stop one short of the radius
// (`d < RADIUS`, stencil_math.h:55-76) while dividing by 4*RADIUS+1 (:82-83); REACH
// = RADIUS-1 reproduces its numbers, REACH = RADIUS is the full cross.
template<int TILE_X, int TILE_Y, int RADIUS, int REACH>
__device__ __forceinline__ void perform_stencil(const float2* buffer, const unsigned tx, const unsigned ty,
                                                float2* dst_ptr)
{
  constexpr int kPitch = TILE_X + 2 * RADIUS;
  const float2* centre = buffer + (ty + RADIUS) * kPitch + (tx + RADIUS);
  float2 accum = centre[0];
#pragma unroll
  for (int d = 1; d <= REACH; ++d) { const float2 v = centre[-d]; accum.x += v.x; accum.y += v.y; }
#pragma unroll
  for (int d = 1; d <= REACH; ++d) { const float2 v = centre[d]; accum.x += v.x; accum.y += v.y; }
#pragma unroll
  for (int d = 1; d <= REACH; ++d) { const float2 v = centre[-d * kPitch]; accum.x += v.x; accum.y += v.y; }
#pragma unroll
  for (int d = 1; d <= REACH; ++d) { const float2 v = centre[d * kPitch]; accum.x += v.x; accum.y += v.y; }
  accum.x /= float(4 * RADIUS + 1);
  accum.y /= float(4 * RADIUS + 1);
  *dst_ptr = accum;
}

template<int TILE_X, int TILE_Y, int RADIUS>
struct StencilTile {
  static constexpr int kRows = TILE_Y + 2 * RADIUS;
  static constexpr int kRowBytes = (TILE_X + 2 * RADIUS) * int(sizeof(float2));
  static constexpr int kElmts = kRows * (TILE_X + 2 * RADIUS);
  static constexpr int kComputeThreads = TILE_X * TILE_Y;
};

#define HIPDMA_STENCIL2D_ARGS                                                                      \
  const float2* __restrict__ src_buffer, float2* __restrict__ dst_buffer, const int offset,        \
  const int row_stride, const int slice_stride, const int z_steps

// One buffer, one DMA group.  Launch TILE_X*TILE_Y + DMA_THREADS threads.
template<int ALIGNMENT, int BYTES_PER_THREAD, int TILE_X, int TILE_Y, int RADIUS, int REACH, int DMA_THREADS>
__global__ void stencil_2D_warp_specialized_single_buffer(HIPDMA_STENCIL2D_ARGS)
{
  typedef StencilTile<TILE_X, TILE_Y, RADIUS> tile;
  __shared__ __attribute__((aligned(16))) float2 buffer[tile::kElmts];

  CudaDMAStrided<true, ALIGNMENT, BYTES_PER_THREAD, tile::kRowBytes, DMA_THREADS, tile::kRows>
    dma_ld(0, tile::kComputeThreads, tile::kComputeThreads,
           row_stride * int(sizeof(float2)), tile::kRowBytes);

  const long long block_offset = offset + (long long)blockIdx.x * TILE_X + (long long)blockIdx.y * TILE_Y * row_stride;
  if (dma_ld.owns_this_thread()) {
    const float2* src_ptr = src_buffer + block_offset - (RADIUS * row_stride + RADIUS);
    for (int iz = 0; iz < z_steps; ++iz) {
      dma_ld.template execute_dma<true>(src_ptr, buffer);
      src_ptr += slice_stride;
    }
  } else {
    dma_ld.start_async_dma();
    const unsigned tx = threadIdx.x % TILE_X, ty = threadIdx.x / TILE_X;
    float2* dst_ptr = dst_buffer + block_offset + ty * row_stride + tx;
    for (int iz = 0; iz < z_steps; ++iz) {
      dma_ld.wait_for_dma_finish();
      perform_stencil<TILE_X, TILE_Y, RADIUS, REACH>(buffer, tx, ty, dst_ptr);
      if (iz + 1 < z_steps) dma_ld.start_async_dma();
      dst_ptr += slice_stride;
    }
  }
}

// Two buffers, two DMA groups on disjoint wavefronts.  Launch TILE_X*TILE_Y + 2*DMA_THREADS threads.
template<int ALIGNMENT, int BYTES_PER_THREAD, int TILE_X, int TILE_Y, int RADIUS, int REACH, int DMA_THREADS>
__global__ void stencil_2D_warp_specialized_double_buffer(HIPDMA_STENCIL2D_ARGS)
{
  typedef StencilTile<TILE_X, TILE_Y, RADIUS> tile;
  __shared__ __attribute__((aligned(16))) float2 buffer0[tile::kElmts];
  __shared__ __attribute__((aligned(16))) float2 buffer1[tile::kElmts];

  typedef CudaDMAStrided<true, ALIGNMENT, BYTES_PER_THREAD, tile::kRowBytes, DMA_THREADS, tile::kRows> dma_t;
  dma_t dma_ld0(0, tile::kComputeThreads, tile::kComputeThreads,
                row_stride * int(sizeof(float2)), tile::kRowBytes);
  dma_t dma_ld1(1, tile::kComputeThreads, tile::kComputeThreads + DMA_THREADS,
                row_stride * int(sizeof(float2)), tile::kRowBytes);

  const long long block_offset = offset + (long long)blockIdx.x * TILE_X + (long long)blockIdx.y * TILE_Y * row_stride;
  const float2* src_halo = src_buffer + block_offset - (RADIUS * row_stride + RADIUS);
  if (dma_ld0.owns_this_thread()) {
    const float2* src_ptr = src_halo;
    for (int iz = 0; iz < z_steps; iz += 2) {
      dma_ld0.template execute_dma<true>(src_ptr, buffer0);
      src_ptr += 2 * (long long)slice_stride;
    }
  } else if (dma_ld1.owns_this_thread()) {
    const float2* src_ptr = src_halo + slice_stride;
    for (int iz = 1; iz < z_steps; iz += 2) {
      dma_ld1.template execute_dma<true>(src_ptr, buffer1);
      src_ptr += 2 * (long long)slice_stride;
    }
  } else {
    dma_ld0.start_async_dma();
    dma_ld1.start_async_dma();
    const unsigned tx = threadIdx.x % TILE_X, ty = threadIdx.x / TILE_X;
    float2* dst_ptr = dst_buffer + block_offset + ty * row_stride + tx;
    for (int iz = 0; iz < z_steps; iz += 2) {
      dma_ld0.wait_for_dma_finish();
      perform_stencil<TILE_X, TILE_Y, RADIUS, REACH>(buffer0, tx, ty, dst_ptr);
      if (iz + 2 < z_steps) dma_ld0.start_async_dma();
      dst_ptr += slice_stride;
      dma_ld1.wait_for_dma_finish();
      perform_stencil<TILE_X, TILE_Y, RADIUS, REACH>(buffer1, tx, ty, dst_ptr);
      if (iz + 2 < z_steps) dma_ld1.start_async_dma();
      dst_ptr += slice_stride;
    }
  }
}

// Two buffers, two objects that share ONE DMA group; the group keeps the loads of
// both objects in flight through the two-phase calls.  Launch TILE_X*TILE_Y + DMA_THREADS threads.
template<int ALIGNMENT, int BYTES_PER_THREAD, int TILE_X, int TILE_Y, int RADIUS, int REACH, int DMA_THREADS>
__global__ void stencil_2D_warp_specialized_manual_buffer(HIPDMA_STENCIL2D_ARGS)
{
  typedef StencilTile<TILE_X, TILE_Y, RADIUS> tile;
  __shared__ __attribute__((aligned(16))) float2 buffer0[tile::kElmts];
  __shared__ __attribute__((aligned(16))) float2 buffer1[tile::kElmts];

  typedef CudaDMAStrided<true, ALIGNMENT, BYTES_PER_THREAD, tile::kRowBytes, DMA_THREADS, tile::kRows> dma_t;
  dma_t dma_ld0(0, tile::kComputeThreads, tile::kComputeThreads,
                row_stride * int(sizeof(float2)), tile::kRowBytes);
  dma_t dma_ld1(1, tile::kComputeThreads, tile::kComputeThreads,
                row_stride * int(sizeof(float2)), tile::kRowBytes);

  const long long block_offset = offset + (long long)blockIdx.x * TILE_X + (long long)blockIdx.y * TILE_Y * row_stride;
  if (dma_ld0.owns_this_thread()) {
    const float2* src_ptr = src_buffer + block_offset - (RADIUS * row_stride + RADIUS);
    dma_ld0.template start_xfer_async<true>(src_ptr);
    src_ptr += slice_stride;
    dma_ld1.template start_xfer_async<true>(src_ptr);
    src_ptr += slice_stride;
    for (int iz = 0; iz < z_steps - 2; iz += 2) {
      dma_ld0.template wait_xfer_finish<true>(buffer0);
      dma_ld0.template start_xfer_async<true>(src_ptr);
      src_ptr += slice_stride;
      dma_ld1.template wait_xfer_finish<true>(buffer1);
      dma_ld1.template start_xfer_async<true>(src_ptr);
      src_ptr += slice_stride;
    }
    dma_ld0.template wait_xfer_finish<true>(buffer0);
    dma_ld1.template wait_xfer_finish<true>(buffer1);
  } else {
    dma_ld0.start_async_dma();
    dma_ld1.start_async_dma();
    const unsigned tx = threadIdx.x % TILE_X, ty = threadIdx.x / TILE_X;
    float2* dst_ptr = dst_buffer + block_offset + ty * row_stride + tx;
    for (int iz = 0; iz < z_steps; iz += 2) {
      dma_ld0.wait_for_dma_finish();
      perform_stencil<TILE_X, TILE_Y, RADIUS, REACH>(buffer0, tx, ty, dst_ptr);
      if (iz + 2 < z_steps) dma_ld0.start_async_dma();
      dst_ptr += slice_stride;
      dma_ld1.wait_for_dma_finish();
      perform_stencil<TILE_X, TILE_Y, RADIUS, REACH>(buffer1, tx, ty, dst_ptr);
      if (iz + 2 < z_steps) dma_ld1.start_async_dma();
      dst_ptr += slice_stride;
    }
  }
}

// No specialisation: every thread transfers, then every thread computes; one buffer
// and two workgroup barriers per slice.  Launch TILE_X*TILE_Y threads.
template<int ALIGNMENT, int BYTES_PER_THREAD, int TILE_X, int TILE_Y, int RADIUS, int REACH>
__global__ void stencil_2D_non_warp_specialized_single_buffer(HIPDMA_STENCIL2D_ARGS)
{
  typedef StencilTile<TILE_X, TILE_Y, RADIUS> tile;
  __shared__ __attribute__((aligned(16))) float2 buffer[tile::kElmts];

  CudaDMAStrided<false, ALIGNMENT, BYTES_PER_THREAD, tile::kRowBytes, tile::kComputeThreads, tile::kRows>
    dma_ld(row_stride * int(sizeof(float2)), tile::kRowBytes);

  const long long block_offset = offset + (long long)blockIdx.x * TILE_X + (long long)blockIdx.y * TILE_Y * row_stride;
  const float2* src_ptr = src_buffer + block_offset - (RADIUS * row_stride + RADIUS);
  const unsigned tx = threadIdx.x % TILE_X, ty = threadIdx.x / TILE_X;
  float2* dst_ptr = dst_buffer + block_offset + ty * row_stride + tx;
  for (int iz = 0; iz < z_steps; ++iz) {
    dma_ld.template execute_dma<true>(src_ptr, buffer);
    src_ptr += slice_stride;
    __syncthreads();                       // buffer full
    perform_stencil<TILE_X, TILE_Y, RADIUS, REACH>(buffer, tx, ty, dst_ptr);
    dst_ptr += slice_stride;
    __syncthreads();                       // buffer free again
  }
}

// No specialisation, two buffers and two objects: the loads of the slice after next
// are in flight (held in registers by the two-phase calls) while a slice is consumed,
// one barrier per slice.  Launch TILE_X*TILE_Y threads.
template<int ALIGNMENT, int BYTES_PER_THREAD, int TILE_X, int TILE_Y, int RADIUS, int REACH>
__global__ void stencil_2D_non_warp_specialized_double_buffer(HIPDMA_STENCIL2D_ARGS)
{
  typedef StencilTile<TILE_X, TILE_Y, RADIUS> tile;
  __shared__ __attribute__((aligned(16))) float2 buffer0[tile::kElmts];
  __shared__ __attribute__((aligned(16))) float2 buffer1[tile::kElmts];

  typedef CudaDMAStrided<false, ALIGNMENT, BYTES_PER_THREAD, tile::kRowBytes, tile::kComputeThreads, tile::kRows> dma_t;
  dma_t dma_ld0(row_stride * int(sizeof(float2)), tile::kRowBytes);
  dma_t dma_ld1(row_stride * int(sizeof(float2)), tile::kRowBytes);

  const long long block_offset = offset + (long long)blockIdx.x * TILE_X + (long long)blockIdx.y * TILE_Y * row_stride;
  const float2* src_ptr = src_buffer + block_offset - (RADIUS * row_stride + RADIUS);
  const unsigned tx = threadIdx.x % TILE_X, ty = threadIdx.x / TILE_X;
  float2* dst_ptr = dst_buffer + block_offset + ty * row_stride + tx;

  dma_ld0.template start_xfer_async<true>(src_ptr);
  src_ptr += slice_stride;
  dma_ld1.template start_xfer_async<true>(src_ptr);
  src_ptr += slice_stride;
  for (int iz = 0; iz < z_steps - 2; iz += 2) {
    dma_ld0.template wait_xfer_finish<true>(buffer0);
    dma_ld0.template start_xfer_async<true>(src_ptr);
    src_ptr += slice_stride;
    __syncthreads();
    perform_stencil<TILE_X, TILE_Y, RADIUS, REACH>(buffer0, tx, ty, dst_ptr);
    dst_ptr += slice_stride;

    dma_ld1.template wait_xfer_finish<true>(buffer1);
    dma_ld1.template start_xfer_async<true>(src_ptr);
    src_ptr += slice_stride;
    __syncthreads();
    perform_stencil<TILE_X, TILE_Y, RADIUS, REACH>(buffer1, tx, ty, dst_ptr);
    dst_ptr += slice_stride;
  }
  dma_ld0.template wait_xfer_finish<true>(buffer0);
  __syncthreads();
  perform_stencil<TILE_X, TILE_Y, RADIUS, REACH>(buffer0, tx, ty, dst_ptr);
  dst_ptr += slice_stride;
  dma_ld1.template wait_xfer_finish<true>(buffer1);
  __syncthreads();
  perform_stencil<TILE_X, TILE_Y, RADIUS, REACH>(buffer1, tx, ty, dst_ptr);
}

#undef HIPDMA_STENCIL2D_ARGS

}  // namespace examples
