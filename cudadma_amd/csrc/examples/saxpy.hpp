// saxpy staged through LDS by DMA wavefronts, written against the
// first-generation class names (cudaDMASequential of include/cudaDMA.h) to show
// that a kernel of that style builds on the wave64 objects.
//
// What the reference's example computes: src/examples/saxpy/saxpy_cudaDMA_kernel.cu
// (baseline :55-61, single-buffered DMA :270-315, double-buffered DMA :322-418):
// y[i] = a * x[i] + y[i], contracted to one fused multiply-add by the device
// compiler.  The kernels here move 16 B per compute thread per chunk instead of
// 4 B, and walk the chunks of the vector with a grid stride so any vector whose
// length is a multiple of the chunk works with any number of workgroups.
#pragma once

#include "../../../include/cudaDMA.h"

namespace examples {

// One element per thread, grid stride: the yardstick without LDS.
__global__ void saxpy_baseline(float* __restrict__ y, const float* __restrict__ x, float a, long long n)
{
  const long long stride = (long long)gridDim.x * blockDim.x;
  for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride)
    y[i] = __builtin_fmaf(a, x[i], y[i]);
}

// Four elements per thread (dwordx4 accesses), grid stride.
__global__ void saxpy_vec4(float* __restrict__ y, const float* __restrict__ x, float a, long long n)
{
  const long long stride = (long long)gridDim.x * blockDim.x;
  const float4* x4 = reinterpret_cast<const float4*>(x);
  float4* y4 = reinterpret_cast<float4*>(y);
  for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < n / 4; i += stride) {
    const float4 xv = x4[i];
    float4 yv = y4[i];
    yv.x = __builtin_fmaf(a, xv.x, yv.x);
    yv.y = __builtin_fmaf(a, xv.y, yv.y);
    yv.z = __builtin_fmaf(a, xv.z, yv.z);
    yv.w = __builtin_fmaf(a, xv.w, yv.w);
    y4[i] = yv;
  }
}

template<int COMPUTE_THREADS>
struct SaxpyChunk {
  static constexpr int kFloats = 4 * COMPUTE_THREADS;     // one float4 per compute thread
  static constexpr int kBytes = 4 * kFloats;
};

__device__ __forceinline__ void saxpy_store(float a, const float4& xv, float4 yv, float* y_chunk, int tid)
{
  yv.x = __builtin_fmaf(a, xv.x, yv.x);
  yv.y = __builtin_fmaf(a, xv.y, yv.y);
  yv.z = __builtin_fmaf(a, xv.z, yv.z);
  yv.w = __builtin_fmaf(a, xv.w, yv.w);
  reinterpret_cast<float4*>(y_chunk)[tid] = yv;
}

// One buffer per vector: a DMA group for x and one for y, the compute threads
// copy their operands to registers, hand the buffers back and only then do the
// arithmetic and the store (saxpy_cudaDMA_kernel.cu:270-315).
// Launch with COMPUTE_THREADS + 2*DMA_THREADS_PER_LD threads.
template<int COMPUTE_THREADS, int DMA_THREADS_PER_LD>
__global__ void saxpy_dma_single(float* __restrict__ y, const float* __restrict__ x, float a, long long num_chunks)
{
  typedef SaxpyChunk<COMPUTE_THREADS> chunk;
  __shared__ __attribute__((aligned(16))) float sx[chunk::kFloats];
  __shared__ __attribute__((aligned(16))) float sy[chunk::kFloats];

  cudaDMASequential<true, 16, chunk::kBytes, DMA_THREADS_PER_LD>
    dma_ld_x(1, COMPUTE_THREADS, COMPUTE_THREADS);
  cudaDMASequential<true, 16, chunk::kBytes, DMA_THREADS_PER_LD>
    dma_ld_y(2, COMPUTE_THREADS, COMPUTE_THREADS + DMA_THREADS_PER_LD);

  const long long first = blockIdx.x, step = gridDim.x;
  const int tid = threadIdx.x;
  if (tid < COMPUTE_THREADS) {
    if (first >= num_chunks) return;
    dma_ld_x.start_async_dma();
    dma_ld_y.start_async_dma();
    for (long long c = first; c < num_chunks; c += step) {
      const bool more = c + step < num_chunks;
      float4 xv, yv;
      dma_ld_x.wait_for_dma_finish();
      xv = reinterpret_cast<const float4*>(sx)[tid];
      if (more) dma_ld_x.start_async_dma();
      dma_ld_y.wait_for_dma_finish();
      yv = reinterpret_cast<const float4*>(sy)[tid];
      if (more) dma_ld_y.start_async_dma();
      saxpy_store(a, xv, yv, y + c * chunk::kFloats, tid);
    }
  } else if (dma_ld_x.owns_this_thread()) {
    for (long long c = first; c < num_chunks; c += step)
      dma_ld_x.execute_dma(x + c * chunk::kFloats, sx);
  } else if (dma_ld_y.owns_this_thread()) {
    for (long long c = first; c < num_chunks; c += step)
      dma_ld_y.execute_dma(y + c * chunk::kFloats, sy);
  }
}

// Two buffers per vector, four DMA groups on disjoint wavefronts
// (saxpy_cudaDMA_kernel.cu:322-418); chunk k of a workgroup goes through buffer k & 1.
// Launch with COMPUTE_THREADS + 4*DMA_THREADS_PER_LD threads.
template<int COMPUTE_THREADS, int DMA_THREADS_PER_LD>
__global__ void saxpy_dma_double(float* __restrict__ y, const float* __restrict__ x, float a, long long num_chunks)
{
  typedef SaxpyChunk<COMPUTE_THREADS> chunk;
  __shared__ __attribute__((aligned(16))) float sx0[chunk::kFloats];
  __shared__ __attribute__((aligned(16))) float sx1[chunk::kFloats];
  __shared__ __attribute__((aligned(16))) float sy0[chunk::kFloats];
  __shared__ __attribute__((aligned(16))) float sy1[chunk::kFloats];

  typedef cudaDMASequential<true, 16, chunk::kBytes, DMA_THREADS_PER_LD> dma_t;
  dma_t dma_ld_x_0(1, COMPUTE_THREADS, COMPUTE_THREADS);
  dma_t dma_ld_y_0(2, COMPUTE_THREADS, COMPUTE_THREADS + DMA_THREADS_PER_LD);
  dma_t dma_ld_x_1(3, COMPUTE_THREADS, COMPUTE_THREADS + 2 * DMA_THREADS_PER_LD);
  dma_t dma_ld_y_1(4, COMPUTE_THREADS, COMPUTE_THREADS + 3 * DMA_THREADS_PER_LD);

  const long long first = blockIdx.x, step = gridDim.x;
  const int tid = threadIdx.x;
  if (tid < COMPUTE_THREADS) {
    if (first < num_chunks) { dma_ld_x_0.start_async_dma(); dma_ld_y_0.start_async_dma(); }
    if (first + step < num_chunks) { dma_ld_x_1.start_async_dma(); dma_ld_y_1.start_async_dma(); }
    for (long long c = first; c < num_chunks; c += 2 * step) {
      float4 xv, yv;
      {
        const bool more = c + 2 * step < num_chunks;
        dma_ld_x_0.wait_for_dma_finish();
        xv = reinterpret_cast<const float4*>(sx0)[tid];
        if (more) dma_ld_x_0.start_async_dma();
        dma_ld_y_0.wait_for_dma_finish();
        yv = reinterpret_cast<const float4*>(sy0)[tid];
        if (more) dma_ld_y_0.start_async_dma();
        saxpy_store(a, xv, yv, y + c * chunk::kFloats, tid);
      }
      if (c + step < num_chunks) {
        const bool more = c + 3 * step < num_chunks;
        dma_ld_x_1.wait_for_dma_finish();
        xv = reinterpret_cast<const float4*>(sx1)[tid];
        if (more) dma_ld_x_1.start_async_dma();
        dma_ld_y_1.wait_for_dma_finish();
        yv = reinterpret_cast<const float4*>(sy1)[tid];
        if (more) dma_ld_y_1.start_async_dma();
        saxpy_store(a, xv, yv, y + (c + step) * chunk::kFloats, tid);
      }
    }
  } else if (dma_ld_x_0.owns_this_thread()) {
    for (long long c = first; c < num_chunks; c += 2 * step)
      dma_ld_x_0.execute_dma(x + c * chunk::kFloats, sx0);
  } else if (dma_ld_y_0.owns_this_thread()) {
    for (long long c = first; c < num_chunks; c += 2 * step)
      dma_ld_y_0.execute_dma(y + c * chunk::kFloats, sy0);
  } else if (dma_ld_x_1.owns_this_thread()) {
    for (long long c = first + step; c < num_chunks; c += 2 * step)
      dma_ld_x_1.execute_dma(x + c * chunk::kFloats, sx1);
  } else if (dma_ld_y_1.owns_this_thread()) {
    for (long long c = first + step; c < num_chunks; c += 2 * step)
      dma_ld_y_1.execute_dma(y + c * chunk::kFloats, sy1);
  }
}

}  // namespace examples
