// sgemv ("n" form: y = alpha * A x, A column-major) with the vector, or the
// vector and the matrix panel, staged through LDS by DMA wavefronts.
//
// What the reference's example computes: src/examples/sgemv/sgemv_dma.cu
// (vector staged, one buffer :140-175; vector staged, two objects on the same
// DMA threads :262-325; vector and matrix staged :329-388 and :392-470).  Thread
// `row` owns one row: res = fma(A[row + j*lda], x[j], res) for ascending j from
// 0.0f, y[row] = alpha * res.  Written against the first-generation class names
// (cudaDMASequential, cudaDMAStrided of include/cudaDMA.h).
//
// All kernels need m to be a multiple of the columns staged per hand-off and
// lda*4 to be a multiple of 16 B when the matrix is staged; rows beyond n are
// neither read from global memory by compute threads nor written.
#pragma once

#include "../../../include/cudaDMA.h"

namespace examples {

// Vector staged in one buffer; the matrix is read straight from global memory.
// Launch with COMPUTE_THREADS + DMA_THREADS_PER_LD threads.
template<int COMPUTE_THREADS, int DMA_THREADS_PER_LD, int VEC_ELMTS>
__global__ void sgemvn_vec_single(int n, int m, float alpha, const float* __restrict__ A, int lda,
                                  const float* __restrict__ x, float* __restrict__ y)
{
  __shared__ __attribute__((aligned(16))) float buff[VEC_ELMTS];
  cudaDMASequential<true, 16, 4 * VEC_ELMTS, DMA_THREADS_PER_LD>
    dma_ld_0(1, COMPUTE_THREADS, COMPUTE_THREADS);

  if (threadIdx.x < COMPUTE_THREADS) {
    dma_ld_0.start_async_dma();
    const int row = blockIdx.x * COMPUTE_THREADS + threadIdx.x;
    const bool live = row < n;
    const float* a_col = A + (live ? row : 0);
    float res = 0.0f;
    for (int i = 0; i < m; i += VEC_ELMTS) {
      dma_ld_0.wait_for_dma_finish();
#pragma unroll 8
      for (int j = 0; j < VEC_ELMTS; ++j) {
        res = __builtin_fmaf(*a_col, buff[j], res);
        a_col += lda;
      }
      if (i + VEC_ELMTS < m) dma_ld_0.start_async_dma();
    }
    if (live) y[row] = alpha * res;
  } else if (dma_ld_0.owns_this_thread()) {
    for (int i = 0; i < m; i += VEC_ELMTS)
      dma_ld_0.execute_dma(x + i, buff);
  }
}

// Vector staged through two buffers by two objects that share the same DMA
// threads ("manual" double buffering).  Launch with COMPUTE_THREADS + DMA_THREADS_PER_LD threads.
template<int COMPUTE_THREADS, int DMA_THREADS_PER_LD, int VEC_ELMTS>
__global__ void sgemvn_vec_manual(int n, int m, float alpha, const float* __restrict__ A, int lda,
                                  const float* __restrict__ x, float* __restrict__ y)
{
  __shared__ __attribute__((aligned(16))) float buff0[VEC_ELMTS];
  __shared__ __attribute__((aligned(16))) float buff1[VEC_ELMTS];
  typedef cudaDMASequential<true, 16, 4 * VEC_ELMTS, DMA_THREADS_PER_LD> dma_t;
  dma_t dma_ld_0(1, COMPUTE_THREADS, COMPUTE_THREADS);
  dma_t dma_ld_1(2, COMPUTE_THREADS, COMPUTE_THREADS);

  if (threadIdx.x < COMPUTE_THREADS) {
    dma_ld_0.start_async_dma();
    dma_ld_1.start_async_dma();
    const int row = blockIdx.x * COMPUTE_THREADS + threadIdx.x;
    const bool live = row < n;
    const float* a_col = A + (live ? row : 0);
    float res = 0.0f;
    for (int i = 0; i < m; i += 2 * VEC_ELMTS) {
      dma_ld_0.wait_for_dma_finish();
#pragma unroll 8
      for (int j = 0; j < VEC_ELMTS; ++j) {
        res = __builtin_fmaf(*a_col, buff0[j], res);
        a_col += lda;
      }
      if (i + 2 * VEC_ELMTS < m) dma_ld_0.start_async_dma();
      dma_ld_1.wait_for_dma_finish();
#pragma unroll 8
      for (int j = 0; j < VEC_ELMTS; ++j) {
        res = __builtin_fmaf(*a_col, buff1[j], res);
        a_col += lda;
      }
      if (i + 2 * VEC_ELMTS < m) dma_ld_1.start_async_dma();
    }
    if (live) y[row] = alpha * res;
  } else if (dma_ld_0.owns_this_thread()) {
    for (int i = 0; i < m; i += 2 * VEC_ELMTS) {
      dma_ld_0.execute_dma(x + i, buff0);
      dma_ld_1.execute_dma(x + i + VEC_ELMTS, buff1);
    }
  }
}

// Vector and a VEC_ELMTS-column panel of the matrix staged, one buffer each.
// The panel is VEC_ELMTS strided elements (columns) of COMPUTE_THREADS floats,
// packed in LDS by the one-stride constructor of the older interface.
// Launch with COMPUTE_THREADS + (1 + MAT_LDS) * DMA_THREADS_PER_LD threads.
template<int COMPUTE_THREADS, int DMA_THREADS_PER_LD, int VEC_ELMTS, int MAT_LDS>
__global__ void sgemvn_both_single(int n, int m, float alpha, const float* __restrict__ A, int lda,
                                   const float* __restrict__ x, float* __restrict__ y)
{
  __shared__ __attribute__((aligned(16))) float buff[VEC_ELMTS];
  __shared__ __attribute__((aligned(16))) float mat[VEC_ELMTS][COMPUTE_THREADS];

  cudaDMASequential<true, 16, 4 * VEC_ELMTS, DMA_THREADS_PER_LD>
    dma_ld_0(1, COMPUTE_THREADS, COMPUTE_THREADS);
  cudaDMAStrided<true, 16, 4 * COMPUTE_THREADS, MAT_LDS * DMA_THREADS_PER_LD, VEC_ELMTS>
    dma_ld_1(2, COMPUTE_THREADS, COMPUTE_THREADS + DMA_THREADS_PER_LD, 4 * lda);

  if (threadIdx.x < COMPUTE_THREADS) {
    dma_ld_0.start_async_dma();
    dma_ld_1.start_async_dma();
    float res = 0.0f;
    for (int i = 0; i < m; i += VEC_ELMTS) {
      dma_ld_0.wait_for_dma_finish();
      dma_ld_1.wait_for_dma_finish();
#pragma unroll
      for (int j = 0; j < VEC_ELMTS; ++j)
        res = __builtin_fmaf(mat[j][threadIdx.x], buff[j], res);
      if (i + VEC_ELMTS < m) {
        dma_ld_0.start_async_dma();
        dma_ld_1.start_async_dma();
      }
    }
    const int row = blockIdx.x * COMPUTE_THREADS + threadIdx.x;
    if (row < n) y[row] = alpha * res;
  } else if (dma_ld_0.owns_this_thread()) {
    for (int i = 0; i < m; i += VEC_ELMTS)
      dma_ld_0.execute_dma(x + i, buff);
  } else if (dma_ld_1.owns_this_thread()) {
    const float* panel = A + (long long)blockIdx.x * COMPUTE_THREADS;
    for (int i = 0; i < m; i += VEC_ELMTS) {
      dma_ld_1.execute_dma(panel, mat);
      panel += (long long)lda * VEC_ELMTS;
    }
  }
}

// Vector and matrix panel staged through two buffers each, four objects on
// disjoint DMA wavefronts.
// Launch with COMPUTE_THREADS + 2 * (1 + MAT_LDS) * DMA_THREADS_PER_LD threads.
template<int COMPUTE_THREADS, int DMA_THREADS_PER_LD, int VEC_ELMTS, int MAT_LDS>
__global__ void sgemvn_both_double(int n, int m, float alpha, const float* __restrict__ A, int lda,
                                   const float* __restrict__ x, float* __restrict__ y)
{
  __shared__ __attribute__((aligned(16))) float buff0[VEC_ELMTS];
  __shared__ __attribute__((aligned(16))) float buff1[VEC_ELMTS];
  __shared__ __attribute__((aligned(16))) float mat0[VEC_ELMTS][COMPUTE_THREADS];
  __shared__ __attribute__((aligned(16))) float mat1[VEC_ELMTS][COMPUTE_THREADS];

  typedef cudaDMASequential<true, 16, 4 * VEC_ELMTS, DMA_THREADS_PER_LD> vec_dma_t;
  typedef cudaDMAStrided<true, 16, 4 * COMPUTE_THREADS, MAT_LDS * DMA_THREADS_PER_LD, VEC_ELMTS> mat_dma_t;
  constexpr int kMatThreads = MAT_LDS * DMA_THREADS_PER_LD;
  vec_dma_t dma_vec_0(1, COMPUTE_THREADS, COMPUTE_THREADS);
  vec_dma_t dma_vec_1(2, COMPUTE_THREADS, COMPUTE_THREADS + DMA_THREADS_PER_LD);
  mat_dma_t dma_mat_0(3, COMPUTE_THREADS, COMPUTE_THREADS + 2 * DMA_THREADS_PER_LD, 4 * lda);
  mat_dma_t dma_mat_1(4, COMPUTE_THREADS, COMPUTE_THREADS + 2 * DMA_THREADS_PER_LD + kMatThreads, 4 * lda);

  if (threadIdx.x < COMPUTE_THREADS) {
    dma_vec_0.start_async_dma();
    dma_mat_0.start_async_dma();
    if (VEC_ELMTS < m) { dma_vec_1.start_async_dma(); dma_mat_1.start_async_dma(); }
    float res = 0.0f;
    for (int i = 0; i < m; i += 2 * VEC_ELMTS) {
      dma_vec_0.wait_for_dma_finish();
      dma_mat_0.wait_for_dma_finish();
#pragma unroll
      for (int j = 0; j < VEC_ELMTS; ++j)
        res = __builtin_fmaf(mat0[j][threadIdx.x], buff0[j], res);
      if (i + 2 * VEC_ELMTS < m) { dma_vec_0.start_async_dma(); dma_mat_0.start_async_dma(); }
      if (i + VEC_ELMTS < m) {
        dma_vec_1.wait_for_dma_finish();
        dma_mat_1.wait_for_dma_finish();
#pragma unroll
        for (int j = 0; j < VEC_ELMTS; ++j)
          res = __builtin_fmaf(mat1[j][threadIdx.x], buff1[j], res);
        if (i + 3 * VEC_ELMTS < m) { dma_vec_1.start_async_dma(); dma_mat_1.start_async_dma(); }
      }
    }
    const int row = blockIdx.x * COMPUTE_THREADS + threadIdx.x;
    if (row < n) y[row] = alpha * res;
  } else if (dma_vec_0.owns_this_thread()) {
    for (int i = 0; i < m; i += 2 * VEC_ELMTS) dma_vec_0.execute_dma(x + i, buff0);
  } else if (dma_vec_1.owns_this_thread()) {
    for (int i = VEC_ELMTS; i < m; i += 2 * VEC_ELMTS) dma_vec_1.execute_dma(x + i, buff1);
  } else if (dma_mat_0.owns_this_thread()) {
    const float* panel = A + (long long)blockIdx.x * COMPUTE_THREADS;
    for (int i = 0; i < m; i += 2 * VEC_ELMTS)
      dma_mat_0.execute_dma(panel + (long long)lda * i, mat0);
  } else if (dma_mat_1.owns_this_thread()) {
    const float* panel = A + (long long)blockIdx.x * COMPUTE_THREADS;
    for (int i = VEC_ELMTS; i < m; i += 2 * VEC_ELMTS)
      dma_mat_1.execute_dma(panel + (long long)lda * i, mat1);
  }
}

}  // namespace examples
