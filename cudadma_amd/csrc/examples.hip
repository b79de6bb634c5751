// C-ABI launchers of the example consumers (saxpy, sgemv, 2-D stencil) that the
// reference ships under src/examples/; the kernels themselves live in
// examples/*.hpp and are written against the DMA classes only.
#include "common.hpp"
#include "workloads.hpp"
#include "examples/saxpy.hpp"
#include "examples/sgemv.hpp"
#include "examples/stencil2d.hpp"

namespace {

using namespace examples;

// ---- saxpy ----
constexpr int kSaxpyCompute = 256;          // four compute wavefronts
constexpr int kSaxpyDmaPerLd = 64;          // one wavefront per staged vector and buffer
const char* const kSaxpyNames[] = {
  "baseline: one element per thread, no LDS",
  "vec4: dwordx4 per thread, no LDS",
  "cudaDMASequential x2, one buffer per vector",
  "cudaDMASequential x4, two buffers per vector",
};

// ---- sgemv ----
constexpr int kGemvCompute = 128;
constexpr int kGemvDmaPerLd = 64;
constexpr int kGemvVecElmts = 256;          // columns per hand-off when only the vector is staged
constexpr int kGemvPanelCols = 32;          // columns per hand-off when the matrix panel is staged too
constexpr int kGemvMatLds = 2;              // DMA wavefronts on the matrix panel
const char* const kGemvNames[] = {
  "vector staged by cudaDMASequential, one buffer",
  "vector staged by two cudaDMASequential on shared DMA threads",
  "vector by cudaDMASequential + 32-column panel by cudaDMAStrided, one buffer each",
  "vector by cudaDMASequential + 32-column panel by cudaDMAStrided, two buffers each",
};

// ---- 2-D stencil ----
constexpr int kTileX = 32, kTileY = 4, kRadius = 4;
constexpr int kStencilDma = 64, kStencilBpt = 64, kStencilAlign = 16;
const char* const kStencilNames[] = {
  "warp specialized, single buffer",
  "warp specialized, double buffer",
  "warp specialized, manual buffer",
  "non warp specialized, single buffer",
  "non warp specialized, double buffer",
};

template<int REACH>
void launch_stencil(int variant, dim3 grid, hipStream_t s, const float2* src, float2* dst, int offset, int row_stride,
                    int slice_stride, int z_steps)
{
  constexpr int kCompute = kTileX * kTileY;
  switch (variant) {
    case 0:
      hipLaunchKernelGGL((stencil_2D_warp_specialized_single_buffer<kStencilAlign, kStencilBpt, kTileX, kTileY, kRadius, REACH, kStencilDma>),
                         grid, dim3(kCompute + kStencilDma), 0, s, src, dst, offset, row_stride, slice_stride, z_steps);
      break;
    case 1:
      hipLaunchKernelGGL((stencil_2D_warp_specialized_double_buffer<kStencilAlign, kStencilBpt, kTileX, kTileY, kRadius, REACH, kStencilDma>),
                         grid, dim3(kCompute + 2 * kStencilDma), 0, s, src, dst, offset, row_stride, slice_stride, z_steps);
      break;
    case 2:
      hipLaunchKernelGGL((stencil_2D_warp_specialized_manual_buffer<kStencilAlign, kStencilBpt, kTileX, kTileY, kRadius, REACH, kStencilDma>),
                         grid, dim3(kCompute + kStencilDma), 0, s, src, dst, offset, row_stride, slice_stride, z_steps);
      break;
    case 3:
      hipLaunchKernelGGL((stencil_2D_non_warp_specialized_single_buffer<kStencilAlign, kStencilBpt, kTileX, kTileY, kRadius, REACH>),
                         grid, dim3(kCompute), 0, s, src, dst, offset, row_stride, slice_stride, z_steps);
      break;
    default:
      hipLaunchKernelGGL((stencil_2D_non_warp_specialized_double_buffer<kStencilAlign, kStencilBpt, kTileX, kTileY, kRadius, REACH>),
                         grid, dim3(kCompute), 0, s, src, dst, offset, row_stride, slice_stride, z_steps);
      break;
  }
}

template<typename T, int N> constexpr int count_of(T (&)[N]) { return N; }

}  // namespace

extern "C" int cudadma_example_num_variants(int example)
{
  switch (example) {
    case CUDADMA_EXAMPLE_SAXPY: return count_of(kSaxpyNames);
    case CUDADMA_EXAMPLE_SGEMV: return count_of(kGemvNames);
    case CUDADMA_EXAMPLE_STENCIL2D: return count_of(kStencilNames);
    default: return 0;
  }
}

extern "C" const char* cudadma_example_variant_name(int example, int variant)
{
  if (variant < 0 || variant >= cudadma_example_num_variants(example)) return nullptr;
  switch (example) {
    case CUDADMA_EXAMPLE_SAXPY: return kSaxpyNames[variant];
    case CUDADMA_EXAMPLE_SGEMV: return kGemvNames[variant];
    default: return kStencilNames[variant];
  }
}

extern "C" int cudadma_example_saxpy(int variant, float a, const float* d_x, float* d_y, long long n, void* stream)
{
  if (variant < 0 || variant >= count_of(kSaxpyNames)) {
    cudadma_host::set_error("saxpy has no variant %d", variant);
    return CUDADMA_ERANGE;
  }
  constexpr int kChunk = SaxpyChunk<kSaxpyCompute>::kFloats;
  CUDADMA_REQUIRE(n >= 0, "n (%lld) is negative", n);
  CUDADMA_REQUIRE(variant == 0 || (n % kChunk) == 0, "n (%lld) must be a multiple of %d floats for this variant", n, kChunk);
  if (n == 0) return CUDADMA_OK;
  CUDADMA_REQUIRE(d_x != nullptr && d_y != nullptr, "NULL pointer");
  CUDADMA_REQUIRE(cudadma_host::aligned_to(d_x, 16) && cudadma_host::aligned_to(d_y, 16), "pointers must be 16-byte aligned");
  hipStream_t s = (hipStream_t)stream;
  const long long chunks = (n + kChunk - 1) / kChunk;
  const int grid = workloads::persistent_grid(chunks, 4);
  switch (variant) {
    case 0: hipLaunchKernelGGL(saxpy_baseline, dim3(grid), dim3(kSaxpyCompute), 0, s, d_y, d_x, a, n); break;
    case 1: hipLaunchKernelGGL(saxpy_vec4, dim3(grid), dim3(kSaxpyCompute), 0, s, d_y, d_x, a, n); break;
    case 2:
      hipLaunchKernelGGL((saxpy_dma_single<kSaxpyCompute, kSaxpyDmaPerLd>), dim3(grid), dim3(kSaxpyCompute + 2 * kSaxpyDmaPerLd),
                         0, s, d_y, d_x, a, chunks);
      break;
    default:
      hipLaunchKernelGGL((saxpy_dma_double<kSaxpyCompute, kSaxpyDmaPerLd>), dim3(grid), dim3(kSaxpyCompute + 4 * kSaxpyDmaPerLd),
                         0, s, d_y, d_x, a, chunks);
      break;
  }
  CUDADMA_HIP_CHECK(hipGetLastError());
  return CUDADMA_OK;
}

extern "C" int cudadma_example_sgemv(int variant, int n, int m, float alpha, const float* d_a, int lda, const float* d_x,
                                     float* d_y, void* stream)
{
  if (variant < 0 || variant >= count_of(kGemvNames)) {
    cudadma_host::set_error("sgemv has no variant %d", variant);
    return CUDADMA_ERANGE;
  }
  CUDADMA_REQUIRE(n >= 0 && m >= 0, "negative dimension (n %d, m %d)", n, m);
  CUDADMA_REQUIRE(lda >= n, "lda (%d) is smaller than n (%d)", lda, n);
  if (n == 0) return CUDADMA_OK;
  CUDADMA_REQUIRE(d_a != nullptr && d_x != nullptr && d_y != nullptr, "NULL pointer");
  CUDADMA_REQUIRE(cudadma_host::aligned_to(d_x, 16), "x must be 16-byte aligned");
  const int grid = (n + kGemvCompute - 1) / kGemvCompute;
  const int cols = variant == 0 ? kGemvVecElmts : variant == 1 ? 2 * kGemvVecElmts : kGemvPanelCols;
  CUDADMA_REQUIRE(m > 0 && (m % cols) == 0, "m (%d) must be a positive multiple of %d for this variant", m, cols);
  if (variant >= 2) {
    // the panel transfer reads whole groups of kGemvCompute rows with dwordx4 loads
    CUDADMA_REQUIRE(lda >= grid * kGemvCompute, "lda (%d) must cover %d rows (n rounded up to %d) when the matrix is staged",
                    lda, grid * kGemvCompute, kGemvCompute);
    CUDADMA_REQUIRE((lda % 4) == 0 && cudadma_host::aligned_to(d_a, 16), "A and lda*4 must be 16-byte aligned when the matrix is staged");
  }
  hipStream_t s = (hipStream_t)stream;
  switch (variant) {
    case 0:
      hipLaunchKernelGGL((sgemvn_vec_single<kGemvCompute, kGemvDmaPerLd, kGemvVecElmts>), dim3(grid),
                         dim3(kGemvCompute + kGemvDmaPerLd), 0, s, n, m, alpha, d_a, lda, d_x, d_y);
      break;
    case 1:
      hipLaunchKernelGGL((sgemvn_vec_manual<kGemvCompute, kGemvDmaPerLd, kGemvVecElmts>), dim3(grid),
                         dim3(kGemvCompute + kGemvDmaPerLd), 0, s, n, m, alpha, d_a, lda, d_x, d_y);
      break;
    case 2:
      hipLaunchKernelGGL((sgemvn_both_single<kGemvCompute, kGemvDmaPerLd, kGemvPanelCols, kGemvMatLds>), dim3(grid),
                         dim3(kGemvCompute + (1 + kGemvMatLds) * kGemvDmaPerLd), 0, s, n, m, alpha, d_a, lda, d_x, d_y);
      break;
    default:
      hipLaunchKernelGGL((sgemvn_both_double<kGemvCompute, kGemvDmaPerLd, kGemvPanelCols, kGemvMatLds>), dim3(grid),
                         dim3(kGemvCompute + 2 * (1 + kGemvMatLds) * kGemvDmaPerLd), 0, s, n, m, alpha, d_a, lda, d_x, d_y);
      break;
  }
  CUDADMA_HIP_CHECK(hipGetLastError());
  return CUDADMA_OK;
}

extern "C" int cudadma_example_stencil2d(int variant, const float* d_src, float* d_dst, int dimx, int dimy, int dimz,
                                         int full_cross, void* stream)
{
  if (variant < 0 || variant >= count_of(kStencilNames)) {
    cudadma_host::set_error("stencil2d has no variant %d", variant);
    return CUDADMA_ERANGE;
  }
  CUDADMA_REQUIRE(dimx > 0 && dimy > 0 && dimz > 0, "dimensions must be positive (%d x %d x %d)", dimx, dimy, dimz);
  CUDADMA_REQUIRE((dimx % kTileX) == 0 && (dimy % kTileY) == 0, "dimx must be a multiple of %d and dimy of %d", kTileX, kTileY);
  CUDADMA_REQUIRE(variant == 0 || variant == 3 || (dimz % 2) == 0, "dimz (%d) must be even for the variants with two buffers", dimz);
  CUDADMA_REQUIRE(d_src != nullptr && d_dst != nullptr, "NULL pointer");
  CUDADMA_REQUIRE(cudadma_host::aligned_to(d_src, 16) && cudadma_host::aligned_to(d_dst, 8), "src must be 16-byte, dst 8-byte aligned");
  const long long row_stride = dimx + 2 * kRadius;
  const long long slice_stride = (dimy + 2 * kRadius) * row_stride;
  const long long offset = kRadius * slice_stride + kRadius * row_stride + kRadius;
  CUDADMA_REQUIRE(slice_stride * (dimz + 2 * kRadius) <= 0x7fffffffLL / 8, "volume too large for int element offsets");
  const dim3 grid(dimx / kTileX, dimy / kTileY);
  hipStream_t s = (hipStream_t)stream;
  const float2* src = reinterpret_cast<const float2*>(d_src);
  float2* dst = reinterpret_cast<float2*>(d_dst);
  if (full_cross)
    launch_stencil<kRadius>(variant, grid, s, src, dst, (int)offset, (int)row_stride, (int)slice_stride, dimz);
  else
    launch_stencil<kRadius - 1>(variant, grid, s, src, dst, (int)offset, (int)row_stride, (int)slice_stride, dimz);
  CUDADMA_HIP_CHECK(hipGetLastError());
  return CUDADMA_OK;
}
