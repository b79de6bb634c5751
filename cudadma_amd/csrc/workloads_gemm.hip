// Config 5: C = A * B, bf16 inputs, fp32 accumulate, warp-specialised and
// double-buffered.  The reference has no GEMM; the nearest code is the SGEMV of
// src/examples/sgemv/sgemv_dma.cu:329-388 (Strided matrix tiles staged by DMA
// warps, FMA loop in the compute warps).  Here:
//   * workgroup tile 128 x 128 of C, K step 64;
//   * wavefront 4 stages the A tile (128 rows x 128 B, source stride K*2 bytes),
//     wavefront 5 the B tile (64 rows x 256 B, source stride N*2 bytes), each with
//     one CudaDMAStrided object that alternates between two LDS stages.  One
//     object can guard two buffers because the handshake words only count: the
//     compute wavefronts hand out two "empty" credits up front, then one per
//     consumed tile;
//   * wavefronts 0..3 each own a 64 x 64 quadrant: 2 x 2 blocks of
//     v_mfma_f32_32x32x16_bf16.  A fragments are ds_read_b128 from rows padded to
//     144 B; B stays row-major [k][n] in LDS (rows padded to 272 B) and is turned
//     into k-major fragments on the way to the registers by ds_read_b64_tr_b16.
#include "workloads.hpp"

namespace {

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4_t __attribute__((ext_vector_type(4)));
typedef float f32x16_t __attribute__((ext_vector_type(16)));

constexpr int kBM = 128, kBN = 128, kBK = 64;
constexpr int kComputeThreads = 256;
constexpr int kDmaWave = 64;
constexpr int kAPitch = kBK * 2 + 16;        // 144 B per A row in LDS
constexpr int kBPitch = kBN * 2 + 16;        // 272 B per B row in LDS
constexpr int kAStage = kBM * kAPitch;       // 18432
constexpr int kBStage = kBK * kBPitch;       // 17408

typedef CudaDMAStrided<true, 16, kBM * kBK * 2 / kDmaWave, kBK * 2, kDmaWave, kBM> dma_a_t;   // 128 rows x 128 B
typedef CudaDMAStrided<true, 16, kBK * kBN * 2 / kDmaWave, kBN * 2, kDmaWave, kBK> dma_b_t;   // 64 rows x 256 B

__global__ void __launch_bounds__(kComputeThreads + 2 * kDmaWave)
gemm_bf16_ws(const unsigned short* __restrict__ a, const unsigned short* __restrict__ b, float* __restrict__ c,
             const int m, const int n, const int k)
{
  __shared__ __attribute__((aligned(16))) char lds_a[2][kAStage];
  __shared__ __attribute__((aligned(16))) char lds_b[2][kBStage];
  dma_a_t dma_a(0, kComputeThreads, kComputeThreads, k * 2, kAPitch);
  dma_b_t dma_b(1, kComputeThreads, kComputeThreads + kDmaWave, n * 2, kBPitch);
  const int tiles_n = n / kBN;
  const int tile_m = blockIdx.x / tiles_n, tile_n = blockIdx.x % tiles_n;
  const int ksteps = k / kBK;

  if (dma_a.owns_this_thread()) {
    const unsigned short* src = a + (size_t)tile_m * kBM * k;
    dma_a.template start_xfer_async<true, LOAD_CACHE_ALL, STORE_LDS>(src);
    for (int kt = 0; kt < ksteps; ++kt) {
      dma_a.template wait_xfer_finish<true, LOAD_CACHE_ALL, STORE_LDS>(lds_a[kt & 1]);
      // past the last step the last tile is requested again: the loads stay unconditional
      const int kn = (kt + 1 < ksteps) ? (kt + 1) : kt;
      dma_a.template start_xfer_async<true, LOAD_CACHE_ALL, STORE_LDS>(src + (size_t)kn * kBK);
    }
  } else if (dma_b.owns_this_thread()) {
    const unsigned short* src = b + (size_t)tile_n * kBN;
    dma_b.template start_xfer_async<true, LOAD_CACHE_ALL, STORE_LDS>(src);
    for (int kt = 0; kt < ksteps; ++kt) {
      dma_b.template wait_xfer_finish<true, LOAD_CACHE_ALL, STORE_LDS>(lds_b[kt & 1]);
      const int kn = (kt + 1 < ksteps) ? (kt + 1) : kt;
      dma_b.template start_xfer_async<true, LOAD_CACHE_ALL, STORE_LDS>(src + (size_t)kn * kBK * n);
    }
  } else {
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int wm = (wave >> 1) * 64, wn = (wave & 1) * 64;     // quadrant of the 128 x 128 tile
    f32x16_t acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int j = 0; j < 2; ++j)
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.0f;
    // two stages are free to begin with
    dma_a.start_async_dma(); dma_a.start_async_dma();
    dma_b.start_async_dma(); dma_b.start_async_dma();
    // A fragment: row wm + 32*i + lane%32, eight k starting at 16*ks + 8*(lane/32)
    const int a_off = (wm + (lane & 31)) * kAPitch + (lane >> 5) * 16;
    // B fragment through the transposing read: inside a group of 16 lanes, lane j points at
    // row (j/4) of a 4-row block and at column 4*(j%4); lane i then receives rows 0..3 of column i.
    const int j16 = lane & 15;
    const int b_off = ((lane >> 5) * 8 + (j16 >> 2)) * kBPitch + (wn + ((lane >> 4) & 1) * 16 + (j16 & 3) * 4) * 2;
    for (int kt = 0; kt < ksteps; ++kt) {
      dma_a.wait_for_dma_finish();
      dma_b.wait_for_dma_finish();
      const char* sa = lds_a[kt & 1] + a_off;
      const char* sb = lds_b[kt & 1] + b_off;
#pragma unroll
      for (int ks = 0; ks < kBK / 16; ++ks) {
        bf16x8_t fa[2], fb[2];
#pragma unroll
        for (int i = 0; i < 2; ++i)
          fa[i] = *(const bf16x8_t*)(sa + i * 32 * kAPitch + ks * 32);
#pragma unroll
        for (int j = 0; j < 2; ++j) {
          const char* p = sb + ks * 16 * kBPitch + j * 32 * 2;
          const bf16x4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((__attribute__((address_space(3))) bf16x4_t*)p);
          const bf16x4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4bf16(
              (__attribute__((address_space(3))) bf16x4_t*)(p + 4 * kBPitch));
          fb[j] = bf16x8_t{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
        }
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
          for (int j = 0; j < 2; ++j)
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[i], fb[j], acc[i][j], 0, 0, 0);
      }
      dma_a.start_async_dma();
      dma_b.start_async_dma();
    }
    // 32 x 32 block: register e of lane L holds row 8*(e/4) + 4*(L/32) + e%4, column L%32
    float* cbase = c + (size_t)(tile_m * kBM + wm) * n + (size_t)tile_n * kBN + wn;
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int j = 0; j < 2; ++j)
#pragma unroll
        for (int e = 0; e < 16; ++e) {
          const int row = i * 32 + 8 * (e / 4) + 4 * (lane >> 5) + (e % 4);
          const int col = j * 32 + (lane & 31);
          cbase[(size_t)row * n + col] = acc[i][j][e];
        }
  }
}

}  // namespace

extern "C" int cudadma_gemm_bf16(const uint16_t* d_a, const uint16_t* d_b, float* d_c, int m, int n, int k,
                                 int variant, void* stream)
{
  CUDADMA_REQUIRE(m > 0 && n > 0 && k > 0, "dimensions must be positive");
  CUDADMA_REQUIRE((m % kBM) == 0 && (n % kBN) == 0 && (k % kBK) == 0,
                  "m and n must be multiples of 128 and k a multiple of 64 (got %d x %d x %d)", m, n, k);
  if (variant < 0 || variant >= cudadma_num_variants(CUDADMA_WORKLOAD_GEMM)) {
    cudadma_host::set_error("gemm has no variant %d", variant);
    return CUDADMA_ERANGE;
  }
  CUDADMA_REQUIRE(d_a != nullptr && d_b != nullptr && d_c != nullptr, "NULL pointer");
  CUDADMA_REQUIRE(cudadma_host::aligned_to(d_a, 16) && cudadma_host::aligned_to(d_b, 16) && cudadma_host::aligned_to(d_c, 16),
                  "pointers must be 16-byte aligned");
  CUDADMA_REQUIRE((long long)k * 2 <= 0x7fffffffLL && (long long)n * 2 <= 0x7fffffffLL, "row pitch must fit an int");
  const long long grid = (long long)(m / kBM) * (n / kBN);
  CUDADMA_REQUIRE(grid <= 0x7fffffffLL, "grid too large");
  hipLaunchKernelGGL(gemm_bf16_ws, dim3((unsigned)grid), dim3(kComputeThreads + 2 * kDmaWave), 0, (hipStream_t)stream,
                     d_a, d_b, d_c, m, n, k);
  CUDADMA_HIP_CHECK(hipGetLastError());
  return CUDADMA_OK;
}
