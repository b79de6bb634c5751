// Config 5: C = A * B, bf16 inputs, fp32 accumulate, warp-specialised and
// double-buffered.  The reference has no GEMM; the nearest code is the SGEMV of
// src/examples/sgemv/sgemv_dma.cu:329-388 (Strided matrix tiles staged by DMA
// warps, FMA loop in the compute warps).  Here:
//   * workgroup tile 128 x 128 of C, K step 64;
//   * wavefronts 4-5 stage the A tiles (128 rows x 128 B, source stride K*2 bytes),
//     wavefronts 6-7 the B tiles (64 rows x 256 B, source stride N*2 bytes).  Each
//     pair owns two CudaDMAStrided objects, one per LDS stage, and uses the two-phase
//     calls so that the tile two K steps ahead is already in flight (in the
//     object's registers) while the current one is consumed: a K step is shorter
//     than a trip to memory, one tile of look-ahead is not enough;
//   * wavefronts 0..3 each own a 64 x 64 quadrant: 2 x 2 blocks of
//     v_mfma_f32_32x32x16_bf16.  A fragments are ds_read_b128 from rows padded to
//     144 B; B stays row-major [k][n] in LDS (rows padded to 320 B) and is turned
//     into k-major fragments on the way to the registers by ds_read_b64_tr_b16.
#include "workloads.hpp"

namespace {

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4_t __attribute__((ext_vector_type(4)));
typedef float f32x16_t __attribute__((ext_vector_type(16)));

constexpr int kBM = 128, kBN = 128, kBK = 64;
constexpr int kComputeThreads = 256;
constexpr int kDmaWave = 128;              // DMA threads per operand: two wavefronts
constexpr int kAPitch = kBK * 2 + 16;        // 144 B per A row in LDS
constexpr int kBPitch = kBN * 2 + 64;        // 320 B per B row in LDS: the four rows a transposing read touches land 64 B apart modulo 256
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
  dma_a_t dma_a0(0, kComputeThreads, kComputeThreads, k * 2, kAPitch);
  dma_a_t dma_a1(1, kComputeThreads, kComputeThreads, k * 2, kAPitch);
  dma_b_t dma_b0(2, kComputeThreads, kComputeThreads + kDmaWave, n * 2, kBPitch);
  dma_b_t dma_b1(3, kComputeThreads, kComputeThreads + kDmaWave, n * 2, kBPitch);
  const int tiles_n = n / kBN;
  const int tile_m = blockIdx.x / tiles_n, tile_n = blockIdx.x % tiles_n;
  const int ksteps = k / kBK;            // even: k is a multiple of 2 * kBK
  const int klast = ksteps - 1;

  // One DMA wavefront: tiles kt and kt+1 are requested up front, then every landed tile is
  // followed by the request for the tile two steps on (clamped past the end so that no load
  // sits behind a branch and s_waitcnt can leave the younger tile in flight).
  auto stage_tiles = [&](auto& d0, auto& d1, char* s0, char* s1, const unsigned short* src, const size_t step) {
    d0.template start_xfer_async<true, LOAD_CACHE_ALL, STORE_LDS>(src);
    d1.template start_xfer_async<true, LOAD_CACHE_ALL, STORE_LDS>(src + step);
    for (int kt = 0; kt < ksteps; kt += 2) {
      d0.template wait_xfer_finish<true, LOAD_CACHE_ALL, STORE_LDS>(s0);
      d0.template start_xfer_async<true, LOAD_CACHE_ALL, STORE_LDS>(src + (size_t)(kt + 2 < klast ? kt + 2 : klast) * step);
      d1.template wait_xfer_finish<true, LOAD_CACHE_ALL, STORE_LDS>(s1);
      d1.template start_xfer_async<true, LOAD_CACHE_ALL, STORE_LDS>(src + (size_t)(kt + 3 < klast ? kt + 3 : klast) * step);
    }
  };
  if (dma_a0.owns_this_thread()) {
    stage_tiles(dma_a0, dma_a1, lds_a[0], lds_a[1], a + (size_t)tile_m * kBM * k, (size_t)kBK);
  } else if (dma_b0.owns_this_thread()) {
    stage_tiles(dma_b0, dma_b1, lds_b[0], lds_b[1], b + (size_t)tile_n * kBN, (size_t)kBK * n);
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
    // both stages are free to begin with
    dma_a0.start_async_dma(); dma_a1.start_async_dma();
    dma_b0.start_async_dma(); dma_b1.start_async_dma();
    // A fragment: row wm + 32*i + lane%32, eight k starting at 16*ks + 8*(lane/32)
    const int a_off = (wm + (lane & 31)) * kAPitch + (lane >> 5) * 16;
    // B fragment through the transposing read: inside a group of 16 lanes, lane j points at
    // row (j/4) of a 4-row block and at column 4*(j%4); lane i then receives rows 0..3 of column i.
    const int j16 = lane & 15;
    const int b_off = ((lane >> 5) * 8 + (j16 >> 2)) * kBPitch + (wn + ((lane >> 4) & 1) * 16 + (j16 & 3) * 4) * 2;
    auto k_step = [&](const dma_a_t& da, const dma_b_t& db, const char* sa, const char* sb) {
      da.wait_for_dma_finish();
      db.wait_for_dma_finish();
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
      da.start_async_dma();
      db.start_async_dma();
    };
    for (int kt = 0; kt < ksteps; kt += 2) {
      k_step(dma_a0, dma_b0, lds_a[0] + a_off, lds_b[0] + b_off);
      k_step(dma_a1, dma_b1, lds_a[1] + a_off, lds_b[1] + b_off);
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
  CUDADMA_REQUIRE((m % kBM) == 0 && (n % kBN) == 0 && (k % (2 * kBK)) == 0,
                  "m, n and k must be multiples of 128 (got %d x %d x %d)", m, n, k);
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
