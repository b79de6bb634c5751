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

constexpr int kBK = 64;
constexpr int kComputeThreads = 256;
constexpr int kDmaWave = 128;              // DMA threads per operand: two wavefronts

// Tile geometry for compute wavefronts that each own WI x WJ blocks of 32 x 32: the four
// wavefronts sit 2 x 2, so the workgroup tile is 64*WI x 64*WJ.
template<int WI, int WJ>
struct GemmShape {
  static constexpr int kBM = 64 * WI, kBN = 64 * WJ;
  static constexpr int kAPitch = kBK * 2 + 16;      // 144 B per A row in LDS
  static constexpr int kBPitch = kBN * 2 + 64;      // B row in LDS: the four rows a transposing read touches land 64 B apart modulo 256
  static constexpr int kAStage = kBM * kAPitch;
  static constexpr int kBStage = kBK * kBPitch;
  typedef CudaDMAStrided<false, 16, kBM * kBK * 2 / kDmaWave, kBK * 2, kDmaWave, kBM> dma_a_t;   // kBM rows x 128 B
  typedef CudaDMAStrided<false, 16, kBK * kBN * 2 / kDmaWave, kBN * 2, kDmaWave, kBK> dma_b_t;   // 64 rows x 2*kBN B
};

// Workgroup -> tile.  Workgroup b runs on XCD b % 8; when the tile grid divides into eight
// 2-D blocks (4 along m, 2 along n) every XCD gets one compact block, so its L2 holds few
// distinct A and B panels; otherwise tiles are dealt row-major.
__device__ __forceinline__ void tile_of_workgroup(const int b, const int tiles_m, const int tiles_n, int& tile_m, int& tile_n)
{
  if ((tiles_m % 4) == 0 && (tiles_n % 2) == 0) {
    const int xcd = b & 7, idx = b >> 3;
    const int bm = tiles_m / 4, bn = tiles_n / 2;       // block of one XCD
    tile_m = (xcd >> 1) * bm + idx / bn;
    tile_n = (xcd & 1) * bn + idx % bn;
  } else {
    tile_m = b / tiles_n;
    tile_n = b % tiles_n;
  }
}

// Order of one slice for the instruction scheduler: MFMAs matrix instructions with the READS
// LDS requests of the next slice issued two at a time behind the first of them; the last
// matrix instructions run with nothing behind them, so the data has landed when the next
// slice starts.
template<int G, int MFMAS, int READS>
__device__ __forceinline__ void pin_slice()
{
  if constexpr (G < MFMAS) {
    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);                                    // one MFMA
    if constexpr (2 * G + 2 <= READS) __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);   // two LDS reads
    else if constexpr (2 * G < READS) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
    pin_slice<G + 1, MFMAS, READS>();
  }
}

template<int WI, int WJ>
__global__ void __launch_bounds__(kComputeThreads + 2 * kDmaWave)
gemm_bf16_ws(const unsigned short* __restrict__ a, const unsigned short* __restrict__ b, float* __restrict__ c,
             const int m, const int n, const int k)
{
  typedef GemmShape<WI, WJ> shape;
  typedef typename shape::dma_a_t dma_a_t;
  typedef typename shape::dma_b_t dma_b_t;
  constexpr int kAPitch = shape::kAPitch, kBPitch = shape::kBPitch;
  __shared__ __attribute__((aligned(16))) char lds_a[2][shape::kAStage];
  __shared__ __attribute__((aligned(16))) char lds_b[2][shape::kBStage];
  // The transfer objects carry no handshake of their own: a stage holds an A tile and a B tile,
  // and one sync object per stage covers the four DMA wavefronts of both operands, so the
  // compute wavefronts wait and signal once per stage instead of once per operand.
  dma_a_t dma_a0(k * 2, kAPitch, kComputeThreads);
  dma_a_t dma_a1(k * 2, kAPitch, kComputeThreads);
  dma_b_t dma_b0(n * 2, kBPitch, kComputeThreads + kDmaWave);
  dma_b_t dma_b1(n * 2, kBPitch, kComputeThreads + kDmaWave);
  cudaDMACustom stage0(0, 2 * kDmaWave, kComputeThreads, kComputeThreads);
  cudaDMACustom stage1(1, 2 * kDmaWave, kComputeThreads, kComputeThreads);
  int tile_m, tile_n;
  tile_of_workgroup(blockIdx.x, m / shape::kBM, n / shape::kBN, tile_m, tile_n);
  const int ksteps = k / kBK;            // even: k is a multiple of 2 * kBK
  const int klast = ksteps - 1;

  // One DMA wavefront: tiles kt and kt+1 are requested up front, then every landed tile is
  // followed by the request for the tile two steps on (clamped past the end so that no load
  // sits behind a branch and s_waitcnt can leave the younger tile in flight).
  auto stage_tiles = [&](auto& d0, auto& d1, char* s0, char* s1, const unsigned short* src, const size_t step) {
    d0.template start_xfer_async<true, LOAD_CACHE_ALL, STORE_LDS>(src);
    d1.template start_xfer_async<true, LOAD_CACHE_ALL, STORE_LDS>(src + step);
    for (int kt = 0; kt < ksteps; kt += 2) {
      stage0.wait_for_dma_start();
      d0.template wait_xfer_finish<true, LOAD_CACHE_ALL, STORE_LDS>(s0);
      stage0.finish_async_dma();
      d0.template start_xfer_async<true, LOAD_CACHE_ALL, STORE_LDS>(src + (size_t)(kt + 2 < klast ? kt + 2 : klast) * step);
      stage1.wait_for_dma_start();
      d1.template wait_xfer_finish<true, LOAD_CACHE_ALL, STORE_LDS>(s1);
      stage1.finish_async_dma();
      d1.template start_xfer_async<true, LOAD_CACHE_ALL, STORE_LDS>(src + (size_t)(kt + 3 < klast ? kt + 3 : klast) * step);
    }
  };
  if (dma_a0.owns_this_thread()) {
    stage_tiles(dma_a0, dma_a1, lds_a[0], lds_a[1], a + (size_t)tile_m * shape::kBM * k, (size_t)kBK);
  } else if (dma_b0.owns_this_thread()) {
    stage_tiles(dma_b0, dma_b1, lds_b[0], lds_b[1], b + (size_t)tile_n * shape::kBN, (size_t)kBK * n);
  } else {
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int wm = (wave >> 1) * 32 * WI, wn = (wave & 1) * 32 * WJ;     // this wavefront's corner in the workgroup tile
    f32x16_t acc[WI][WJ];
#pragma unroll
    for (int i = 0; i < WI; ++i)
#pragma unroll
      for (int j = 0; j < WJ; ++j)
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.0f;
    // both stages are free to begin with
    stage0.start_async_dma();
    stage1.start_async_dma();
    // A fragment: row wm + 32*i + lane%32, eight k starting at 16*ks + 8*(lane/32)
    const int a_off = (wm + (lane & 31)) * kAPitch + (lane >> 5) * 16;
    // B fragment through the transposing read: inside a group of 16 lanes, lane j points at
    // row (j/4) of a 4-row block and at column 4*(j%4); lane i then receives rows 0..3 of column i.
    const int j16 = lane & 15;
    const int b_off = ((lane >> 5) * 8 + (j16 >> 2)) * kBPitch + (wn + ((lane >> 4) & 1) * 16 + (j16 & 3) * 4) * 2;
    // With 128 accumulator registers a SIMD holds one compute wavefront, which has to hide its
    // own LDS latency: the order "request the next slice, then multiply the current one" is
    // pinned against the instruction scheduler.  With the small tile two workgroups share a
    // compute unit and the scheduler's own order does better.
    constexpr bool kPinned = (WI * WJ >= 8);
    // Fragments of one 16-deep slice of the K step: WI row blocks of A, WJ column blocks of B.
    auto load_frags = [&](bf16x8_t (&fa)[WI], bf16x8_t (&fb)[WJ], const char* sa, const char* sb, const int ks)
        __attribute__((always_inline)) {
#pragma unroll
      for (int i = 0; i < WI; ++i)
        fa[i] = *(const bf16x8_t*)(sa + i * 32 * kAPitch + ks * 32);
#pragma unroll
      for (int j = 0; j < WJ; ++j) {
        const char* p = sb + ks * 16 * kBPitch + j * 32 * 2;
        const bf16x4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((__attribute__((address_space(3))) bf16x4_t*)p);
        const bf16x4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4bf16(
            (__attribute__((address_space(3))) bf16x4_t*)(p + 4 * kBPitch));
        fb[j] = bf16x8_t{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
      }
    };
    auto multiply = [&](const bf16x8_t (&fa)[WI], const bf16x8_t (&fb)[WJ]) __attribute__((always_inline)) {
#pragma unroll
      for (int i = 0; i < WI; ++i)
#pragma unroll
        for (int j = 0; j < WJ; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[i], fb[j], acc[i][j], 0, 0, 0);
    };
    // One slice of the pinned schedule: the WI + 2*WJ LDS requests of the next slice are
    // issued one by one in the shadow of the WI*WJ matrix instructions of the current slice
    // (a matrix instruction holds its pipe for 32 cycles, the wavefront is free to issue an
    // LDS request meanwhile), and nothing moves across the ends of the slice.
    auto interleave = [&]() __attribute__((always_inline)) {
      if constexpr (kPinned) {
        pin_slice<0, WI * WJ, WI + 2 * WJ>();
        __builtin_amdgcn_sched_barrier(0);
      }
    };
    // The one compute wavefront of a SIMD has to keep the matrix core fed by itself: the
    // fragments of the next slice are requested before the products of the current one are
    // issued, across the stage boundary too (the next stage is waited for, and its first slice
    // requested, ahead of the last products of the current stage).
    const char* sa0 = lds_a[0] + a_off; const char* sb0 = lds_b[0] + b_off;
    const char* sa1 = lds_a[1] + a_off; const char* sb1 = lds_b[1] + b_off;
    bf16x8_t fa0[WI], fb0[WJ], fa1[WI], fb1[WJ];
    static_assert(kBK / 16 == 4, "the slice schedule below is written for four slices per stage");
    if constexpr (!kPinned) {
      for (int kt = 0; kt < ksteps; kt += 2) {
        stage0.wait_for_dma_finish();
#pragma unroll
        for (int ks = 0; ks < kBK / 16; ++ks) { load_frags(fa0, fb0, sa0, sb0, ks); multiply(fa0, fb0); }
        stage0.start_async_dma();
        stage1.wait_for_dma_finish();
#pragma unroll
        for (int ks = 0; ks < kBK / 16; ++ks) { load_frags(fa0, fb0, sa1, sb1, ks); multiply(fa0, fb0); }
        stage1.start_async_dma();
      }
    } else {
      stage0.wait_for_dma_finish();
      load_frags(fa0, fb0, sa0, sb0, 0);
      for (int kt = 0; kt < ksteps; kt += 2) {
        load_frags(fa1, fb1, sa0, sb0, 1); multiply(fa0, fb0); interleave();
        load_frags(fa0, fb0, sa0, sb0, 2); multiply(fa1, fb1); interleave();
        // the `full` word of the next stage is read here and looked at one slice later
        const unsigned seen1 = stage1.peek_dma_finish();
        load_frags(fa1, fb1, sa0, sb0, 3); multiply(fa0, fb0); interleave();
        stage1.wait_for_dma_finish(seen1);
        load_frags(fa0, fb0, sa1, sb1, 0); multiply(fa1, fb1); interleave();
        stage0.start_async_dma();
        load_frags(fa1, fb1, sa1, sb1, 1); multiply(fa0, fb0); interleave();
        load_frags(fa0, fb0, sa1, sb1, 2); multiply(fa1, fb1); interleave();
        const unsigned seen0 = stage0.peek_dma_finish();
        load_frags(fa1, fb1, sa1, sb1, 3); multiply(fa0, fb0); interleave();
        if (kt + 2 < ksteps) {
          stage0.wait_for_dma_finish(seen0);
          load_frags(fa0, fb0, sa0, sb0, 0);
        }
        multiply(fa1, fb1); interleave();
        stage1.start_async_dma();
      }
    }
    // 32 x 32 block: register e of lane L holds row 8*(e/4) + 4*(L/32) + e%4, column L%32
    float* cbase = c + (size_t)(tile_m * shape::kBM + wm) * n + (size_t)tile_n * shape::kBN + wn;
#pragma unroll
    for (int i = 0; i < WI; ++i)
#pragma unroll
      for (int j = 0; j < WJ; ++j)
#pragma unroll
        for (int e = 0; e < 16; ++e) {
          const int row = i * 32 + 8 * (e / 4) + 4 * (lane >> 5) + (e % 4);
          const int col = j * 32 + (lane & 31);
          cbase[(size_t)row * n + col] = acc[i][j][e];
        }
  }
}

template<int WI, int WJ>
int launch_gemm(const uint16_t* d_a, const uint16_t* d_b, float* d_c, int m, int n, int k, hipStream_t stream)
{
  typedef GemmShape<WI, WJ> shape;
  CUDADMA_REQUIRE((m % shape::kBM) == 0 && (n % shape::kBN) == 0,
                  "this variant needs m a multiple of %d and n of %d (got %d x %d)", shape::kBM, shape::kBN, m, n);
  const long long grid = (long long)(m / shape::kBM) * (n / shape::kBN);
  CUDADMA_REQUIRE(grid <= 0x7fffffffLL, "grid too large");
  hipLaunchKernelGGL((gemm_bf16_ws<WI, WJ>), dim3((unsigned)grid), dim3(kComputeThreads + 2 * kDmaWave), 0, stream,
                     d_a, d_b, d_c, m, n, k);
  CUDADMA_HIP_CHECK(hipGetLastError());
  return CUDADMA_OK;
}

}  // namespace

extern "C" int cudadma_gemm_bf16(const uint16_t* d_a, const uint16_t* d_b, float* d_c, int m, int n, int k,
                                 int variant, void* stream)
{
  CUDADMA_REQUIRE(m > 0 && n > 0 && k > 0, "dimensions must be positive");
  CUDADMA_REQUIRE((m % 128) == 0 && (n % 128) == 0 && (k % (2 * kBK)) == 0,
                  "m, n and k must be multiples of 128 (got %d x %d x %d)", m, n, k);
  if (variant < 0 || variant >= cudadma_num_variants(CUDADMA_WORKLOAD_GEMM)) {
    cudadma_host::set_error("gemm has no variant %d", variant);
    return CUDADMA_ERANGE;
  }
  CUDADMA_REQUIRE(d_a != nullptr && d_b != nullptr && d_c != nullptr, "NULL pointer");
  CUDADMA_REQUIRE(cudadma_host::aligned_to(d_a, 16) && cudadma_host::aligned_to(d_b, 16) && cudadma_host::aligned_to(d_c, 16),
                  "pointers must be 16-byte aligned");
  CUDADMA_REQUIRE((long long)k * 2 <= 0x7fffffffLL && (long long)n * 2 <= 0x7fffffffLL, "row pitch must fit an int");
  hipStream_t s = (hipStream_t)stream;
  if (variant == 0) variant = (m % 256) == 0 ? 3 : 1;      // the largest tile that divides the problem
  switch (variant) {
    case 1: return launch_gemm<2, 2>(d_a, d_b, d_c, m, n, k, s);
    case 2: return launch_gemm<2, 4>(d_a, d_b, d_c, m, n, k, s);
    default: return launch_gemm<4, 2>(d_a, d_b, d_c, m, n, k, s);
  }
}
