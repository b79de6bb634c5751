// Config 5: C = A * B, bf16 inputs, fp32 accumulate, warp-specialised and
// double-buffered.  The reference has no GEMM; the nearest code is the SGEMV of
// src/examples/sgemv/sgemv_dma.cu:329-388 (Strided matrix tiles staged by DMA
// warps, FMA loop in the compute warps).  Here, for a workgroup tile BM x BN and K step 64:
//   * the first WM x WN wavefronts compute, each on WI x WJ blocks of
//     v_mfma_f32_32x32x16_bf16 (BM = 32*WI*WM, BN = 32*WJ*WN).  A fragments are
//     ds_read_b128 from rows padded to 144 B; B stays row-major [k][n] in LDS (rows
//     padded by 64 B) and is turned into k-major fragments on the way to the
//     registers by ds_read_b64_tr_b16;
//   * the next two wavefronts stage the A tiles (BM rows x 128 B, source stride K*2
//     bytes), the last two the B tiles (64 rows x 2*BN B, source stride N*2 bytes).
//     Each pair owns two CudaDMAStrided objects, one per LDS stage, and uses the
//     two-phase calls so that the tile two K steps ahead is already in flight (in the
//     object's registers) while the current one is consumed: a K step is shorter
//     than a trip to memory, one tile of look-ahead is not enough.
// Four compute wavefronts (2 x 2) share the SIMDs with the four DMA wavefronts one to
// one and get 256 registers each; eight (2 x 4, the 256 x 256 tile) make it three
// wavefronts per SIMD and 168 registers each, but two of them compute.
#include "workloads.hpp"

namespace {

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4_t __attribute__((ext_vector_type(4)));
typedef float f32x16_t __attribute__((ext_vector_type(16)));

constexpr int kBK = 64;
constexpr int kComputeThreads = 256;
constexpr int kDmaWave = 128;              // DMA threads per operand: two wavefronts

// Tile geometry for compute wavefronts that each own WI x WJ blocks of 32 x 32: the WM x WN
// wavefronts sit in a grid, so the workgroup tile is 32*WI*WM x 32*WJ*WN.
template<int WI, int WJ, int WM = 2, int WN = 2>
struct GemmShape {
  static constexpr int kCompute = 64 * WM * WN;     // compute threads; the DMA threads follow them
  static constexpr int kBM = 32 * WI * WM, kBN = 32 * WJ * WN;
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

template<int WI, int WJ, int WM = 2, int WN = 2>
__global__ void __launch_bounds__(64 * WM * WN + 2 * kDmaWave)
gemm_bf16_ws(const unsigned short* __restrict__ a, const unsigned short* __restrict__ b, float* __restrict__ c,
             const int m, const int n, const int k)
{
  typedef GemmShape<WI, WJ, WM, WN> shape;
  constexpr int kComputeThreads = shape::kCompute;
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
  auto stage_tiles = [&](auto& d0, auto& d1, char* s0, char* s1, const unsigned short* src, const size_t step)
      __attribute__((always_inline)) {
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
    const int wm = (wave / WN) * 32 * WI, wn = (wave % WN) * 32 * WJ;     // this wavefront's corner in the workgroup tile
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
    constexpr bool kPinned = (WI * WJ >= 8) && (WM * WN == 4);
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
          __builtin_nontemporal_store(acc[i][j][e], &cbase[(size_t)row * n + col]);
        }
  }
}

// ---- the same GEMM with the tiles brought in by global_load_lds_dwordx4 ----
// Why: a ds_write_b128 and a ds_read of another wavefront take turns on the LDS, a direct-to-LDS
// load does not hold up the reads (measured: readers + ds_write run as long as the sum of the
// two, readers + global_load_lds as long as the loads alone).  The tiles land unpadded, with the
// chunks of every row XOR-swizzled (STORE_LDS_DIRECT_SWIZZLE); without padding three stages fit
// in LDS (3 x 48 KB), and they are needed: a direct transfer cannot be requested before its stage
// is free, so the memory latency has to fit into two K steps instead of being bridged by
// registers.  Each DMA wavefront keeps two transfers in flight (issue_direct + wait_direct_loads).
template<typename T>
struct Three {
  T a0, a1, a2;
  template<int I> __device__ __forceinline__ T& get() { if constexpr (I == 0) return a0; else if constexpr (I == 1) return a1; else return a2; }
};

#ifdef HIPDMA_SWEEP_VARIANTS
__global__ void __launch_bounds__(kComputeThreads + 2 * kDmaWave)
gemm_bf16_ws_direct(const unsigned short* __restrict__ a, const unsigned short* __restrict__ b, float* __restrict__ c,
                    const int m, const int n, const int k)
{
  constexpr int WI = 4, WJ = 2, kStages = 3;
  constexpr int kBM = 64 * WI, kBN = 64 * WJ;
  constexpr int kARow = kBK * 2, kBRow = kBN * 2;                 // 128 B and 256 B, unpadded
  constexpr int kAStage = kBM * kARow, kBStage = kBK * kBRow;     // 32 KB and 16 KB
  typedef CudaDMAStrided<false, 16, 16, kARow, kDmaWave, kBM> dma_a_t;
  typedef CudaDMAStrided<false, 16, 16, kBRow, kDmaWave, kBK> dma_b_t;
  __shared__ __attribute__((aligned(1024))) char lds_a[kStages][kAStage];
  __shared__ __attribute__((aligned(1024))) char lds_b[kStages][kBStage];
  dma_a_t dma_a(k * 2, kARow, kComputeThreads);
  dma_b_t dma_b(n * 2, kBRow, kComputeThreads + kDmaWave);
  Three<cudaDMACustom> stage{cudaDMACustom(0, 2 * kDmaWave, kComputeThreads, kComputeThreads),
                             cudaDMACustom(1, 2 * kDmaWave, kComputeThreads, kComputeThreads),
                             cudaDMACustom(2, 2 * kDmaWave, kComputeThreads, kComputeThreads)};
  int tile_m, tile_n;
  tile_of_workgroup(blockIdx.x, m / kBM, n / kBN, tile_m, tile_n);
  const int ksteps = k / kBK;

  // One DMA wavefront: tile t lands in stage t % 3.  Tiles t+1 and t+2 are in flight while the
  // compute wavefronts work on tile t: the wavefront waits for tile t (leaving the younger
  // loads in flight), reports it, and then requests tile t+2 as soon as its stage is free.
  auto feed = [&](auto& dma, char* lds, auto stage_bytes, const unsigned short* src, const size_t step)
      __attribute__((always_inline)) {
    constexpr int kStageBytes = decltype(stage_bytes)::value;
    constexpr int kLoads = std::remove_reference<decltype(dma)>::type::loads_per_thread();
    stage.a0.wait_for_dma_start_direct();
    dma.template issue_direct<STORE_LDS_DIRECT_SWIZZLE>(src, lds);
    stage.a1.wait_for_dma_start_direct();
    dma.template issue_direct<STORE_LDS_DIRECT_SWIZZLE>(src + step, lds + kStageBytes);
    auto land = [&](auto cur, auto nxt2, const int t) __attribute__((always_inline)) {
      if (t + 1 < ksteps) hipdma::wait_direct_loads<kLoads>(); else hipdma::wait_direct_loads<0>();
      stage.template get<decltype(cur)::value>().finish_async_dma_direct();
      if (t + 2 < ksteps) {
        stage.template get<decltype(nxt2)::value>().wait_for_dma_start_direct();
        dma.template issue_direct<STORE_LDS_DIRECT_SWIZZLE>(src + (size_t)(t + 2) * step, lds + decltype(nxt2)::value * kStageBytes);
      }
    };
    typedef std::integral_constant<int, 0> s0;
    typedef std::integral_constant<int, 1> s1;
    typedef std::integral_constant<int, 2> s2;
    for (int t = 0; t < ksteps; t += 3) {
      land(s0(), s2(), t);
      if (t + 1 < ksteps) land(s1(), s0(), t + 1);
      if (t + 2 < ksteps) land(s2(), s1(), t + 2);
    }
  };
  if (dma_a.owns_this_thread()) {
    feed(dma_a, &lds_a[0][0], std::integral_constant<int, kAStage>(), a + (size_t)tile_m * kBM * k, (size_t)kBK);
  } else if (dma_b.owns_this_thread()) {
    feed(dma_b, &lds_b[0][0], std::integral_constant<int, kBStage>(), b + (size_t)tile_n * kBN, (size_t)kBK * n);
  } else {
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int wm = (wave >> 1) * 32 * WI, wn = (wave & 1) * 32 * WJ;
    f32x16_t acc[WI][WJ];
#pragma unroll
    for (int i = 0; i < WI; ++i)
#pragma unroll
      for (int j = 0; j < WJ; ++j)
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.0f;
    stage.a0.start_async_dma();
    stage.a1.start_async_dma();
    stage.a2.start_async_dma();
    // A fragment of slice ks: row wm + 32*i + lane%32, chunk 2*ks + lane/32 of the 8 chunks of the row,
    // found at chunk position (2*ks + lane/32) ^ key(row); the key only depends on lane%32 here.
    int a_lane[kBK / 16];
    {
      const int row = wm + (lane & 31);
#pragma unroll
      for (int ks = 0; ks < kBK / 16; ++ks)
        a_lane[ks] = row * kARow + hipdma::swizzled_chunk(row, 2 * ks + (lane >> 5), kARow / 16) * 16;
    }
    // B fragment through the transposing read: inside a group of 16 lanes, lane j points at row (j/4) of a
    // 4-row block and at column 4*(j%4); the rows of the "lo" and "hi" reads are 4 apart.  Adding 16 rows
    // (the next slice) does not change a row's key.
    int b_lo[WJ], b_hi[WJ];
    {
      const int j16 = lane & 15;
      const int row = (lane >> 5) * 8 + (j16 >> 2);
#pragma unroll
      for (int j = 0; j < WJ; ++j) {
        const int col_bytes = (wn + j * 32 + ((lane >> 4) & 1) * 16 + (j16 & 3) * 4) * 2;
        b_lo[j] = row * kBRow + hipdma::swizzled_chunk(row, col_bytes >> 4, kBRow / 16) * 16 + (col_bytes & 15);
        b_hi[j] = (row + 4) * kBRow + hipdma::swizzled_chunk(row + 4, col_bytes >> 4, kBRow / 16) * 16 + (col_bytes & 15);
      }
    }
    auto load_frags = [&](bf16x8_t (&fa)[WI], bf16x8_t (&fb)[WJ], const char* sa, const char* sb, const int ks)
        __attribute__((always_inline)) {
#pragma unroll
      for (int i = 0; i < WI; ++i)
        fa[i] = *(const bf16x8_t*)(sa + i * 32 * kARow + a_lane[ks]);
#pragma unroll
      for (int j = 0; j < WJ; ++j) {
        const bf16x4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4bf16(
            (__attribute__((address_space(3))) bf16x4_t*)(sb + ks * 16 * kBRow + b_lo[j]));
        const bf16x4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4bf16(
            (__attribute__((address_space(3))) bf16x4_t*)(sb + ks * 16 * kBRow + b_hi[j]));
        fb[j] = bf16x8_t{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
      }
    };
    auto multiply = [&](const bf16x8_t (&fa)[WI], const bf16x8_t (&fb)[WJ]) __attribute__((always_inline)) {
#pragma unroll
      for (int i = 0; i < WI; ++i)
#pragma unroll
        for (int j = 0; j < WJ; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[i], fb[j], acc[i][j], 0, 0, 0);
      pin_slice<0, WI * WJ, WI + 2 * WJ>();
      __builtin_amdgcn_sched_barrier(0);
    };
    bf16x8_t fa0[WI], fb0[WJ], fa1[WI], fb1[WJ];
    // One stage: on entry fa0/fb0 hold its slice 0; on exit they hold slice 0 of the next stage.
    auto k_stage = [&](const cudaDMACustom& cur, const cudaDMACustom& nxt, const int s, const int sn, const bool has_next)
        __attribute__((always_inline)) {
      const char* sa = lds_a[s]; const char* sb = lds_b[s];
      load_frags(fa1, fb1, sa, sb, 1); multiply(fa0, fb0);
      load_frags(fa0, fb0, sa, sb, 2); multiply(fa1, fb1);
      const unsigned seen = nxt.peek_dma_finish();
      load_frags(fa1, fb1, sa, sb, 3); multiply(fa0, fb0);
      if (has_next) {
        nxt.wait_for_dma_finish(seen);
        load_frags(fa0, fb0, lds_a[sn], lds_b[sn], 0);
      }
      multiply(fa1, fb1);
      cur.start_async_dma();
    };
    stage.a0.wait_for_dma_finish();
    load_frags(fa0, fb0, lds_a[0], lds_b[0], 0);
    for (int kt = 0; kt < ksteps; kt += 3) {
      k_stage(stage.a0, stage.a1, 0, 1, kt + 1 < ksteps);
      if (kt + 1 < ksteps) k_stage(stage.a1, stage.a2, 1, 2, kt + 2 < ksteps);
      if (kt + 2 < ksteps) k_stage(stage.a2, stage.a0, 2, 0, kt + 3 < ksteps);
    }
    float* cbase = c + (size_t)(tile_m * kBM + wm) * n + (size_t)tile_n * kBN + wn;
#pragma unroll
    for (int i = 0; i < WI; ++i)
#pragma unroll
      for (int j = 0; j < WJ; ++j)
#pragma unroll
        for (int e = 0; e < 16; ++e) {
          const int row = i * 32 + 8 * (e / 4) + 4 * (lane >> 5) + (e % 4);
          const int col = j * 32 + (lane & 31);
          __builtin_nontemporal_store(acc[i][j][e], &cbase[(size_t)row * n + col]);
        }
  }
}
#endif  // HIPDMA_SWEEP_VARIANTS

// ---- 256 x 256 tile, K step 32, four unpadded swizzled stages filled by global_load_lds_dwordx4 ----
// Eight compute wavefronts (2 x 4, 128 x 64 each, two per SIMD) and four DMA wavefronts.  A stage is
// 32 KB (A: 256 rows x 64 B, B: 32 rows x 512 B); each DMA wavefront keeps three transfers in flight.
template<typename T>
struct Four4 {
  T a0, a1, a2, a3;
  template<int I> __device__ __forceinline__ T& get() { if constexpr (I == 0) return a0; else if constexpr (I == 1) return a1; else if constexpr (I == 2) return a2; else return a3; }
};

constexpr int kDirect4DmaThreads = 128;    // DMA threads per operand
constexpr int kDirect4Ahead = 3;           // transfers in flight per DMA wavefront (2: 3 % slower; 4 stages allow no more)
#ifdef HIPDMA_SWEEP_VARIANTS
__global__ void __launch_bounds__(512 + 2 * kDirect4DmaThreads)
gemm_bf16_ws_direct4(const unsigned short* __restrict__ a, const unsigned short* __restrict__ b, float* __restrict__ c,
                     const int m, const int n, const int k)
{
  constexpr int WI = 4, WJ = 2, WN = 4, kStages = 4, kBK4 = 32, kCompute = 512, kDmaWave = kDirect4DmaThreads;
  constexpr int kBM = 256, kBN = 256;
  constexpr int kARow = kBK4 * 2, kBRow = kBN * 2;                 // 64 B and 512 B, unpadded
  constexpr int kAStage = kBM * kARow, kBStage = kBK4 * kBRow;     // 16 KB and 16 KB
  typedef CudaDMAStrided<false, 16, 16, kARow, kDmaWave, kBM> dma_a_t;
  typedef CudaDMAStrided<false, 16, 16, kBRow, kDmaWave, kBK4> dma_b_t;
  __shared__ __attribute__((aligned(1024))) char lds_a[kStages][kAStage];
  __shared__ __attribute__((aligned(1024))) char lds_b[kStages][kBStage];
  dma_a_t dma_a(k * 2, kARow, kCompute);
  dma_b_t dma_b(n * 2, kBRow, kCompute + kDmaWave);
  Four4<cudaDMACustom> stage{cudaDMACustom(0, 2 * kDmaWave, kCompute, kCompute), cudaDMACustom(1, 2 * kDmaWave, kCompute, kCompute),
                             cudaDMACustom(2, 2 * kDmaWave, kCompute, kCompute), cudaDMACustom(3, 2 * kDmaWave, kCompute, kCompute)};
  int tile_m, tile_n;
  tile_of_workgroup(blockIdx.x, m / kBM, n / kBN, tile_m, tile_n);
  const int ksteps = k / kBK4;            // a multiple of four: k is a multiple of 128

  // One DMA wavefront: tile t lands in stage t % 4; tiles t+1 .. t+3 are in flight while the compute
  // wavefronts work on tile t.
  auto feed = [&](auto& dma, char* lds, auto stage_bytes, const unsigned short* src, const size_t step)
      __attribute__((always_inline)) {
    constexpr int kStageBytes = decltype(stage_bytes)::value;
    constexpr int kLoads = std::remove_reference<decltype(dma)>::type::loads_per_thread();
    constexpr int kAhead = kDirect4Ahead;       // transfers in flight per DMA wavefront
    stage.a0.wait_for_dma_start_direct();
    dma.template issue_direct<STORE_LDS_DIRECT_SWIZZLE>(src, lds);
    if constexpr (kAhead > 1) {
      stage.a1.wait_for_dma_start_direct();
      dma.template issue_direct<STORE_LDS_DIRECT_SWIZZLE>(src + step, lds + kStageBytes);
    }
    if constexpr (kAhead > 2) {
      stage.a2.wait_for_dma_start_direct();
      dma.template issue_direct<STORE_LDS_DIRECT_SWIZZLE>(src + 2 * step, lds + 2 * kStageBytes);
    }
    auto land = [&](auto cur, const int t) __attribute__((always_inline)) {
      constexpr int kCur = decltype(cur)::value, kNext = (kCur + kAhead) % kStages;
      // the younger transfers stay in flight (fewer at the end)
      if (t + kAhead - 1 < ksteps) hipdma::wait_direct_loads<(kAhead - 1) * kLoads>();
      else if (kAhead > 2 && t + 1 < ksteps) hipdma::wait_direct_loads<kLoads>();
      else hipdma::wait_direct_loads<0>();
      stage.template get<kCur>().finish_async_dma_direct();
      if (t + kAhead < ksteps) {
        stage.template get<kNext>().wait_for_dma_start_direct();
        dma.template issue_direct<STORE_LDS_DIRECT_SWIZZLE>(src + (size_t)(t + kAhead) * step, lds + kNext * kStageBytes);
      }
    };
    typedef std::integral_constant<int, 0> s0;
    typedef std::integral_constant<int, 1> s1;
    typedef std::integral_constant<int, 2> s2;
    typedef std::integral_constant<int, 3> s3;
    for (int t = 0; t < ksteps; t += 4) {
      land(s0(), t);
      land(s1(), t + 1);
      land(s2(), t + 2);
      land(s3(), t + 3);
    }
  };
  if (dma_a.owns_this_thread()) {
    feed(dma_a, &lds_a[0][0], std::integral_constant<int, kAStage>(), a + (size_t)tile_m * kBM * k, (size_t)kBK4);
  } else if (dma_b.owns_this_thread()) {
    feed(dma_b, &lds_b[0][0], std::integral_constant<int, kBStage>(), b + (size_t)tile_n * kBN, (size_t)kBK4 * n);
  } else {
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int wm = (wave / WN) * 32 * WI, wn = (wave % WN) * 32 * WJ;
    f32x16_t acc[WI][WJ];
#pragma unroll
    for (int i = 0; i < WI; ++i)
#pragma unroll
      for (int j = 0; j < WJ; ++j)
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.0f;
    stage.a0.start_async_dma();
    stage.a1.start_async_dma();
    stage.a2.start_async_dma();
    stage.a3.start_async_dma();
    // A fragment of slice ks: row wm + 32*i + lane%32, chunk 2*ks + lane/32 of the 4 chunks of the row, found at
    // chunk position (2*ks + lane/32) ^ key(row); the key only depends on lane%32 (wm and 32*i are multiples of 32).
    int a_lane[kBK4 / 16];
    {
      const int row = wm + (lane & 31);
#pragma unroll
      for (int ks = 0; ks < kBK4 / 16; ++ks)
        a_lane[ks] = row * kARow + hipdma::swizzled_chunk(row, 2 * ks + (lane >> 5), kARow / 16) * 16;
    }
    // B fragment through the transposing read; adding 16 rows (the next slice) does not change a row's key.
    int b_lo[WJ], b_hi[WJ];
    {
      const int j16 = lane & 15;
      const int row = (lane >> 5) * 8 + (j16 >> 2);
#pragma unroll
      for (int j = 0; j < WJ; ++j) {
        const int col_bytes = (wn + j * 32 + ((lane >> 4) & 1) * 16 + (j16 & 3) * 4) * 2;
        b_lo[j] = row * kBRow + hipdma::swizzled_chunk(row, col_bytes >> 4, kBRow / 16) * 16 + (col_bytes & 15);
        b_hi[j] = (row + 4) * kBRow + hipdma::swizzled_chunk(row + 4, col_bytes >> 4, kBRow / 16) * 16 + (col_bytes & 15);
      }
    }
    auto k_stage = [&](const cudaDMACustom& cur, const int s) __attribute__((always_inline)) {
      const char* sa = lds_a[s]; const char* sb = lds_b[s];
      cur.wait_for_dma_finish();
#pragma unroll
      for (int ks = 0; ks < kBK4 / 16; ++ks) {
        bf16x8_t fa[WI], fb[WJ];
#pragma unroll
        for (int i = 0; i < WI; ++i) fa[i] = *(const bf16x8_t*)(sa + i * 32 * kARow + a_lane[ks]);
#pragma unroll
        for (int j = 0; j < WJ; ++j) {
          const bf16x4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4bf16(
              (__attribute__((address_space(3))) bf16x4_t*)(sb + ks * 16 * kBRow + b_lo[j]));
          const bf16x4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4bf16(
              (__attribute__((address_space(3))) bf16x4_t*)(sb + ks * 16 * kBRow + b_hi[j]));
          fb[j] = bf16x8_t{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
        }
#pragma unroll
        for (int i = 0; i < WI; ++i)
#pragma unroll
          for (int j = 0; j < WJ; ++j)
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[i], fb[j], acc[i][j], 0, 0, 0);
      }
      cur.start_async_dma();
    };
    for (int kt = 0; kt < ksteps; kt += 4) {
      k_stage(stage.a0, 0);
      k_stage(stage.a1, 1);
      k_stage(stage.a2, 2);
      k_stage(stage.a3, 3);
    }
    float* cbase = c + (size_t)(tile_m * kBM + wm) * n + (size_t)tile_n * kBN + wn;
#pragma unroll
    for (int i = 0; i < WI; ++i)
#pragma unroll
      for (int j = 0; j < WJ; ++j)
#pragma unroll
        for (int e = 0; e < 16; ++e) {
          const int row = i * 32 + 8 * (e / 4) + 4 * (lane >> 5) + (e % 4);
          const int col = j * 32 + (lane & 31);
          __builtin_nontemporal_store(acc[i][j][e], &cbase[(size_t)row * n + col]);
        }
  }
}
#endif  // HIPDMA_SWEEP_VARIANTS

// ---- the same kernel with A rows of 128 B: an A transfer covers two K steps ----
// A K step of 32 takes 64 B of every A row, half a cache line: the L1 fetches each line of the A
// panel twice, a step apart, and the compute wavefronts wait for the DMA wavefronts (measured with
// s_memtime stamps: 900 of 2350 cycles per step).  Here an A transfer brings 256 rows x 128 B
// (two K steps, whole lines) into one of two 32 KB buffers with its own guard; B keeps the four
// 16 KB stages of one K step each.  The compute wavefronts wait for a B stage every step and for
// an A buffer every other step.
__global__ void __launch_bounds__(512 + 2 * kDirect4DmaThreads)
gemm_bf16_ws_direct4_a64(const unsigned short* __restrict__ a, const unsigned short* __restrict__ b, float* __restrict__ c,
                         const int m, const int n, const int k)
{
  constexpr int WI = 4, WJ = 2, WN = 4, kBStages = 4, kBK4 = 32, kCompute = 512, kDmaWave = kDirect4DmaThreads;
  constexpr int kBM = 256, kBN = 256;
  constexpr int kARow = 4 * kBK4, kBRow = kBN * 2;                 // 128 B (two K steps) and 512 B, unpadded
  constexpr int kABuf = kBM * kARow, kBStage = kBK4 * kBRow;       // 32 KB and 16 KB
  typedef CudaDMAStrided<false, 16, 16, kARow, kDmaWave, kBM> dma_a_t;
  typedef CudaDMAStrided<false, 16, 16, kBRow, kDmaWave, kBK4> dma_b_t;
  __shared__ __attribute__((aligned(1024))) char lds_a[2][kABuf];
  __shared__ __attribute__((aligned(1024))) char lds_b[kBStages][kBStage];
  dma_a_t dma_a(k * 2, kARow, kCompute);
  dma_b_t dma_b(n * 2, kBRow, kCompute + kDmaWave);
  Four4<cudaDMACustom> gb{cudaDMACustom(0, kDmaWave, kCompute, kCompute + kDmaWave), cudaDMACustom(1, kDmaWave, kCompute, kCompute + kDmaWave),
                          cudaDMACustom(2, kDmaWave, kCompute, kCompute + kDmaWave), cudaDMACustom(3, kDmaWave, kCompute, kCompute + kDmaWave)};
  cudaDMACustom ga0(4, kDmaWave, kCompute, kCompute);
  cudaDMACustom ga1(5, kDmaWave, kCompute, kCompute);
  int tile_m, tile_n;
  tile_of_workgroup(blockIdx.x, m / kBM, n / kBN, tile_m, tile_n);
  const int ksteps = k / kBK4;            // a multiple of four: k is a multiple of 128

  if (dma_a.owns_this_thread()) {
    // Transfer p (K steps 2p and 2p+1) lands in buffer p % 2; transfer p+1 is requested as soon as
    // p has landed (its buffer was released when the compute wavefronts left transfer p-1).
    const unsigned short* src = a + (size_t)tile_m * kBM * k;
    const int transfers = ksteps / 2;     // even
    ga0.wait_for_dma_start_direct();
    dma_a.template issue_direct<STORE_LDS_DIRECT_SWIZZLE>(src, lds_a[0]);
    for (int p = 0; p < transfers; p += 2) {
      hipdma::wait_direct_loads<0>();
      ga0.finish_async_dma_direct();
      ga1.wait_for_dma_start_direct();
      dma_a.template issue_direct<STORE_LDS_DIRECT_SWIZZLE>(src + (size_t)(p + 1) * (2 * kBK4), lds_a[1]);
      hipdma::wait_direct_loads<0>();
      ga1.finish_async_dma_direct();
      if (p + 2 < transfers) {
        ga0.wait_for_dma_start_direct();
        dma_a.template issue_direct<STORE_LDS_DIRECT_SWIZZLE>(src + (size_t)(p + 2) * (2 * kBK4), lds_a[0]);
      }
    }
  } else if (dma_b.owns_this_thread()) {
    // Tile t lands in stage t % 4; tiles t+1 .. t+3 are in flight while the compute wavefronts work on tile t.
    const unsigned short* src = b + (size_t)tile_n * kBN;
    const size_t step = (size_t)kBK4 * n;
    constexpr int kLoads = dma_b_t::loads_per_thread();
    constexpr int kAhead = kDirect4Ahead;
    gb.a0.wait_for_dma_start_direct();
    dma_b.template issue_direct<STORE_LDS_DIRECT_SWIZZLE>(src, lds_b[0]);
    gb.a1.wait_for_dma_start_direct();
    dma_b.template issue_direct<STORE_LDS_DIRECT_SWIZZLE>(src + step, lds_b[1]);
    gb.a2.wait_for_dma_start_direct();
    dma_b.template issue_direct<STORE_LDS_DIRECT_SWIZZLE>(src + 2 * step, lds_b[2]);
    auto land = [&](auto cur, const int t) __attribute__((always_inline)) {
      constexpr int kCur = decltype(cur)::value, kNext = (kCur + kAhead) % kBStages;
      if (t + kAhead - 1 < ksteps) hipdma::wait_direct_loads<(kAhead - 1) * kLoads>();
      else if (t + 1 < ksteps) hipdma::wait_direct_loads<kLoads>();
      else hipdma::wait_direct_loads<0>();
      gb.template get<kCur>().finish_async_dma_direct();
      if (t + kAhead < ksteps) {
        gb.template get<kNext>().wait_for_dma_start_direct();
        dma_b.template issue_direct<STORE_LDS_DIRECT_SWIZZLE>(src + (size_t)(t + kAhead) * step, lds_b[kNext]);
      }
    };
    for (int t = 0; t < ksteps; t += 4) {
      land(std::integral_constant<int, 0>(), t);
      land(std::integral_constant<int, 1>(), t + 1);
      land(std::integral_constant<int, 2>(), t + 2);
      land(std::integral_constant<int, 3>(), t + 3);
    }
  } else {
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int wm = (wave / WN) * 32 * WI, wn = (wave % WN) * 32 * WJ;
    f32x16_t acc[WI][WJ];
#pragma unroll
    for (int i = 0; i < WI; ++i)
#pragma unroll
      for (int j = 0; j < WJ; ++j)
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.0f;
    gb.a0.start_async_dma();
    gb.a1.start_async_dma();
    gb.a2.start_async_dma();
    gb.a3.start_async_dma();
    ga0.start_async_dma();
    ga1.start_async_dma();
    // A fragment of slice ks (0..3 inside a buffer): row wm + 32*i + lane%32, chunk 2*ks + lane/32 of the 8 chunks
    // of the row, found at chunk position (2*ks + lane/32) ^ key(row); the key only depends on lane%32.
    int a_lane[4];
    {
      const int row = wm + (lane & 31);
#pragma unroll
      for (int ks = 0; ks < 4; ++ks)
        a_lane[ks] = row * kARow + hipdma::swizzled_chunk(row, 2 * ks + (lane >> 5), kARow / 16) * 16;
    }
    // B fragment through the transposing read; adding 16 rows (the next slice) does not change a row's key.
    int b_lo[WJ], b_hi[WJ];
    {
      const int j16 = lane & 15;
      const int row = (lane >> 5) * 8 + (j16 >> 2);
#pragma unroll
      for (int j = 0; j < WJ; ++j) {
        const int col_bytes = (wn + j * 32 + ((lane >> 4) & 1) * 16 + (j16 & 3) * 4) * 2;
        b_lo[j] = row * kBRow + hipdma::swizzled_chunk(row, col_bytes >> 4, kBRow / 16) * 16 + (col_bytes & 15);
        b_hi[j] = (row + 4) * kBRow + hipdma::swizzled_chunk(row + 4, col_bytes >> 4, kBRow / 16) * 16 + (col_bytes & 15);
      }
    }
    // One K step: B stage s, slices 2*half and 2*half+1 of A buffer `abuf`.
    auto k_step = [&](const cudaDMACustom& gbs, const int s, const cudaDMACustom& gas, const int abuf, auto half)
        __attribute__((always_inline)) {
      constexpr int kHalf = decltype(half)::value;
      const char* sa = lds_a[abuf]; const char* sb = lds_b[s];
      if constexpr (kHalf == 0) gas.wait_for_dma_finish();
      gbs.wait_for_dma_finish();
#pragma unroll
      for (int ks = 0; ks < kBK4 / 16; ++ks) {
        bf16x8_t fa[WI], fb[WJ];
#pragma unroll
        for (int i = 0; i < WI; ++i) fa[i] = *(const bf16x8_t*)(sa + i * 32 * kARow + a_lane[2 * kHalf + ks]);
#pragma unroll
        for (int j = 0; j < WJ; ++j) {
          const bf16x4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4bf16(
              (__attribute__((address_space(3))) bf16x4_t*)(sb + ks * 16 * kBRow + b_lo[j]));
          const bf16x4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4bf16(
              (__attribute__((address_space(3))) bf16x4_t*)(sb + ks * 16 * kBRow + b_hi[j]));
          fb[j] = bf16x8_t{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
        }
#pragma unroll
        for (int i = 0; i < WI; ++i)
#pragma unroll
          for (int j = 0; j < WJ; ++j)
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[i], fb[j], acc[i][j], 0, 0, 0);
      }
      gbs.start_async_dma();
      if constexpr (kHalf == 1) gas.start_async_dma();
    };
    typedef std::integral_constant<int, 0> h0;
    typedef std::integral_constant<int, 1> h1;
    for (int kt = 0; kt < ksteps; kt += 4) {
      k_step(gb.a0, 0, ga0, 0, h0());
      k_step(gb.a1, 1, ga0, 0, h1());
      k_step(gb.a2, 2, ga1, 1, h0());
      k_step(gb.a3, 3, ga1, 1, h1());
    }
    float* cbase = c + (size_t)(tile_m * kBM + wm) * n + (size_t)tile_n * kBN + wn;
#pragma unroll
    for (int i = 0; i < WI; ++i)
#pragma unroll
      for (int j = 0; j < WJ; ++j)
#pragma unroll
        for (int e = 0; e < 16; ++e) {
          const int row = i * 32 + 8 * (e / 4) + 4 * (lane >> 5) + (e % 4);
          const int col = j * 32 + (lane & 31);
          __builtin_nontemporal_store(acc[i][j][e], &cbase[(size_t)row * n + col]);
        }
  }
}

// ---- 256 x 256 tile without warp specialisation: four wavefronts that each fetch and multiply ----
// The objects are the form of CudaDMAStrided that is not warp-specialised (all 256 threads issue their
// share of a stage with issue_direct; src/examples/stencil/non_warp_specialized_single_buffer.h:47-57 is
// the reference's use of that form).  A wavefront owns a SIMD and a 128 x 128 block of C: 256 accumulator
// registers, 0.5 KB of fragments read per matrix instruction instead of 0.75, no DMA wavefronts to share the
// register file with.  Four stages of one K step (32); a K step starts with one s_barrier: by then every
// wavefront has waited for its own loads of the next stage, so that stage is complete, and every wavefront has
// left the previous stage, so that buffer takes the loads of the stage three steps on.  Those eight loads per
// thread are issued one at a time between groups of four products (issued back to back they hold the wavefront,
// and with it its matrix core, for 550 cycles: the address unit takes one 16-byte load of a wavefront per
// sixteen cycles); the fragments of the next slice, in the second half those of the next stage, are requested
// under the products of the current one.
#ifdef HIPDMA_SWEEP_VARIANTS
__global__ void __launch_bounds__(256)
gemm_bf16_all_direct(const unsigned short* __restrict__ a, const unsigned short* __restrict__ b, float* __restrict__ c,
                     const int m, const int n, const int k)
{
  constexpr int WI = 4, WJ = 4, kStages = 4, kBK4 = 32, kThreads = 256;
  constexpr int kBM = 256, kBN = 256;
  constexpr int kARow = kBK4 * 2, kBRow = kBN * 2;                 // 64 B and 512 B, unpadded
  constexpr int kAStage = kBM * kARow, kBStage = kBK4 * kBRow;     // 16 KB and 16 KB
  typedef CudaDMAStrided<false, 16, 16, kARow, kThreads, kBM> dma_a_t;
  typedef CudaDMAStrided<false, 16, 16, kBRow, kThreads, kBK4> dma_b_t;
  constexpr int kLoads = dma_a_t::loads_per_thread() + dma_b_t::loads_per_thread();     // per stage and thread
  __shared__ __attribute__((aligned(1024))) char lds_a[kStages][kAStage];
  __shared__ __attribute__((aligned(1024))) char lds_b[kStages][kBStage];
  dma_a_t dma_a(k * 2, kARow);
  dma_b_t dma_b(n * 2, kBRow);
  int tile_m, tile_n;
  tile_of_workgroup(blockIdx.x, m / kBM, n / kBN, tile_m, tile_n);
  const int ksteps = k / kBK4;            // a multiple of four
  const int klast = ksteps - 1;
  const unsigned short* const src_a = a + (size_t)tile_m * kBM * k;
  const unsigned short* const src_b = b + (size_t)tile_n * kBN;
  const size_t step_b = (size_t)kBK4 * n;
  // Stage t of the K loop into buffer t % 4: round g of the A loads (g < 4) or round g - 4 of the B loads.  Past
  // the end the last stage is requested again (into a buffer nobody reads any more): the loop keeps one shape and
  // one wait count.
  static_assert(dma_a_t::loads_per_thread() == 4 && dma_b_t::loads_per_thread() == 4, "eight loads per thread and stage");
  auto issue = [&](const int t, const int buf, const int g) __attribute__((always_inline)) {
    const int tt = t < klast ? t : klast;
    if (g < 4) dma_a.template issue_direct_part<STORE_LDS_DIRECT_SWIZZLE, true>(src_a + (size_t)tt * kBK4, lds_a[buf], g, 1);
    else dma_b.template issue_direct_part<STORE_LDS_DIRECT_SWIZZLE, true>(src_b + (size_t)tt * step_b, lds_b[buf], g - 4, 1);
  };
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int wm = (wave >> 1) * 32 * WI, wn = (wave & 1) * 32 * WJ;
  f32x16_t acc[WI][WJ];
#pragma unroll
  for (int i = 0; i < WI; ++i)
#pragma unroll
    for (int j = 0; j < WJ; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.0f;
  int a_lane[kBK4 / 16];
  {
    const int row = wm + (lane & 31);
#pragma unroll
    for (int ks = 0; ks < kBK4 / 16; ++ks)
      a_lane[ks] = row * kARow + hipdma::swizzled_chunk(row, 2 * ks + (lane >> 5), kARow / 16) * 16;
  }
  int b_lo[WJ], b_hi[WJ];
  {
    const int j16 = lane & 15;
    const int row = (lane >> 5) * 8 + (j16 >> 2);
#pragma unroll
    for (int j = 0; j < WJ; ++j) {
      const int col_bytes = (wn + j * 32 + ((lane >> 4) & 1) * 16 + (j16 & 3) * 4) * 2;
      b_lo[j] = row * kBRow + hipdma::swizzled_chunk(row, col_bytes >> 4, kBRow / 16) * 16 + (col_bytes & 15);
      b_hi[j] = (row + 4) * kBRow + hipdma::swizzled_chunk(row + 4, col_bytes >> 4, kBRow / 16) * 16 + (col_bytes & 15);
    }
  }
  auto load_frags = [&](bf16x8_t (&fa)[WI], bf16x8_t (&fb)[WJ], const int buf, const int ks) __attribute__((always_inline)) {
    const char* sa = lds_a[buf]; const char* sb = lds_b[buf];
#pragma unroll
    for (int i = 0; i < WI; ++i) fa[i] = *(const bf16x8_t*)(sa + i * 32 * kARow + a_lane[ks]);
#pragma unroll
    for (int j = 0; j < WJ; ++j) {
      const bf16x4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4bf16(
          (__attribute__((address_space(3))) bf16x4_t*)(sb + ks * 16 * kBRow + b_lo[j]));
      const bf16x4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4bf16(
          (__attribute__((address_space(3))) bf16x4_t*)(sb + ks * 16 * kBRow + b_hi[j]));
      fb[j] = bf16x8_t{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
    }
  };
  // Half a K step: the sixteen products of the slice in (fa, fb) in four groups of four.  Under the first three
  // groups the fragments of the slice (nbuf, nks) are requested into (na, nb): the four A blocks, then two B blocks
  // twice.  Behind every group goes one load of stage t + 3.  Nothing moves across the ends of a group.
  auto half_step = [&](const bf16x8_t (&fa)[WI], const bf16x8_t (&fb)[WJ], bf16x8_t (&na)[WI], bf16x8_t (&nb)[WJ],
                       const int nbuf, const int nks, const int t, const int buf, const int first_load)
      __attribute__((always_inline)) {
    const char* sa = lds_a[nbuf]; const char* sb = lds_b[nbuf];
#pragma unroll
    for (int i = 0; i < WI; ++i) {
      if (i == 0) {
#pragma unroll
        for (int q = 0; q < WI; ++q) na[q] = *(const bf16x8_t*)(sa + q * 32 * kARow + a_lane[nks]);
      } else if (i < 3) {
#pragma unroll
        for (int j = 2 * (i - 1); j < 2 * i; ++j) {
          const bf16x4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4bf16(
              (__attribute__((address_space(3))) bf16x4_t*)(sb + nks * 16 * kBRow + b_lo[j]));
          const bf16x4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4bf16(
              (__attribute__((address_space(3))) bf16x4_t*)(sb + nks * 16 * kBRow + b_hi[j]));
          nb[j] = bf16x8_t{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
        }
      }
#pragma unroll
      for (int j = 0; j < WJ; ++j)
        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[i], fb[j], acc[i][j], 0, 0, 0);
      // product, request, product, request, ...
#pragma unroll
      for (int q = 0; q < WJ; ++q) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        if (i < 3) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
      }
      __builtin_amdgcn_sched_barrier(0);
      issue(t + 3, (buf + 3) % kStages, first_load + i);
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  bf16x8_t fa0[WI], fb0[WJ], fa1[WI], fb1[WJ];
#pragma unroll
  for (int g = 0; g < 8; ++g) issue(0, 0, g);
#pragma unroll
  for (int g = 0; g < 8; ++g) issue(1, 1, g);
#pragma unroll
  for (int g = 0; g < 8; ++g) issue(2, 2, g);
  hipdma::wait_direct_loads<2 * kLoads>();
  __builtin_amdgcn_s_barrier();
  load_frags(fa0, fb0, 0, 0);
  // One K step on buffer `buf`: on entry fa0/fb0 hold its first slice and stages t + 1, t + 2 are in flight; on
  // exit fa0/fb0 hold the first slice of the next step.
  auto k_step = [&](const int t, const int buf) __attribute__((always_inline)) {
    hipdma::wait_direct_loads<kLoads>();          // this thread's part of stage t + 1 (stage t + 2 stays in flight)
    __builtin_amdgcn_s_barrier();
    half_step(fa0, fb0, fa1, fb1, buf, 1, t, buf, 0);
    half_step(fa1, fb1, fa0, fb0, (buf + 1) % kStages, 0, t, buf, 4);
  };
  for (int kt = 0; kt < ksteps; kt += 4) {
    k_step(kt, 0);
    k_step(kt + 1, 1);
    k_step(kt + 2, 2);
    k_step(kt + 3, 3);
  }
  hipdma::wait_direct_loads<0>();
  float* cbase = c + (size_t)(tile_m * kBM + wm) * n + (size_t)tile_n * kBN + wn;
#pragma unroll
  for (int i = 0; i < WI; ++i)
#pragma unroll
    for (int j = 0; j < WJ; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        const int row = i * 32 + 8 * (e / 4) + 4 * (lane >> 5) + (e % 4);
        const int col = j * 32 + (lane & 31);
        __builtin_nontemporal_store(acc[i][j][e], &cbase[(size_t)row * n + col]);
      }
}
#endif  // HIPDMA_SWEEP_VARIANTS

// ---- the same kernel with A transfers of two K steps (rows of 128 B) ----
// A K step of 32 takes 64 B of an A row, half a cache line, and the L1 asks the L2 for every line of the A panel
// twice (TCP_TCC_READ_REQ: 12.8 M requests per 4096^3 launch instead of 8.4 M).  Here an A transfer is 256 rows x
// 128 B for two K steps.  Three A buffers (96 KB) and the four B stages (64 KB) are all of the LDS: an A buffer is
// free two K steps after its last read and its next transfer has to be complete a step before its first, so two
// buffers would leave it one K step to land.  The A buffers form a ring indexed at run time (three does not divide
// the K steps of every problem); a K step still issues eight loads, four of B and half an A transfer.
__global__ void __launch_bounds__(256)
gemm_bf16_all_direct_a64(const unsigned short* __restrict__ a, const unsigned short* __restrict__ b, float* __restrict__ c,
                         const int m, const int n, const int k)
{
  constexpr int WI = 4, WJ = 4, kBStages = 4, kABufs = 3, kBK4 = 32, kThreads = 256;
  constexpr int kBM = 256, kBN = 256;
  constexpr int kARow = 4 * kBK4, kBRow = kBN * 2;                 // 128 B (two K steps) and 512 B, unpadded
  constexpr int kABuf = kBM * kARow, kBStage = kBK4 * kBRow;       // 32 KB and 16 KB
  typedef CudaDMAStrided<false, 16, 16, kARow, kThreads, kBM> dma_a_t;
  typedef CudaDMAStrided<false, 16, 16, kBRow, kThreads, kBK4> dma_b_t;
  static_assert(dma_a_t::loads_per_thread() == 8 && dma_b_t::loads_per_thread() == 4, "eight loads per thread and K step");
  constexpr int kLoads = 8;
  __shared__ __attribute__((aligned(1024))) char lds_a[kABufs * kABuf];
  __shared__ __attribute__((aligned(1024))) char lds_b[kBStages][kBStage];
  dma_a_t dma_a(k * 2, kARow);
  dma_b_t dma_b(n * 2, kBRow);
  int tile_m, tile_n;
  tile_of_workgroup(blockIdx.x, m / kBM, n / kBN, tile_m, tile_n);
  const int ksteps = k / kBK4;            // a multiple of four
  const int klast = ksteps - 1, dlast = ksteps / 2 - 1;
  const unsigned short* const src_a = a + (size_t)tile_m * kBM * k;
  const unsigned short* const src_b = b + (size_t)tile_n * kBN;
  const size_t step_b = (size_t)kBK4 * n;
  // Round r of the B stage of K step t into B buffer `buf`; round r of A transfer d (K steps 2d, 2d+1) into A
  // buffer `buf`.  Past the end the last one is requested again, into a buffer nobody reads any more.
  auto issue_b = [&](const int t, const int buf, const int r) __attribute__((always_inline)) {
    const int tt = t < klast ? t : klast;
    dma_b.template issue_direct_part<STORE_LDS_DIRECT_SWIZZLE, true>(src_b + (size_t)tt * step_b, lds_b[buf], r, 1);
  };
  auto issue_a = [&](const int d, const int buf, const int r) __attribute__((always_inline)) {
    const int dd = d < dlast ? d : dlast;
    dma_a.template issue_direct_part<STORE_LDS_DIRECT_SWIZZLE, true>(src_a + (size_t)dd * (2 * kBK4), lds_a + buf * kABuf, r, 1);
  };
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int wm = (wave >> 1) * 32 * WI, wn = (wave & 1) * 32 * WJ;
  f32x16_t acc[WI][WJ];
#pragma unroll
  for (int i = 0; i < WI; ++i)
#pragma unroll
    for (int j = 0; j < WJ; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.0f;
  // A fragment of slice q (0..3 inside a buffer): row wm + 32*i + lane%32, chunk 2*q + lane/32 of the 8 chunks of the row
  int a_lane[4];
  {
    const int row = wm + (lane & 31);
#pragma unroll
    for (int q = 0; q < 4; ++q)
      a_lane[q] = row * kARow + hipdma::swizzled_chunk(row, 2 * q + (lane >> 5), kARow / 16) * 16;
  }
  int b_lo[WJ], b_hi[WJ];
  {
    const int j16 = lane & 15;
    const int row = (lane >> 5) * 8 + (j16 >> 2);
#pragma unroll
    for (int j = 0; j < WJ; ++j) {
      const int col_bytes = (wn + j * 32 + ((lane >> 4) & 1) * 16 + (j16 & 3) * 4) * 2;
      b_lo[j] = row * kBRow + hipdma::swizzled_chunk(row, col_bytes >> 4, kBRow / 16) * 16 + (col_bytes & 15);
      b_hi[j] = (row + 4) * kBRow + hipdma::swizzled_chunk(row + 4, col_bytes >> 4, kBRow / 16) * 16 + (col_bytes & 15);
    }
  }
  // Half a K step: sixteen products in four groups; under the first three the fragments of slice q of A buffer
  // `abuf` and of slice ks of B stage `bbuf` are requested into (na, nb); `after_group(i)` places the loads.
  auto half_step = [&](const bf16x8_t (&fa)[WI], const bf16x8_t (&fb)[WJ], bf16x8_t (&na)[WI], bf16x8_t (&nb)[WJ],
                       const int abuf, const int q, const int bbuf, const int ks, auto after_group)
      __attribute__((always_inline)) {
    const char* sa = lds_a + abuf * kABuf; const char* sb = lds_b[bbuf];
#pragma unroll
    for (int i = 0; i < WI; ++i) {
      if (i == 0) {
#pragma unroll
        for (int r = 0; r < WI; ++r) na[r] = *(const bf16x8_t*)(sa + r * 32 * kARow + a_lane[q]);
      } else if (i < 3) {
#pragma unroll
        for (int j = 2 * (i - 1); j < 2 * i; ++j) {
          const bf16x4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4bf16(
              (__attribute__((address_space(3))) bf16x4_t*)(sb + ks * 16 * kBRow + b_lo[j]));
          const bf16x4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4bf16(
              (__attribute__((address_space(3))) bf16x4_t*)(sb + ks * 16 * kBRow + b_hi[j]));
          nb[j] = bf16x8_t{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
        }
      }
#pragma unroll
      for (int j = 0; j < WJ; ++j)
        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[i], fb[j], acc[i][j], 0, 0, 0);
#pragma unroll
      for (int r = 0; r < WJ; ++r) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        if (i < 3) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
      }
      __builtin_amdgcn_sched_barrier(0);
      after_group(i);
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  bf16x8_t fa0[WI], fb0[WJ], fa1[WI], fb1[WJ];
  // Before the loop, in the order the loop's wait counts assume: (A transfer 0, B stage 0), then what K steps -2
  // and -1 would have issued: (B stage 1, first half of A transfer 1), (B stage 2, second half of A transfer 1).
#pragma unroll
  for (int r = 0; r < 8; ++r) issue_a(0, 0, r);
#pragma unroll
  for (int r = 0; r < 4; ++r) issue_b(0, 0, r);
#pragma unroll
  for (int r = 0; r < 4; ++r) issue_b(1, 1, r);
#pragma unroll
  for (int r = 0; r < 4; ++r) issue_a(1, 1, r);
#pragma unroll
  for (int r = 0; r < 4; ++r) issue_b(2, 2, r);
#pragma unroll
  for (int r = 4; r < 8; ++r) issue_a(1, 1, r);
  hipdma::wait_direct_loads<2 * kLoads>();
  __builtin_amdgcn_s_barrier();
  // first slice of K step 0
  {
#pragma unroll
    for (int r = 0; r < WI; ++r) fa0[r] = *(const bf16x8_t*)(lds_a + r * 32 * kARow + a_lane[0]);
#pragma unroll
    for (int j = 0; j < WJ; ++j) {
      const bf16x4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((__attribute__((address_space(3))) bf16x4_t*)(lds_b[0] + b_lo[j]));
      const bf16x4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((__attribute__((address_space(3))) bf16x4_t*)(lds_b[0] + b_hi[j]));
      fb0[j] = bf16x8_t{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
    }
  }
  // One K step t on B buffer bbuf and slices (2*h, 2*h+1) of A buffer abuf; the next step starts in A buffer nabuf
  // at slice nq.  It issues B stage t + 3 and rounds [ar, ar + 4) of A transfer ad into A buffer aibuf.
  auto k_step = [&](const int t, const int bbuf, const int abuf, const int h, const int nabuf, const int nq,
                    const int ad, const int aibuf, const int ar) __attribute__((always_inline)) {
    hipdma::wait_direct_loads<kLoads>();          // everything up to K step t - 2; what step t - 1 issued stays in flight
    __builtin_amdgcn_s_barrier();
    half_step(fa0, fb0, fa1, fb1, abuf, 2 * h + 1, bbuf, 1, [&](const int i) __attribute__((always_inline)) {
      issue_b(t + 3, (bbuf + 3) % kBStages, i);
    });
    half_step(fa1, fb1, fa0, fb0, nabuf, nq, (bbuf + 1) % kBStages, 0, [&](const int i) __attribute__((always_inline)) {
      issue_a(ad, aibuf, ar + i);
    });
  };
  int ab0 = 0;                                // A buffer of transfer kt / 2
  for (int kt = 0; kt < ksteps; kt += 4) {
    const int ab1 = ab0 == 2 ? 0 : ab0 + 1;   // transfer kt / 2 + 1
    const int ab2 = ab1 == 2 ? 0 : ab1 + 1;   // transfer kt / 2 + 2, requested during K steps kt and kt + 1
    const int d = kt >> 1;
    k_step(kt, 0, ab0, 0, ab0, 2, d + 2, ab2, 0);
    k_step(kt + 1, 1, ab0, 1, ab1, 0, d + 2, ab2, 4);
    k_step(kt + 2, 2, ab1, 0, ab1, 2, d + 3, ab0, 0);     // transfer kt / 2 + 3 takes the buffer transfer kt / 2 has left
    k_step(kt + 3, 3, ab1, 1, ab2, 0, d + 3, ab0, 4);
    ab0 = ab2;
  }
  hipdma::wait_direct_loads<0>();
  float* cbase = c + (size_t)(tile_m * kBM + wm) * n + (size_t)tile_n * kBN + wn;
#pragma unroll
  for (int i = 0; i < WI; ++i)
#pragma unroll
    for (int j = 0; j < WJ; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        const int row = i * 32 + 8 * (e / 4) + 4 * (lane >> 5) + (e % 4);
        const int col = j * 32 + (lane & 31);
        __builtin_nontemporal_store(acc[i][j][e], &cbase[(size_t)row * n + col]);
      }
}

template<int WI, int WJ, int WM = 2, int WN = 2>
int launch_gemm(const uint16_t* d_a, const uint16_t* d_b, float* d_c, int m, int n, int k, hipStream_t stream)
{
  typedef GemmShape<WI, WJ, WM, WN> shape;
  CUDADMA_REQUIRE((m % shape::kBM) == 0 && (n % shape::kBN) == 0,
                  "this variant needs m a multiple of %d and n of %d (got %d x %d)", shape::kBM, shape::kBN, m, n);
  const long long grid = (long long)(m / shape::kBM) * (n / shape::kBN);
  CUDADMA_REQUIRE(grid <= 0x7fffffffLL, "grid too large");
  hipLaunchKernelGGL((gemm_bf16_ws<WI, WJ, WM, WN>), dim3((unsigned)grid), dim3(shape::kCompute + 2 * kDmaWave), 0, stream,
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
  if (variant == 0) {
    // the largest tile that divides the problem and still gives every compute unit a tile; the small one otherwise
    const long long cus = workloads::device_cus();
    const bool m256 = (m % 256) == 0, n256 = (n % 256) == 0;
    if (m256 && n256 && (long long)(m / 256) * (n / 256) >= cus) variant = 9;
    else if (m256 && (long long)(m / 256) * (n / 128) >= cus) variant = 3;
    else if (n256 && (long long)(m / 128) * (n / 256) >= cus) variant = 2;
    else variant = 1;
  }
  switch (variant) {
    case 1: return launch_gemm<2, 2>(d_a, d_b, d_c, m, n, k, s);
    case 2: return launch_gemm<2, 4>(d_a, d_b, d_c, m, n, k, s);
    case 3: return launch_gemm<4, 2>(d_a, d_b, d_c, m, n, k, s);
#ifdef HIPDMA_SWEEP_VARIANTS
    case 5: return launch_gemm<4, 2, 2, 4>(d_a, d_b, d_c, m, n, k, s);
#endif
    case 6: case 7: case 8: case 9: {
      CUDADMA_REQUIRE((m % 256) == 0 && (n % 256) == 0, "this variant needs m and n multiples of 256 (got %d x %d)", m, n);
      const long long grid = (long long)(m / 256) * (n / 256);
      CUDADMA_REQUIRE(grid <= 0x7fffffffLL, "grid too large");
      if (variant == 7) hipLaunchKernelGGL(gemm_bf16_ws_direct4_a64, dim3((unsigned)grid), dim3(512 + 2 * kDirect4DmaThreads), 0, s, d_a, d_b, d_c, m, n, k);
      else if (variant == 9) hipLaunchKernelGGL(gemm_bf16_all_direct_a64, dim3((unsigned)grid), dim3(256), 0, s, d_a, d_b, d_c, m, n, k);
#ifdef HIPDMA_SWEEP_VARIANTS
      else if (variant == 6) hipLaunchKernelGGL(gemm_bf16_ws_direct4, dim3((unsigned)grid), dim3(512 + 2 * kDirect4DmaThreads), 0, s, d_a, d_b, d_c, m, n, k);
      else hipLaunchKernelGGL(gemm_bf16_all_direct, dim3((unsigned)grid), dim3(256), 0, s, d_a, d_b, d_c, m, n, k);
#else
      else CUDADMA_REQUIRE(false, "gemm variant %d is a sweep kernel: build the library with make EXTRA=-DHIPDMA_SWEEP_VARIANTS", variant);
#endif
      CUDADMA_HIP_CHECK(hipGetLastError());
      return CUDADMA_OK;
    }
    default: {
#ifdef HIPDMA_SWEEP_VARIANTS
      CUDADMA_REQUIRE((m % 256) == 0, "this variant needs m a multiple of 256 (got %d)", m);
      const long long grid = (long long)(m / 256) * (n / 128);
      CUDADMA_REQUIRE(grid <= 0x7fffffffLL, "grid too large");
      hipLaunchKernelGGL(gemm_bf16_ws_direct, dim3((unsigned)grid), dim3(kComputeThreads + 2 * kDmaWave), 0, s, d_a, d_b, d_c, m, n, k);
      CUDADMA_HIP_CHECK(hipGetLastError());
      return CUDADMA_OK;
#else
      CUDADMA_REQUIRE(false, "gemm variant %d is a sweep kernel: build the library with make EXTRA=-DHIPDMA_SWEEP_VARIANTS", variant);
#endif
    }
  }
}
