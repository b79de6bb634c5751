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
#include <utility>
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

// 4 x 4 transposition among the four lanes of a quad: lane i of the quad gives word k to lane k and
// ends up holding word i of lanes 0..3 (two butterfly stages of quad-permute moves).
template<int CTRL>
__device__ __forceinline__ unsigned quad_move(const unsigned v)
{ return (unsigned)__builtin_amdgcn_update_dpp(0, (int)v, CTRL, 0xf, 0xf, false); }

__device__ __forceinline__ vec4_t quad_transpose(const vec4_t a, const int lane)
{
  constexpr int kSwapPairs = 0x4E;     // quad_perm [2, 3, 0, 1]
  constexpr int kSwapLanes = 0xB1;     // quad_perm [1, 0, 3, 2]
  const bool upper = (lane & 2) != 0, odd = (lane & 1) != 0;
  const unsigned p0 = quad_move<kSwapPairs>(a[0]), p1 = quad_move<kSwapPairs>(a[1]);
  const unsigned p2 = quad_move<kSwapPairs>(a[2]), p3 = quad_move<kSwapPairs>(a[3]);
  const vec4_t b = {upper ? p2 : a[0], upper ? p3 : a[1], upper ? a[2] : p0, upper ? a[3] : p1};
  const unsigned q0 = quad_move<kSwapLanes>(b[0]), q1 = quad_move<kSwapLanes>(b[1]);
  const unsigned q2 = quad_move<kSwapLanes>(b[2]), q3 = quad_move<kSwapLanes>(b[3]);
  return vec4_t{odd ? q1 : b[0], odd ? b[1] : q0, odd ? q3 : b[2], odd ? b[3] : q2};
}

// 4 x 4 transposition among the four lanes l, l + 16, l + 32, l + 48: lane 16 i + m gives word k to lane 16 k + m and
// ends up holding word i of the four lanes.  Two butterfly stages of the swap instructions gfx950 adds
// (v_permlane32_swap: the upper half of one register against the lower half of another; v_permlane16_swap: the odd
// rows of sixteen lanes against the even ones).
__device__ __forceinline__ vec4_t group_transpose(const vec4_t a)
{
  const auto p02 = __builtin_amdgcn_permlane32_swap(a[0], a[2], false, false);
  const auto p13 = __builtin_amdgcn_permlane32_swap(a[1], a[3], false, false);
  const auto q01 = __builtin_amdgcn_permlane16_swap(p02[0], p13[0], false, false);
  const auto q23 = __builtin_amdgcn_permlane16_swap(p02[1], p13[1], false, false);
  return vec4_t{q01[0], q01[1], q23[0], q23[1]};
}

// NT: the stores carry the non-temporal hint (the output is not read again by this kernel).
template<int LDS_ROW_BYTES, bool SWIZZLED = false, bool QUAD = false, bool NT = false, typename Dma>
__device__ __forceinline__ void write_tile_transposed(const char* lds_tile, float* __restrict__ out, const int n,
                                                      const int ty, const int tx, const Dma& dma)
{
  // compute thread: lane = tile row, wavefront w handles tile columns [32w, 32w+32)
  const int lane = threadIdx.x & 63;
  const int w = threadIdx.x >> 6;
  vec4_t v[8];
  // SWIZZLED: the 16-byte unit c of row r sits at unit c ^ bitreverse4(r & 15) of the unpadded 256-byte row
  // (hipdma::swizzled_chunk), so the sixteen lanes of a quarter wavefront still hit sixteen
  // different units.
  const vec4_t* row = (const vec4_t*)(lds_tile + lane * LDS_ROW_BYTES);
#pragma unroll
  for (int j = 0; j < 8; ++j) v[j] = row[SWIZZLED ? hipdma::swizzled_chunk(lane, w * 8 + j, kRowBytes / 16) : (w * 8 + j)];
  dma.start_async_dma();
  // element (r = lane, c) of the tile goes to out[(tx*64 + c) * n + ty*64 + r]
  if constexpr (QUAD) {
    // After the transposition inside each quad, lane 4q + i holds rows 4q .. 4q+3 of tile column
    // 32w + 4j + i: four consecutive words of output row 32w + 4j + i.  One dwordx4 store per unit
    // then covers four output rows with 256 contiguous bytes each.
    float* o = out + (size_t)(tx * kTile + w * 32 + (lane & 3)) * n + (size_t)ty * kTile + (lane & ~3);
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const vec4_t t = quad_transpose(v[j], lane);
      if constexpr (NT) __builtin_nontemporal_store(t, (vec4_t*)(o + (size_t)(4 * j) * n));
      else *(vec4_t*)(o + (size_t)(4 * j) * n) = t;
    }
  } else {
    float* o = out + (size_t)(tx * kTile + w * 32) * n + (size_t)ty * kTile + lane;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        if constexpr (NT) __builtin_nontemporal_store(__uint_as_float(v[j][k]), o + (size_t)(4 * j + k) * n);
        else o[(size_t)(4 * j + k) * n] = __uint_as_float(v[j][k]);
      }
    }
  }
}

template<int LDS_ROW_BYTES, bool QUAD = false>
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
    if (t + 3 * stride < num_tiles) {
      // Steady state with no branch around any load, entered from a prologue that has none either:
      // every path into a wait then carries the same loads, and the wait for one object's tile
      // leaves the other object's eight loads in flight (s_waitcnt vmcnt(15..8), not vmcnt(7..0)).
      dma0.template start_xfer_async<true, LOAD_CACHE_ALL, STORE_LDS>(src_of(t));
      dma1.template start_xfer_async<true, LOAD_CACHE_ALL, STORE_LDS>(src_of(t + stride));
      do {
        dma0.template wait_xfer_finish<true, LOAD_CACHE_ALL, STORE_LDS>(buf0);
        dma0.template start_xfer_async<true, LOAD_CACHE_ALL, STORE_LDS>(src_of(t + 2 * stride));
        dma1.template wait_xfer_finish<true, LOAD_CACHE_ALL, STORE_LDS>(buf1);
        dma1.template start_xfer_async<true, LOAD_CACHE_ALL, STORE_LDS>(src_of(t + 3 * stride));
        t += 2 * stride;
      } while (t + 3 * stride < num_tiles);
    } else {
      if (t < num_tiles) dma0.template start_xfer_async<true, LOAD_CACHE_ALL, STORE_LDS>(src_of(t));
      if (t + stride < num_tiles) dma1.template start_xfer_async<true, LOAD_CACHE_ALL, STORE_LDS>(src_of(t + stride));
    }
    // the last tiles of this workgroup
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
      write_tile_transposed<LDS_ROW_BYTES, false, QUAD>(buf0, out, n, ty, tx, dma0);
      if (t + stride < num_tiles) {
        tile_coords(t + stride, tiles_per_side, band, ty, tx);
        dma1.wait_for_dma_finish();
        write_tile_transposed<LDS_ROW_BYTES, false, QUAD>(buf1, out, n, ty, tx, dma1);
      }
    }
  }
}

// The smallest warp-specialised shape: one DMA wavefront and one compute wavefront per workgroup, two
// objects on the DMA wavefront (each holds a whole tile, 16 dwordx4 per lane), two LDS tiles.  The
// handshake then runs between two wavefronts only.
template<bool QUAD>
__global__ void __launch_bounds__(128)
transpose_pairs(const float* __restrict__ in, float* __restrict__ out, const int n, const int num_tiles, const int band)
{
  constexpr int kLdsRow = 272;
  __shared__ __attribute__((aligned(16))) char buf0[kTile * kLdsRow];
  __shared__ __attribute__((aligned(16))) char buf1[kTile * kLdsRow];
  typedef CudaDMAStrided<true, 16, kTile * kRowBytes / 64, kRowBytes, 64, kTile> dma_t;
  dma_t dma0(0, 64, 64, n * 4, kLdsRow);
  dma_t dma1(1, 64, 64, n * 4, kLdsRow);
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
    const int lane = threadIdx.x;
    auto write_out = [&](const char* lds_tile, const int t, const dma_t& dma) __attribute__((always_inline)) {
      int ty, tx;
      tile_coords(t, tiles_per_side, band, ty, tx);
      vec4_t v[16];
      const vec4_t* row = (const vec4_t*)(lds_tile + lane * kLdsRow);
#pragma unroll
      for (int j = 0; j < 16; ++j) v[j] = row[j];
      dma.start_async_dma();
      if constexpr (QUAD) {
        float* o = out + (size_t)(tx * kTile + (lane & 3)) * n + (size_t)ty * kTile + (lane & ~3);
#pragma unroll
        for (int j = 0; j < 16; ++j) *(vec4_t*)(o + (size_t)(4 * j) * n) = quad_transpose(v[j], lane);
      } else {
        float* o = out + (size_t)(tx * kTile) * n + (size_t)ty * kTile + lane;
#pragma unroll
        for (int j = 0; j < 16; ++j) {
#pragma unroll
          for (int k = 0; k < 4; ++k) o[(size_t)(4 * j + k) * n] = __uint_as_float(v[j][k]);
        }
      }
    };
    dma0.start_async_dma();
    dma1.start_async_dma();
    for (int t = blockIdx.x; t < num_tiles; t += 2 * stride) {
      dma0.wait_for_dma_finish();
      write_out(buf0, t, dma0);
      if (t + stride < num_tiles) {
        dma1.wait_for_dma_finish();
        write_out(buf1, t + stride, dma1);
      }
    }
  }
}

// Two DMA groups of one wavefront, one object and one LDS tile each
// (src/perf/sequential/perf_sequential.cu:116-173).  A wavefront's loads complete in
// issue order and s_waitcnt counts them in that order, so a wavefront that owns a
// single object waits for exactly its own tile; the second tile in flight belongs
// to the other wavefront.  Each DMA thread holds a whole tile share of 16 dwordx4.
template<int LDS_ROW_BYTES, int SQ = STORE_LDS>
__global__ void __launch_bounds__(kDmaThreads + kComputeThreads)
transpose_double_groups(const float* __restrict__ in, float* __restrict__ out, const int n, const int num_tiles,
                        const int band)
{
  __shared__ __attribute__((aligned(16))) char buf0[kTile * LDS_ROW_BYTES];
  __shared__ __attribute__((aligned(16))) char buf1[kTile * LDS_ROW_BYTES];
  constexpr int kGroup = kDmaThreads / 2;
  typedef CudaDMAStrided<true, 16, kTile * kRowBytes / kGroup, kRowBytes, kGroup, kTile> dma_t;
  dma_t dma0(0, kComputeThreads, kComputeThreads, n * 4, LDS_ROW_BYTES);
  dma_t dma1(1, kComputeThreads, kComputeThreads + kGroup, n * 4, LDS_ROW_BYTES);
  const int tiles_per_side = n / kTile;
  const int stride = gridDim.x;
  auto src_of = [&](const int t) {
    int ty, tx;
    tile_coords(t, tiles_per_side, band, ty, tx);
    return (const void*)(in + (size_t)ty * kTile * n + (size_t)tx * kTile);
  };
  // always inlined: called once per DMA group, and an object that is passed to a real function
  // lives in scratch memory
  auto dma_loop = [&](dma_t& dma, char* buf, int t) __attribute__((always_inline)) {
    if (t < num_tiles) dma.template start_xfer_async<true, LOAD_CACHE_ALL, SQ>(src_of(t));
    for (; t + 2 * stride < num_tiles; t += 2 * stride) {
      dma.template wait_xfer_finish<true, LOAD_CACHE_ALL, SQ>(buf);
      dma.template start_xfer_async<true, LOAD_CACHE_ALL, SQ>(src_of(t + 2 * stride));
    }
    if (t < num_tiles) dma.template wait_xfer_finish<true, LOAD_CACHE_ALL, SQ>(buf);
  };
  if (dma0.owns_this_thread()) {
    dma_loop(dma0, buf0, blockIdx.x);
  } else if (dma1.owns_this_thread()) {
    dma_loop(dma1, buf1, blockIdx.x + stride);
  } else {
    dma0.start_async_dma();
    dma1.start_async_dma();
    for (int t = blockIdx.x; t < num_tiles; t += 2 * stride) {
      int ty, tx;
      tile_coords(t, tiles_per_side, band, ty, tx);
      dma0.wait_for_dma_finish();
      write_tile_transposed<LDS_ROW_BYTES, hipdma::detail::store_is_swizzled(SQ)>(buf0, out, n, ty, tx, dma0);
      if (t + stride < num_tiles) {
        tile_coords(t + stride, tiles_per_side, band, ty, tx);
        dma1.wait_for_dma_finish();
        write_tile_transposed<LDS_ROW_BYTES, hipdma::detail::store_is_swizzled(SQ)>(buf1, out, n, ty, tx, dma1);
      }
    }
  }
}

// The form that is not warp-specialised (src/examples/stencil/non_warp_specialized_double_buffer.h:52-89):
// all four wavefronts move the tile into LDS, meet, and all four write it out
// transposed.  The next tile is requested (two-phase call) before the current one
// is consumed, so its loads are in flight under the LDS reads and the stores.
__global__ void __launch_bounds__(kDmaThreads + kComputeThreads)
transpose_not_specialized(const float* __restrict__ in, float* __restrict__ out, const int n, const int num_tiles,
                          const int band)
{
  constexpr int kLdsRow = 272;
  constexpr int kThreads = kDmaThreads + kComputeThreads;
  __shared__ __attribute__((aligned(16))) char buf[kTile * kLdsRow];
  CudaDMAStrided<false, 16, kTile * kRowBytes / kThreads, kRowBytes, kThreads, kTile> dma(n * 4, kLdsRow);
  const int tiles_per_side = n / kTile;
  const int stride = gridDim.x;
  const int last = num_tiles - 1;
  auto src_of = [&](const int t) {
    int ty, tx;
    tile_coords(t, tiles_per_side, band, ty, tx);
    return (const void*)(in + (size_t)ty * kTile * n + (size_t)tx * kTile);
  };
  const int lane = threadIdx.x & 63;
  const int w = threadIdx.x >> 6;          // wavefront w writes tile columns [16w, 16w+16)
  int t = blockIdx.x;
  if (t >= num_tiles) return;
  dma.template start_xfer_async<true, LOAD_CACHE_ALL, STORE_LDS>(src_of(t));
  for (; t < num_tiles; t += stride) {
    dma.template wait_xfer_finish<true, LOAD_CACHE_ALL, STORE_LDS>(buf);
    __syncthreads();
    // past the last tile the last one is requested again: the loads stay unconditional
    const int tn = (t + stride < num_tiles) ? (t + stride) : last;
    dma.template start_xfer_async<true, LOAD_CACHE_ALL, STORE_LDS>(src_of(tn));
    vec4_t v[4];
    const vec4_t* row = (const vec4_t*)(buf + lane * kLdsRow) + w * 4;
#pragma unroll
    for (int j = 0; j < 4; ++j) v[j] = row[j];
    __syncthreads();
    int ty, tx;
    tile_coords(t, tiles_per_side, band, ty, tx);
    float* o = out + (size_t)(tx * kTile + w * 16) * n + (size_t)ty * kTile + lane;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
#pragma unroll
      for (int k = 0; k < 4; ++k) o[(size_t)(4 * j + k) * n] = __uint_as_float(v[j][k]);
    }
  }
}

// STREAM: the loads and the stores carry the streaming / non-temporal hints.  At one workgroup per compute unit, where
// a tile takes one trip to memory, they are worth 5 %; with more in flight they change nothing.
template<bool STREAM, bool QUAD = false>
__global__ void __launch_bounds__(kDmaThreads + kComputeThreads)
transpose_single(const float* __restrict__ in, float* __restrict__ out, const int n, const int num_tiles, const int band)
{
  constexpr int kLoadQual = STREAM ? LOAD_CACHE_STREAMING : LOAD_CACHE_ALL;
  constexpr int kLdsRow = 272;
  __shared__ __attribute__((aligned(16))) char buf[kTile * kLdsRow];
  CudaDMAStrided<true, 16, kBytesPerThread, kRowBytes, kDmaThreads, kTile>
      dma(0, kComputeThreads, kComputeThreads, n * 4, kLdsRow);
  const int tiles_per_side = n / kTile;
  if (dma.owns_this_thread()) {
    for (int t = blockIdx.x; t < num_tiles; t += gridDim.x) {
      int ty, tx;
      tile_coords(t, tiles_per_side, band, ty, tx);
      dma.template execute_dma<true, kLoadQual, STORE_LDS>(in + (size_t)ty * kTile * n + (size_t)tx * kTile, buf);
    }
  } else {
    dma.start_async_dma();
    for (int t = blockIdx.x; t < num_tiles; t += gridDim.x) {
      int ty, tx;
      tile_coords(t, tiles_per_side, band, ty, tx);
      dma.wait_for_dma_finish();
      write_tile_transposed<kLdsRow, false, QUAD, STREAM>(buf, out, n, ty, tx, dma);
    }
  }
}

// The single-tile kernel with the split of the workgroup between the two roles as a parameter: DW DMA wavefronts,
// CW compute wavefronts, and AHEAD tiles requested beyond the one in LDS (1: what execute_dma does; 2: two objects
// that share the DMA wavefronts and the LDS tile, each holding one requested tile in registers, in the manner of
// src/examples/stencil/warp_specialized_manual_buffer.h:54-71).  The objects carry no handshake of their own; one
// sync-only object guards the tile (include/cudaDMA.h:4184-4208).  Streaming loads, quad transposition, non-temporal
// dwordx4 stores as in transpose_single<true, true>.
// GROUPS: the compute lanes take the tile rows so that the transposition runs among lanes sixteen apart (lane 16 i + m
// reads row 4 m + i); sixteen consecutive lanes then store 256 contiguous bytes of one output row, where the
// transposition inside a quad leaves four consecutive lanes on four different output rows (the address unit then
// handles 64 pieces per store instruction instead of 16).  The price: lanes sixteen apart read rows whose 16-byte
// units coincide modulo 256 B whatever the padding, a two-way bank conflict in every ds_read_b128.
template<int DW, int CW, int AHEAD, bool GROUPS = false>
__global__ void __launch_bounds__((DW + CW) * 64)
transpose_split(const float* __restrict__ in, float* __restrict__ out, const int n, const int num_tiles, const int band)
{
  const int first_tile = blockIdx.x;
  static_assert(CW == 1 || CW == 2 || CW == 4, "the compute wavefronts share the sixteen 16-byte columns of a tile row evenly");
  static_assert(AHEAD >= 1 && AHEAD <= 3, "one or two tiles requested ahead, or (3) one in flight with two register sets");
  constexpr int kLdsRow = 272;
  constexpr int kDma = DW * 64, kCompute = CW * 64;
  constexpr int kChunks = kTile * kRowBytes / 16;
  constexpr int kBpt = ((kChunks + kDma - 1) / kDma) * 16;
  __shared__ __attribute__((aligned(16))) char buf[kTile * kLdsRow];
  cudaDMACustom guard(0, kDma, kCompute, kCompute);
  typedef CudaDMAStrided<false, 16, kBpt, kRowBytes, kDma, kTile> obj_t;
  const int tiles_per_side = n / kTile;
  const int stride = gridDim.x;
  const int last = num_tiles - 1;
  auto src_of = [&](const int t) {
    int ty, tx;
    tile_coords(t < num_tiles ? t : last, tiles_per_side, band, ty, tx);     // past the end: the last tile again, loads stay unconditional
    return (const void*)(in + (size_t)ty * kTile * n + (size_t)tx * kTile);
  };
  if (guard.owns_this_thread()) {
    obj_t a(n * 4, kLdsRow, kCompute), b(n * 4, kLdsRow, kCompute);
    auto land = [&](obj_t& o) __attribute__((always_inline)) {
      guard.wait_for_dma_start();
      o.template wait_xfer_finish<true, LOAD_CACHE_STREAMING, STORE_LDS>(buf);
      guard.finish_async_dma();
    };
    int t = first_tile;
    if (t >= num_tiles) return;
    a.template start_xfer_async<true, LOAD_CACHE_STREAMING, STORE_LDS>(src_of(t));
    if constexpr (AHEAD == 3) {
      // two register sets but one tile in flight: the next tile is requested as soon as the loads of the current one
      // have returned, before it is stored to LDS, so that the store and the handshake leave the round trip
      auto returned = [&]() __attribute__((always_inline)) {
        asm volatile("" ::: "memory");
        hipdma::detail::wait_lds_direct();                 // s_waitcnt vmcnt(0)
        asm volatile("" ::: "memory");
      };
      for (; t < num_tiles; t += 2 * stride) {
        returned();
        b.template start_xfer_async<true, LOAD_CACHE_STREAMING, STORE_LDS>(src_of(t + stride));
        land(a);
        if (t + stride < num_tiles) {
          returned();
          a.template start_xfer_async<true, LOAD_CACHE_STREAMING, STORE_LDS>(src_of(t + 2 * stride));
          land(b);
        }
      }
      return;
    }
    if constexpr (AHEAD == 2) b.template start_xfer_async<true, LOAD_CACHE_STREAMING, STORE_LDS>(src_of(t + stride));
    for (; t < num_tiles; t += AHEAD * stride) {
      land(a);
      a.template start_xfer_async<true, LOAD_CACHE_STREAMING, STORE_LDS>(src_of(t + AHEAD * stride));
      if constexpr (AHEAD == 2) {
        if (t + stride < num_tiles) land(b);
        b.template start_xfer_async<true, LOAD_CACHE_STREAMING, STORE_LDS>(src_of(t + 3 * stride));
      }
    }
  } else {
    // lane = tile row; wavefront w takes the 16 / CW 16-byte columns [w * 16 / CW, (w + 1) * 16 / CW) of that row
    constexpr int kUnits = 16 / CW;
    const int lane = threadIdx.x & 63;
    const int w = threadIdx.x >> 6;
    guard.start_async_dma();
    for (int t = first_tile; t < num_tiles; t += stride) {
      int ty, tx;
      tile_coords(t, tiles_per_side, band, ty, tx);
      guard.wait_for_dma_finish();
      vec4_t v[kUnits];
      const int tile_row = GROUPS ? 4 * (lane & 15) + (lane >> 4) : lane;
      const vec4_t* row = (const vec4_t*)(buf + tile_row * kLdsRow) + w * kUnits;
#pragma unroll
      for (int j = 0; j < kUnits; ++j) v[j] = row[j];
      guard.start_async_dma();
      if constexpr (GROUPS) {
        float* o = out + (size_t)(tx * kTile + w * 4 * kUnits + (lane >> 4)) * n + (size_t)ty * kTile + 4 * (lane & 15);
#pragma unroll
        for (int j = 0; j < kUnits; ++j)
          __builtin_nontemporal_store(group_transpose(v[j]), (vec4_t*)(o + (size_t)(4 * j) * n));
      } else {
        float* o = out + (size_t)(tx * kTile + w * 4 * kUnits + (lane & 3)) * n + (size_t)ty * kTile + (lane & ~3);
#pragma unroll
        for (int j = 0; j < kUnits; ++j)
          __builtin_nontemporal_store(quad_transpose(v[j], lane), (vec4_t*)(o + (size_t)(4 * j) * n));
      }
    }
  }
}

// The double buffer in LDS with one object: two LDS tiles, each with a sync-only guard, filled in turn by one
// CudaDMAStrided object on the DMA wavefronts; the tile after the one that is landing waits in their registers, so one
// tile of loads is in flight (the amount this pattern runs best with) while up to two tiles sit in LDS.  The compute
// side is that of transpose_split.  src/perf/sequential/perf_sequential.cu:116-173 is the reference's double buffering
// (two objects on two DMA groups); with the two-phase calls one object serves both buffers.
template<int DW, int CW>
__global__ void __launch_bounds__((DW + CW) * 64)
transpose_double_lds(const float* __restrict__ in, float* __restrict__ out, const int n, const int num_tiles, const int band)
{
  static_assert(CW == 1 || CW == 2 || CW == 4, "the compute wavefronts share the sixteen 16-byte columns of a tile row evenly");
  constexpr int kLdsRow = 272;
  constexpr int kDma = DW * 64, kCompute = CW * 64;
  constexpr int kChunks = kTile * kRowBytes / 16;
  constexpr int kBpt = ((kChunks + kDma - 1) / kDma) * 16;
  __shared__ __attribute__((aligned(16))) char buf0[kTile * kLdsRow];
  __shared__ __attribute__((aligned(16))) char buf1[kTile * kLdsRow];
  cudaDMACustom guard0(0, kDma, kCompute, kCompute);
  cudaDMACustom guard1(1, kDma, kCompute, kCompute);
  typedef CudaDMAStrided<false, 16, kBpt, kRowBytes, kDma, kTile> obj_t;
  const int tiles_per_side = n / kTile;
  const int stride = gridDim.x;
  const int last = num_tiles - 1;
  auto src_of = [&](const int t) {
    int ty, tx;
    tile_coords(t < num_tiles ? t : last, tiles_per_side, band, ty, tx);     // past the end: the last tile again, loads stay unconditional
    return (const void*)(in + (size_t)ty * kTile * n + (size_t)tx * kTile);
  };
  if (guard0.owns_this_thread()) {
    obj_t a(n * 4, kLdsRow, kCompute);
    int t = blockIdx.x;
    if (t >= num_tiles) return;
    a.template start_xfer_async<true, LOAD_CACHE_STREAMING, STORE_LDS>(src_of(t));
    for (;;) {
      guard0.wait_for_dma_start();
      a.template wait_xfer_finish<true, LOAD_CACHE_STREAMING, STORE_LDS>(buf0);
      guard0.finish_async_dma();
      a.template start_xfer_async<true, LOAD_CACHE_STREAMING, STORE_LDS>(src_of(t + stride));
      if (t + stride >= num_tiles) break;
      guard1.wait_for_dma_start();
      a.template wait_xfer_finish<true, LOAD_CACHE_STREAMING, STORE_LDS>(buf1);
      guard1.finish_async_dma();
      a.template start_xfer_async<true, LOAD_CACHE_STREAMING, STORE_LDS>(src_of(t + 2 * stride));
      t += 2 * stride;
      if (t >= num_tiles) break;
    }
  } else {
    constexpr int kUnits = 16 / CW;
    const int lane = threadIdx.x & 63;
    const int w = threadIdx.x >> 6;
    auto write_out = [&](const char* tile, const cudaDMACustom& guard, const int t) __attribute__((always_inline)) {
      int ty, tx;
      tile_coords(t, tiles_per_side, band, ty, tx);
      guard.wait_for_dma_finish();
      vec4_t v[kUnits];
      const vec4_t* row = (const vec4_t*)(tile + lane * kLdsRow) + w * kUnits;
#pragma unroll
      for (int j = 0; j < kUnits; ++j) v[j] = row[j];
      guard.start_async_dma();
      float* o = out + (size_t)(tx * kTile + w * 4 * kUnits + (lane & 3)) * n + (size_t)ty * kTile + (lane & ~3);
#pragma unroll
      for (int j = 0; j < kUnits; ++j)
        __builtin_nontemporal_store(quad_transpose(v[j], lane), (vec4_t*)(o + (size_t)(4 * j) * n));
    };
    guard0.start_async_dma();
    guard1.start_async_dma();
    for (int t = blockIdx.x; t < num_tiles; t += 2 * stride) {
      write_out(buf0, guard0, t);
      if (t + stride < num_tiles) write_out(buf1, guard1, t + stride);
    }
  }
}

#ifdef HIPDMA_SWEEP_VARIANTS
// The transposition with output rows written 1 KiB at a time.  The DMA side is that of transpose_split (tiles of 64
// rows x 256 B, one tile of loads in flight, NBUF LDS tiles guarded by sync-only objects); the compute wavefront
// gathers four tiles that lie one below the other in the source (so side by side in the output) in a second LDS
// buffer, already transposed (four ds_write_b32 per 16-byte unit, 64 lanes on 64 consecutive words: no conflicts),
// and then writes 64 output rows of 1 KiB, one row per store instruction.  A write-only stream with the
// transposition's addresses runs at 67 % of peak in pieces of 256 B and at 78 % in pieces of 1 KiB; the reads care
// less (87 % in pieces of 256 B against 91 % for a linear stream).  Reads and writes together gain nothing from it:
// 74.0 % against 74.8 % for transpose_split<3, 1, 1> in the same run, which is why this kernel is only built for the
// sweeps.
// order 0: the workgroups that run together take neighbouring groups of four tile rows first (they write whole output
// rows together); order 1: neighbouring tile columns first (they read whole source rows together).
template<int DW, int NBUF>
__global__ void __launch_bounds__((DW + 1) * 64)
transpose_wide_rows(const float* __restrict__ in, float* __restrict__ out, const int n, const int order)
{
  static_assert(NBUF == 1 || NBUF == 2, "one or two LDS tiles");
  constexpr int kLdsRow = 272;
  constexpr int kDma = DW * 64, kCompute = 64;
  constexpr int kChunks = kTile * kRowBytes / 16;
  constexpr int kBpt = ((kChunks + kDma - 1) / kDma) * 16;
  constexpr int kGroup = 4;                               // tiles gathered per pass: 4 x 256 B = 1 KiB of every output row
  __shared__ __attribute__((aligned(16))) char buf[NBUF][kTile * kLdsRow];
  __shared__ __attribute__((aligned(16))) float stage[kTile][kGroup * kTile];
  cudaDMACustom guard0(0, kDma, kCompute, kCompute);
  cudaDMACustom guard1(1, kDma, kCompute, kCompute);
  typedef CudaDMAStrided<false, 16, kBpt, kRowBytes, kDma, kTile> obj_t;
  const int tiles_per_side = n / kTile;
  const int groups_per_side = (tiles_per_side + kGroup - 1) / kGroup;
  const int passes = groups_per_side * tiles_per_side;    // a pass: up to four tiles (group q of tile rows, tile column tx)
  const int stride = gridDim.x;
  auto pass_coords = [&](const int p, int& q, int& tx) {
    if (order == 0) { tx = p / groups_per_side; q = p - tx * groups_per_side; }
    else { q = p / tiles_per_side; tx = p - q * tiles_per_side; }
  };
  auto tiles_in = [&](const int q) { const int left = tiles_per_side - q * kGroup; return left < kGroup ? left : kGroup; };
  if (guard0.owns_this_thread()) {
    obj_t a(n * 4, kLdsRow, kCompute);
    int p = blockIdx.x;
    if (p >= passes) return;
    int q, tx, k = 0;
    pass_coords(p, q, tx);
    int count = tiles_in(q);
    auto src_now = [&]() { return (const void*)(in + (size_t)(q * kGroup + k) * kTile * n + (size_t)tx * kTile); };
    a.template start_xfer_async<true, LOAD_CACHE_STREAMING, STORE_LDS>(src_now());
    unsigned i = 0;
    for (;;) {
      if (NBUF == 2 && (i & 1u)) {
        guard1.wait_for_dma_start();
        a.template wait_xfer_finish<true, LOAD_CACHE_STREAMING, STORE_LDS>(buf[NBUF - 1]);
        guard1.finish_async_dma();
      } else {
        guard0.wait_for_dma_start();
        a.template wait_xfer_finish<true, LOAD_CACHE_STREAMING, STORE_LDS>(buf[0]);
        guard0.finish_async_dma();
      }
      ++i;
      if (++k == count) {
        p += stride;
        if (p >= passes) break;
        pass_coords(p, q, tx);
        count = tiles_in(q);
        k = 0;
      }
      a.template start_xfer_async<true, LOAD_CACHE_STREAMING, STORE_LDS>(src_now());
    }
  } else {
    const int lane = threadIdx.x & 63;
    guard0.start_async_dma();
    if constexpr (NBUF == 2) guard1.start_async_dma();
    unsigned i = 0;
    for (int p = blockIdx.x; p < passes; p += stride) {
      int q, tx;
      pass_coords(p, q, tx);
      const int count = tiles_in(q);
      for (int k = 0; k < count; ++k, ++i) {
        const bool second = NBUF == 2 && (i & 1u);
        if (second) guard1.wait_for_dma_finish(); else guard0.wait_for_dma_finish();
        // lane = tile row r: its sixteen 16-byte units
        vec4_t v[16];
        const vec4_t* row = (const vec4_t*)(buf[second ? NBUF - 1 : 0] + lane * kLdsRow);
#pragma unroll
        for (int j = 0; j < 16; ++j) v[j] = row[j];
        if (second) guard1.start_async_dma(); else guard0.start_async_dma();
        // element (r, c) of tile k becomes word 64 k + r of output row c
        float* col = &stage[0][k * kTile + lane];
#pragma unroll
        for (int j = 0; j < 16; ++j) {
#pragma unroll
          for (int w = 0; w < 4; ++w) col[(4 * j + w) * (kGroup * kTile)] = __uint_as_float(v[j][w]);
        }
      }
      // 64 output rows of count x 256 B: lane l carries the 16 bytes at 16 l of every row
      float* o = out + (size_t)tx * kTile * n + (size_t)q * (kGroup * kTile) + 4 * lane;
      if (lane < 16 * count) {
#pragma unroll
        for (int batch = 0; batch < 4; ++batch) {
          vec4_t w[16];
#pragma unroll
          for (int m = 0; m < 16; ++m) w[m] = *(const vec4_t*)&stage[16 * batch + m][4 * lane];
#pragma unroll
          for (int m = 0; m < 16; ++m) __builtin_nontemporal_store(w[m], (vec4_t*)(o + (size_t)(16 * batch + m) * n));
        }
      }
    }
  }
}

// N copies of an object without a default constructor
template<typename T, int N> struct Copies { T v[N]; };
template<typename T, int... I>
__device__ __forceinline__ Copies<T, (int)sizeof...(I)> copies_of(const T& x, std::integer_sequence<int, I...>)
{ return Copies<T, (int)sizeof...(I)>{{((void)I, x)...}}; }

// transpose_split with the tile requested in K pieces of 64 / K rows, M pieces in flight: between whole numbers of
// tiles ahead (M / K = 1.25, 1.5, 1.75 tiles outstanding per workgroup).  One CudaDMAStrided object per piece in
// flight, all on the same DMA wavefronts (manual buffering, src/examples/stencil/warp_specialized_manual_buffer.h:54-71);
// the LDS tile is handed over whole: the guard is taken before the first piece of a tile lands and released after
// the last.  The compute side is that of transpose_split.
template<int DW, int CW, int K, int M>
__global__ void __launch_bounds__((DW + CW) * 64)
transpose_pieces(const float* __restrict__ in, float* __restrict__ out, const int n, const int num_tiles, const int band)
{
  static_assert(CW == 1 || CW == 2 || CW == 4, "the compute wavefronts share the sixteen 16-byte columns of a tile row evenly");
  static_assert(kTile % K == 0 && 2 * M >= K && M <= 2 * K, "between half a tile and two tiles in flight");
  constexpr int kLdsRow = 272;
  constexpr int kDma = DW * 64, kCompute = CW * 64;
  constexpr int kRows = kTile / K;
  constexpr int kChunks = kRows * kRowBytes / 16;
  constexpr int kBpt = ((kChunks + kDma - 1) / kDma) * 16;
  __shared__ __attribute__((aligned(16))) char buf[kTile * kLdsRow];
  cudaDMACustom guard(0, kDma, kCompute, kCompute);
  typedef CudaDMAStrided<false, 16, kBpt, kRowBytes, kDma, kRows> obj_t;
  const int tiles_per_side = n / kTile;
  const int stride = gridDim.x;
  const int last = num_tiles - 1;
  if (guard.owns_this_thread()) {
    // piece q of this workgroup: part q % K of its tile number q / K; past the end the last tile again, so that the
    // loads stay unconditional
    auto src_of = [&](const int q) {
      const int t = blockIdx.x + (q / K) * stride;
      int ty, tx;
      tile_coords(t < num_tiles ? t : last, tiles_per_side, band, ty, tx);
      return (const void*)(in + ((size_t)ty * kTile + (size_t)((q % K) * kRows)) * n + (size_t)tx * kTile);
    };
    if ((int)blockIdx.x >= num_tiles) return;
    Copies<obj_t, M> objs = copies_of(obj_t(n * 4, kLdsRow, kCompute), std::make_integer_sequence<int, M>());
    obj_t* o = objs.v;
#pragma unroll
    for (int i = 0; i < M; ++i) o[i].template start_xfer_async<true, LOAD_CACHE_STREAMING, STORE_LDS>(src_of(i));
    const int pieces = ((num_tiles - 1 - (int)blockIdx.x) / stride + 1) * K;
    // K * M pieces per turn: object and part of every step are then compile-time constants
    for (int q0 = 0; q0 < pieces; q0 += K * M) {
#pragma unroll
      for (int i = 0; i < K * M; ++i) {
        if (q0 + i < pieces) {
          if (i % K == 0) guard.wait_for_dma_start();
          o[i % M].template wait_xfer_finish<true, LOAD_CACHE_STREAMING, STORE_LDS>(buf + (i % K) * kRows * kLdsRow);
          if (i % K == K - 1) guard.finish_async_dma();
        }
        o[i % M].template start_xfer_async<true, LOAD_CACHE_STREAMING, STORE_LDS>(src_of(q0 + i + M));
      }
    }
  } else {
    constexpr int kUnits = 16 / CW;
    const int lane = threadIdx.x & 63;
    const int w = threadIdx.x >> 6;
    guard.start_async_dma();
    for (int t = blockIdx.x; t < num_tiles; t += stride) {
      int ty, tx;
      tile_coords(t, tiles_per_side, band, ty, tx);
      guard.wait_for_dma_finish();
      vec4_t v[kUnits];
      const vec4_t* row = (const vec4_t*)(buf + lane * kLdsRow) + w * kUnits;
#pragma unroll
      for (int j = 0; j < kUnits; ++j) v[j] = row[j];
      guard.start_async_dma();
      float* o = out + (size_t)(tx * kTile + w * 4 * kUnits + (lane & 3)) * n + (size_t)ty * kTile + (lane & ~3);
#pragma unroll
      for (int j = 0; j < kUnits; ++j)
        __builtin_nontemporal_store(quad_transpose(v[j], lane), (vec4_t*)(o + (size_t)(4 * j) * n));
    }
  }
}
#endif  // HIPDMA_SWEEP_VARIANTS

typedef void (*split_kernel_t)(const float*, float*, int, int, int);
struct SplitEntry { int dw, cw, ahead; split_kernel_t kernel; };
#define SPLIT(DW, CW) {DW, CW, 1, transpose_split<DW, CW, 1>}, {DW, CW, 2, transpose_split<DW, CW, 2>}
// The library holds the split it reports (three DMA wavefronts + one compute wavefront), the even split, and both with
// two tiles ahead.  The other splits, the tile requested in pieces ("tiles ahead" 3 .. 7 with 3 + 1 wavefronts: 3 = 3
// halves in flight (1.5 tiles), 4 = 5 quarters (1.25), 5 = 6 quarters (1.5), 6 = 7 quarters (1.75), 7 = 3 quarters
// (0.75)) and the schedule without a pause (8: two register sets, the next tile requested as soon as the loads of the
// current one have returned) were all measured slower; they are compiled with -DHIPDMA_SWEEP_VARIANTS for the sweeps.
const SplitEntry kSplits[] = {SPLIT(3, 1), SPLIT(2, 2),
#ifdef HIPDMA_SWEEP_VARIANTS
                              // 9: one tile ahead, the transposition among lanes sixteen apart (GROUPS): 0.5 % faster than the
                              // transposition inside a quad at the price of two-way bank conflicts in the LDS reads
                              {3, 1, 9, transpose_split<3, 1, 1, true>}, {2, 2, 9, transpose_split<2, 2, 1, true>},
                              {4, 1, 9, transpose_split<4, 1, 1, true>}, {2, 1, 9, transpose_split<2, 1, 1, true>},
                              {3, 1, 3, transpose_pieces<3, 1, 2, 3>}, {3, 1, 4, transpose_pieces<3, 1, 4, 5>},
                              {3, 1, 5, transpose_pieces<3, 1, 4, 6>}, {3, 1, 6, transpose_pieces<3, 1, 4, 7>},
                              {3, 1, 7, transpose_pieces<3, 1, 4, 3>},
                              {3, 1, 8, transpose_split<3, 1, 3>}, {2, 2, 8, transpose_split<2, 2, 3>},
                              SPLIT(1, 1), SPLIT(1, 2), SPLIT(2, 1), SPLIT(4, 1), SPLIT(3, 2), SPLIT(4, 2), SPLIT(1, 4), SPLIT(2, 4), SPLIT(4, 4),
#endif
};
#undef SPLIT

}  // namespace

extern "C" int cudadma_transpose_splits(int* codes, int capacity)
{
  int n = 0;
  for (const SplitEntry& c : kSplits) {
    if (codes != nullptr && n < capacity) codes[n] = 100 * c.dw + 10 * c.cw + c.ahead;
    ++n;
  }
  return n;
}

extern "C" int cudadma_strided_transpose(const float* d_in, float* d_out, int n, int variant, void* stream)
{
  CUDADMA_REQUIRE(n >= 0 && (n % kTile) == 0, "n (%d) must be a multiple of %d", n, kTile);
  CUDADMA_REQUIRE((long long)n * 4 <= 0x7fffffffLL, "row pitch must fit an int");
  if (variant < 0 || variant >= cudadma_num_variants(CUDADMA_WORKLOAD_STRIDED)) {
    cudadma_host::set_error("strided transpose has no variant %d", variant);
    return CUDADMA_ERANGE;
  }
  if (n == 0) return CUDADMA_OK;
  CUDADMA_REQUIRE(d_in != nullptr && d_out != nullptr && d_in != d_out, "NULL or aliased pointers");
  CUDADMA_REQUIRE(cudadma_host::aligned_to(d_in, 16) && cudadma_host::aligned_to(d_out, 16), "pointers must be 16-byte aligned");
  const int tiles_per_side = n / kTile;
  const int tiles = tiles_per_side * tiles_per_side;
  // The kernels with one LDS tile (variants 1 and 4) run best with exactly one workgroup per compute unit, i.e. one
  // 16 KB tile of loads in flight per compute unit, and with the tiles walked down the columns (the workgroups that
  // run together then write whole output rows); the others with four workgroups and bands of 16 tile rows.
  const bool one_tile = variant == 0 || variant == 1 || variant == 4 || variant == 10 || variant == 14;
  int band = workloads::tuning("transpose_band", one_tile ? tiles_per_side : kDefaultBand);
  if (band > tiles_per_side) band = tiles_per_side;
  while (band > 1 && tiles_per_side % band != 0) band /= 2;      // bands must tile the matrix
  const int forced = workloads::tuning("transpose_workgroups", 0);
  auto grid_for = [&](const int per_cu) {
    return dim3((unsigned)(forced > 0 ? (forced < tiles ? forced : tiles) : workloads::persistent_grid(tiles, per_cu)));
  };
  hipStream_t s = (hipStream_t)stream;
  const dim3 block(kDmaThreads + kComputeThreads);
  switch (variant) {
    case 11: hipLaunchKernelGGL(transpose_manual_double<272>, grid_for(4), block, 0, s, d_in, d_out, n, tiles, band); break;
    case 1: hipLaunchKernelGGL((transpose_single<true, true>), grid_for(1), block, 0, s, d_in, d_out, n, tiles, band); break;
    case 2: hipLaunchKernelGGL(transpose_manual_double<256>, grid_for(4), block, 0, s, d_in, d_out, n, tiles, band); break;
    case 3: hipLaunchKernelGGL(transpose_double_groups<272>, grid_for(4), block, 0, s, d_in, d_out, n, tiles, band); break;
    case 5: hipLaunchKernelGGL((transpose_double_groups<256, STORE_LDS_DIRECT_SWIZZLE>), grid_for(4), block, 0, s, d_in, d_out, n, tiles, band); break;
    case 6: hipLaunchKernelGGL((transpose_double_groups<256, STORE_LDS_SWIZZLE>), grid_for(4), block, 0, s, d_in, d_out, n, tiles, band); break;
    case 7: hipLaunchKernelGGL((transpose_manual_double<272, true>), grid_for(4), block, 0, s, d_in, d_out, n, tiles, band); break;
    case 8: hipLaunchKernelGGL(transpose_pairs<false>, grid_for(4), dim3(128), 0, s, d_in, d_out, n, tiles, band); break;
    case 9: hipLaunchKernelGGL(transpose_pairs<true>, grid_for(4), dim3(128), 0, s, d_in, d_out, n, tiles, band); break;
    case 0:
    case 10: {
      // variant 0 is the library's choice: the fastest split (three DMA wavefronts, one compute wavefront, one tile
      // ahead).  Variant 10 takes the split from the knob "transpose_split" = 100 * DMA wavefronts + 10 * compute
      // wavefronts + tiles ahead (the same default).
      const int code = variant == 0 ? 311 : workloads::tuning("transpose_split", 311);
      const SplitEntry* e = nullptr;
      for (const SplitEntry& c : kSplits)
        if (100 * c.dw + 10 * c.cw + c.ahead == code) e = &c;
      CUDADMA_REQUIRE(e != nullptr, "this build of the library holds no transposition kernel for the split %d (cudadma_transpose_splits lists "
                                       "those it holds; the rest are compiled with -DHIPDMA_SWEEP_VARIANTS)", code);
      hipLaunchKernelGGL(e->kernel, grid_for(1), dim3((e->dw + e->cw) * 64), 0, s, d_in, d_out, n, tiles, band);
      break;
    }
    case 14: hipLaunchKernelGGL((transpose_double_lds<3, 1>), grid_for(1), dim3(256), 0, s, d_in, d_out, n, tiles, band); break;
#ifdef HIPDMA_SWEEP_VARIANTS
    case 12:
    case 13: {
      // output rows written 1 KiB at a time; knobs: "transpose_wide_order" 1 = neighbouring tile columns first,
      // "transpose_wide_dma" = DMA wavefronts (3 by default; 2 or 4)
      const int order = workloads::tuning("transpose_wide_order", 1) - 1;
      const int dw = workloads::tuning("transpose_wide_dma", 3);
      const int passes = ((tiles_per_side + 3) / 4) * tiles_per_side;
      const dim3 g((unsigned)(forced > 0 ? (forced < passes ? forced : passes) : workloads::persistent_grid(passes, 1)));
      CUDADMA_REQUIRE(dw >= 2 && dw <= 4, "transpose_wide_dma: 2, 3 or 4 DMA wavefronts");
      if (variant == 12) {
        if (dw == 2) hipLaunchKernelGGL((transpose_wide_rows<2, 1>), g, dim3(192), 0, s, d_in, d_out, n, order);
        else if (dw == 3) hipLaunchKernelGGL((transpose_wide_rows<3, 1>), g, dim3(256), 0, s, d_in, d_out, n, order);
        else hipLaunchKernelGGL((transpose_wide_rows<4, 1>), g, dim3(320), 0, s, d_in, d_out, n, order);
      } else {
        if (dw == 2) hipLaunchKernelGGL((transpose_wide_rows<2, 2>), g, dim3(192), 0, s, d_in, d_out, n, order);
        else if (dw == 3) hipLaunchKernelGGL((transpose_wide_rows<3, 2>), g, dim3(256), 0, s, d_in, d_out, n, order);
        else hipLaunchKernelGGL((transpose_wide_rows<4, 2>), g, dim3(320), 0, s, d_in, d_out, n, order);
      }
      break;
    }
#else
    case 12:
    case 13: CUDADMA_REQUIRE(false, "variants 12 and 13 are sweep kernels: build the library with make EXTRA=-DHIPDMA_SWEEP_VARIANTS");
#endif
    default: hipLaunchKernelGGL(transpose_not_specialized, grid_for(1), block, 0, s, d_in, d_out, n, tiles, band); break;
  }
  CUDADMA_HIP_CHECK(hipGetLastError());
  return CUDADMA_OK;
}
