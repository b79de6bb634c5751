// Yardsticks shaped like the patterns' own memory accesses, without LDS and without a DMA object: what the
// addresses of the gather, the scatter and the tile transposition cost on this part when nothing but loads and
// stores stands between them and memory.  The benchmark runs them on the patterns' own buffers in the same run
// and reports each pattern as a fraction of its yardstick.  The reference has nothing of the kind (its sweep
// scripts, src/perf/sequential/param_sweep.py:27-58, only vary its own kernels).
#include "workloads.hpp"

namespace {
using workloads::vec4_t;

constexpr int kThreads = 256;
constexpr int kRecBytes = 128;                 // one record: 8 lanes x 16 B
constexpr int kRecsPerTile = 32;               // a wavefront takes 32 records at a time: 4 loads of 8 records
constexpr int kTile = 64;                      // tile side of the transposition, in floats

// xor over the 8 lanes that hold the same 16-byte column of different records (lanes l, l+8, ..., l+56)
__device__ __forceinline__ vec4_t xor_over_records(vec4_t v)
{
#pragma unroll
  for (int shift = 8; shift < 64; shift <<= 1) {
#pragma unroll
    for (int w = 0; w < 4; ++w) v[w] ^= (unsigned)__shfl_xor((int)v[w], shift, 64);
  }
  return v;
}

// d_out[t][j] = xor over r < 32 of d_table[d_idx[32 t + r]][j]: the index words and records the gather reads and the
// 128 bytes per tile it writes, fetched straight into registers.  Tiles are dealt round-robin to the wavefronts.
__global__ void __launch_bounds__(kThreads)
probe_gather_xor(const vec4_t* __restrict__ table, const int* __restrict__ idx, vec4_t* __restrict__ out, const size_t n_tiles)
{
  const int lane = threadIdx.x & 63;
  const size_t wave = (size_t)blockIdx.x * (kThreads / 64) + (threadIdx.x >> 6);
  const size_t waves = (size_t)gridDim.x * (kThreads / 64);
  const int rec = lane >> 3, col = lane & 7;
  for (size_t t = wave; t < n_tiles; t += waves) {
    const int* ix = idx + t * kRecsPerTile + rec;
    const int i0 = __builtin_nontemporal_load(ix), i1 = __builtin_nontemporal_load(ix + 8);
    const int i2 = __builtin_nontemporal_load(ix + 16), i3 = __builtin_nontemporal_load(ix + 24);
    const vec4_t a = table[(size_t)i0 * 8 + col], b = table[(size_t)i1 * 8 + col];
    const vec4_t c = table[(size_t)i2 * 8 + col], d = table[(size_t)i3 * 8 + col];
    const vec4_t x = xor_over_records(a ^ b ^ c ^ d);
    if (lane < 8) __builtin_nontemporal_store(x, out + t * 8 + lane);
  }
}

// d_table[d_idx[i]] = d_records[i]: the scatter's dense reads and indexed 128-byte writes from registers.
__global__ void __launch_bounds__(kThreads)
probe_scatter(const vec4_t* __restrict__ records, const int* __restrict__ idx, vec4_t* __restrict__ table, const size_t n_tiles)
{
  const int lane = threadIdx.x & 63;
  const size_t wave = (size_t)blockIdx.x * (kThreads / 64) + (threadIdx.x >> 6);
  const size_t waves = (size_t)gridDim.x * (kThreads / 64);
  const int rec = lane >> 3, col = lane & 7;
  for (size_t t = wave; t < n_tiles; t += waves) {
    const int* ix = idx + t * kRecsPerTile + rec;
    const vec4_t* src = records + t * (kRecsPerTile * 8) + lane;
    const int i0 = __builtin_nontemporal_load(ix), i1 = __builtin_nontemporal_load(ix + 8);
    const int i2 = __builtin_nontemporal_load(ix + 16), i3 = __builtin_nontemporal_load(ix + 24);
    const vec4_t a = __builtin_nontemporal_load(src), b = __builtin_nontemporal_load(src + 64);
    const vec4_t c = __builtin_nontemporal_load(src + 128), d = __builtin_nontemporal_load(src + 192);
    __builtin_nontemporal_store(a, table + (size_t)i0 * 8 + col);
    __builtin_nontemporal_store(b, table + (size_t)i1 * 8 + col);
    __builtin_nontemporal_store(c, table + (size_t)i2 * 8 + col);
    __builtin_nontemporal_store(d, table + (size_t)i3 * 8 + col);
  }
}

// The tiles of the transposition in its own order (workgroup b takes tiles b, b + G, ...; tile t lies in tile row
// t mod tiles_per_side and tile column t / tiles_per_side): chunk s of a tile is 16 bytes of row s / 16.
__device__ __forceinline__ void tile_of(const size_t t, const int tiles_per_side, int& ty, int& tx)
{ tx = (int)(t / tiles_per_side); ty = (int)(t - (size_t)tx * tiles_per_side); }

// Reads every source tile (64 rows x 256 B, rows n floats apart) and writes one xor of its 16-byte chunks per
// workgroup: the read half of the transposition alone.
__global__ void __launch_bounds__(kThreads)
probe_tile_read(const float* __restrict__ in, vec4_t* __restrict__ out, const int n, const size_t tiles)
{
  __shared__ vec4_t part[kThreads / 64];
  const int tiles_per_side = n / kTile;
  vec4_t acc = {0u, 0u, 0u, 0u};
  for (size_t t = blockIdx.x; t < tiles; t += gridDim.x) {
    int ty, tx;
    tile_of(t, tiles_per_side, ty, tx);
    const float* base = in + (size_t)ty * kTile * n + (size_t)tx * kTile;
    vec4_t v[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const int s = threadIdx.x + k * kThreads;
      v[k] = __builtin_nontemporal_load((const vec4_t*)(base + (size_t)(s >> 4) * n + (s & 15) * 4));
    }
    acc ^= v[0] ^ v[1] ^ v[2] ^ v[3];
  }
#pragma unroll
  for (int shift = 1; shift < 64; shift <<= 1) {
#pragma unroll
    for (int w = 0; w < 4; ++w) acc[w] ^= (unsigned)__shfl_xor((int)acc[w], shift, 64);
  }
  if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = acc;
  __syncthreads();
  if (threadIdx.x == 0) out[blockIdx.x] = part[0] ^ part[1] ^ part[2] ^ part[3];
}

// Writes every destination tile of the transposition in the same order (tile (ty, tx) of the source lands on rows
// 64 tx .. 64 tx + 63, columns 64 ty .. 64 ty + 63 of the output): the write half alone.  Element (r, c) of the
// output receives the 32-bit pattern r * n + c.
// PIECE: bytes of a row that one workgroup writes per turn (256 = one tile; 512 .. 4096 = as many tiles side by side).
// xcd_group: the workgroups of one XCD (every eighth workgroup) take neighbouring pieces instead of every eighth one.
template<int PIECE>
__global__ void __launch_bounds__(kThreads)
probe_tile_write(vec4_t* __restrict__ out, const int n, const size_t blocks, const int xcd_group)
{
  constexpr int kChunksPerRow = PIECE / 16;
  constexpr int kTurns = kTile * kChunksPerRow / kThreads;
  const int pieces_per_row = n * 4 / PIECE;
  const unsigned g = gridDim.x;
  const unsigned b = (xcd_group && (g % 8) == 0) ? (blockIdx.x % 8) * (g / 8) + blockIdx.x / 8 : blockIdx.x;
  for (size_t t = b; t < blocks; t += g) {
    const size_t rb = t / pieces_per_row, cb = t - rb * pieces_per_row;
#pragma unroll
    for (int k = 0; k < kTurns; ++k) {
      const int s = threadIdx.x + k * kThreads;
      const size_t r = rb * kTile + s / kChunksPerRow, c = cb * (PIECE / 4) + (s % kChunksPerRow) * 4;
      const unsigned first = (unsigned)(r * n + c);
      const vec4_t v = {first, first + 1u, first + 2u, first + 3u};
      __builtin_nontemporal_store(v, out + (r * n + c) / 4);
    }
  }
}

// Reads half of a buffer: the 256-byte granules whose index has even parity under `mask`, four loads in flight per
// lane, and writes one xor of the chunks per workgroup.  When the parity of those address bits picks half of the
// memory channels the rate halves; when the bits play no part in the choice of the channel it stays.
__global__ void __launch_bounds__(kThreads)
probe_masked_read(const vec4_t* __restrict__ in, vec4_t* __restrict__ out, const unsigned long long half_granules, const unsigned mask,
                  const int top_bit)
{
  __shared__ vec4_t part[kThreads / 64];
  const unsigned long long lanes = (unsigned long long)gridDim.x * kThreads, total = half_granules * 16;
  // the k-th granule of even parity: k with a bit inserted at the mask's top bit that makes the parity even
  auto chunk_of = [&](const unsigned long long t) {
    const unsigned long long k = t >> 4, low = k & ((1ull << top_bit) - 1), high = k >> top_bit;
    unsigned long long g = (high << (top_bit + 1)) | low;
    g |= (unsigned long long)(__popcll(g & mask) & 1) << top_bit;
    return in + g * 16 + (t & 15);
  };
  vec4_t acc = {0u, 0u, 0u, 0u};
  unsigned long long t = (unsigned long long)blockIdx.x * kThreads + threadIdx.x;
  for (; t + 3 * lanes < total; t += 4 * lanes) {
    const vec4_t a = __builtin_nontemporal_load(chunk_of(t)), b = __builtin_nontemporal_load(chunk_of(t + lanes));
    const vec4_t c = __builtin_nontemporal_load(chunk_of(t + 2 * lanes)), d = __builtin_nontemporal_load(chunk_of(t + 3 * lanes));
    acc ^= a ^ b ^ c ^ d;
  }
  for (; t < total; t += lanes) acc ^= __builtin_nontemporal_load(chunk_of(t));
#pragma unroll
  for (int shift = 1; shift < 64; shift <<= 1) {
#pragma unroll
    for (int w = 0; w < 4; ++w) acc[w] ^= (unsigned)__shfl_xor((int)acc[w], shift, 64);
  }
  if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = acc;
  __syncthreads();
  if (threadIdx.x == 0) out[blockIdx.x] = part[0] ^ part[1] ^ part[2] ^ part[3];
}

// Reads and writes together with the addresses of the transposition but without transposing inside a tile:
// out[64 tx + r][64 ty + c] = in[64 ty + r][64 tx + c].  A workgroup turn moves 16 KB: ROWS = 16 KB / PIECE rows of
// PIECE / 256 tiles that lie side by side in the output (one below the other in the source), so a wavefront's store
// covers PIECE contiguous bytes of an output row (up to 1 KiB) and its load 256-byte pieces of PIECE / 256 source
// tiles.  PIECE = 256 is the transposition's own shape: whole tiles, loads and stores of four rows x 256 B.
template<int PIECE>
__global__ void __launch_bounds__(kThreads)
probe_tile_copy(const float* __restrict__ in, float* __restrict__ out, const int n, const size_t turns, const int xcd_group)
{
  constexpr int kChunksPerRow = PIECE / 16;
  constexpr int kRows = 16384 / PIECE;              // rows per turn
  constexpr int kSubs = kTile / kRows;              // turns per block of 64 output rows
  const int pieces_per_row = n * 4 / PIECE;
  const unsigned g = gridDim.x;
  const unsigned b = (xcd_group && (g % 8) == 0) ? (blockIdx.x % 8) * (g / 8) + blockIdx.x / 8 : blockIdx.x;
  for (size_t t = b; t < turns; t += g) {
    // the turns of one (row block, piece) follow each other in the same workgroup's sequence only when g divides
    // accordingly; the order is: piece fastest, then sub-block, then row block
    const size_t cb = t % pieces_per_row, rest = t / pieces_per_row;
    const int sub = (int)(rest % kSubs);
    const size_t rb = rest / kSubs;
    vec4_t v[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const int s = threadIdx.x + k * kThreads;
      const int row = sub * kRows + s / kChunksPerRow, j = s % kChunksPerRow;
      const size_t ty = cb * (PIECE / 256) + j / 16;
      v[k] = __builtin_nontemporal_load((const vec4_t*)(in + (ty * kTile + row) * n + rb * kTile + (j % 16) * 4));
    }
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const int s = threadIdx.x + k * kThreads;
      const int row = sub * kRows + s / kChunksPerRow, j = s % kChunksPerRow;
      __builtin_nontemporal_store(v[k], (vec4_t*)(out + (rb * kTile + row) * n + cb * (PIECE / 4) + j * 4));
    }
  }
}

}  // namespace

extern "C" long long cudadma_probe_pattern(int mode, const void* d_in, const int32_t* d_idx, void* d_out, size_t n,
                                           size_t n_records, int workgroups, void* stream)
{
  if (mode < 0 || mode >= CUDADMA_PATTERN_PROBE_MODES) {
    cudadma_host::set_error("no pattern probe mode %d", mode);
    return CUDADMA_ERANGE;
  }
  CUDADMA_REQUIRE(workgroups > 0 && workgroups <= 65536, "workgroups must lie in 1..65536");
  CUDADMA_REQUIRE(d_out != nullptr && cudadma_host::aligned_to(d_out, 16), "d_out must be a 16-byte aligned device pointer");
  hipStream_t s = (hipStream_t)stream;
  const dim3 grid((unsigned)workgroups), block(kThreads);
  long long moved = 0;
  if (mode == CUDADMA_PATTERN_PROBE_GATHER_XOR || mode == CUDADMA_PATTERN_PROBE_SCATTER) {
    CUDADMA_REQUIRE(n > 0 && (n % kRecsPerTile) == 0, "n (the number of indices) must be a positive multiple of 32");
    CUDADMA_REQUIRE(n_records > 0 && n_records <= 0x7fffffffu, "n_records must lie in 1..2^31-1");
    CUDADMA_REQUIRE(d_in != nullptr && d_idx != nullptr && cudadma_host::aligned_to(d_in, 16) && cudadma_host::aligned_to(d_idx, 4),
                    "NULL or misaligned pointer");
    const size_t n_tiles = n / kRecsPerTile;
    if (mode == CUDADMA_PATTERN_PROBE_GATHER_XOR) {
      hipLaunchKernelGGL(probe_gather_xor, grid, block, 0, s, (const vec4_t*)d_in, d_idx, (vec4_t*)d_out, n_tiles);
      moved = (long long)(n * (4 + kRecBytes) + n_tiles * kRecBytes);
    } else {
      hipLaunchKernelGGL(probe_scatter, grid, block, 0, s, (const vec4_t*)d_in, d_idx, (vec4_t*)d_out, n_tiles);
      moved = (long long)(n * (4 + 2 * kRecBytes));
    }
  } else if (mode == CUDADMA_PATTERN_PROBE_MASKED_READ) {
    // n: bytes of the buffer (a power of two, at least 64 KiB); n_records: the mask over the index of the 256-byte granules
    CUDADMA_REQUIRE(n >= 65536 && (n & (n - 1)) == 0, "n (the bytes of the buffer) must be a power of two, at least 64 KiB");
    CUDADMA_REQUIRE(n_records > 0 && n_records < n / 256, "n_records (the mask over the granule index) must name bits inside the buffer");
    CUDADMA_REQUIRE(d_in != nullptr && cudadma_host::aligned_to(d_in, 256), "d_in must be a 256-byte aligned device pointer");
    const unsigned mask = (unsigned)n_records;
    hipLaunchKernelGGL(probe_masked_read, grid, block, 0, s, (const vec4_t*)d_in, (vec4_t*)d_out, (unsigned long long)(n / 512), mask,
                       31 - __builtin_clz(mask));
    moved = (long long)(n / 2);
  } else {
    CUDADMA_REQUIRE(n > 0 && (n % kTile) == 0 && n * 4 <= 0x7fffffffu, "n (the matrix side) must be a positive multiple of 64 with rows below 2 GiB");
    const size_t tiles = (n / kTile) * (n / kTile);
    if (mode == CUDADMA_PATTERN_PROBE_TILE_READ) {
      CUDADMA_REQUIRE(d_in != nullptr && cudadma_host::aligned_to(d_in, 16), "d_in must be a 16-byte aligned device pointer");
      hipLaunchKernelGGL(probe_tile_read, grid, block, 0, s, (const float*)d_in, (vec4_t*)d_out, (int)n, tiles);
    } else if (mode == CUDADMA_PATTERN_PROBE_TILE_WRITE) {
      // experiment knobs: bytes of a row per workgroup turn (default 256: one tile) and XCD grouping
      const int piece = workloads::tuning("probe_piece_bytes", 256);
      const int xg = workloads::tuning("probe_xcd_group", 0);
      CUDADMA_REQUIRE((n * 4) % (size_t)piece == 0, "the row must be a multiple of the piece");
      const size_t blocks = (n / kTile) * (n * 4 / piece);
      switch (piece) {
        case 256: hipLaunchKernelGGL(probe_tile_write<256>, grid, block, 0, s, (vec4_t*)d_out, (int)n, blocks, xg); break;
        case 512: hipLaunchKernelGGL(probe_tile_write<512>, grid, block, 0, s, (vec4_t*)d_out, (int)n, blocks, xg); break;
        case 1024: hipLaunchKernelGGL(probe_tile_write<1024>, grid, block, 0, s, (vec4_t*)d_out, (int)n, blocks, xg); break;
        case 2048: hipLaunchKernelGGL(probe_tile_write<2048>, grid, block, 0, s, (vec4_t*)d_out, (int)n, blocks, xg); break;
        case 4096: hipLaunchKernelGGL(probe_tile_write<4096>, grid, block, 0, s, (vec4_t*)d_out, (int)n, blocks, xg); break;
        default: CUDADMA_REQUIRE(false, "probe_piece_bytes: 256, 512, 1024, 2048 or 4096");
      }
    }
    moved = (long long)(n * n * 4);
    if (mode == CUDADMA_PATTERN_PROBE_TILE_COPY) {
      CUDADMA_REQUIRE(d_in != nullptr && cudadma_host::aligned_to(d_in, 16) && d_in != d_out, "d_in must be a 16-byte aligned device pointer other than d_out");
      const int piece = workloads::tuning("probe_piece_bytes", 256);
      const int xg = workloads::tuning("probe_xcd_group", 0);
      CUDADMA_REQUIRE((n * 4) % (size_t)piece == 0, "the row must be a multiple of the piece");
      const size_t turns = n * n * 4 / 16384;
      switch (piece) {
        case 256: hipLaunchKernelGGL(probe_tile_copy<256>, grid, block, 0, s, (const float*)d_in, (float*)d_out, (int)n, turns, xg); break;
        case 512: hipLaunchKernelGGL(probe_tile_copy<512>, grid, block, 0, s, (const float*)d_in, (float*)d_out, (int)n, turns, xg); break;
        case 1024: hipLaunchKernelGGL(probe_tile_copy<1024>, grid, block, 0, s, (const float*)d_in, (float*)d_out, (int)n, turns, xg); break;
        case 2048: hipLaunchKernelGGL(probe_tile_copy<2048>, grid, block, 0, s, (const float*)d_in, (float*)d_out, (int)n, turns, xg); break;
        case 4096: hipLaunchKernelGGL(probe_tile_copy<4096>, grid, block, 0, s, (const float*)d_in, (float*)d_out, (int)n, turns, xg); break;
        default: CUDADMA_REQUIRE(false, "probe_piece_bytes: 256, 512, 1024, 2048 or 4096");
      }
      moved *= 2;
    }
  }
  CUDADMA_HIP_CHECK(hipGetLastError());
  return moved;
}
