// Memory-system probes without LDS and without a DMA object: what a copy-shaped kernel can reach
// on this part, and what the placement of the blocks costs.  They give the yardsticks the
// transposition (config 2) is judged against; the reference has nothing of the kind (its sweep
// scripts, src/perf/sequential/param_sweep.py:27-58, only vary its own kernels).
//
// The block modes view both buffers as n x n float matrices cut into blocks of 64 rows x 256 B,
// the tile of config 2; a wavefront moves one block per step through registers (16 dwordx4 per
// lane in flight) and the wavefronts walk the blocks grid-stride.
#include "workloads.hpp"
#include <type_traits>

namespace {
using workloads::vec4_t;

constexpr int kThreads = 256;
constexpr int kBlockRows = 64;
constexpr int kSegBytes = 256;

__global__ void __launch_bounds__(kThreads)
probe_read(const vec4_t* __restrict__ in, vec4_t* __restrict__ sink, const size_t n_vec)
{
  vec4_t acc = {0u, 0u, 0u, 0u};
  const size_t stride = (size_t)gridDim.x * kThreads;
  size_t i = (size_t)blockIdx.x * kThreads + threadIdx.x;
  // four loads in flight per lane
  for (; i + 3 * stride < n_vec; i += 4 * stride) {
    const vec4_t a = in[i], b = in[i + stride], c = in[i + 2 * stride], d = in[i + 3 * stride];
    acc ^= a ^ b ^ c ^ d;
  }
  for (; i < n_vec; i += stride) acc ^= in[i];
  // never true for the benchmark data (finite floats); keeps the loads alive
  if ((acc.x & acc.y & acc.z & acc.w) == 0xffffffffu && sink != nullptr) sink[threadIdx.x] = acc;
}

template<bool NONTEMPORAL>
__global__ void __launch_bounds__(kThreads)
probe_write(vec4_t* __restrict__ out, const size_t n_vec)
{
  const vec4_t one = {0x3f800000u, 0x3f800000u, 0x3f800000u, 0x3f800000u};
  const size_t stride = (size_t)gridDim.x * kThreads;
  for (size_t i = (size_t)blockIdx.x * kThreads + threadIdx.x; i < n_vec; i += stride) {
    if constexpr (NONTEMPORAL) __builtin_nontemporal_store(one, out + i);
    else out[i] = one;
  }
}

template<bool NONTEMPORAL>
__global__ void __launch_bounds__(kThreads)
probe_copy(const vec4_t* __restrict__ in, vec4_t* __restrict__ out, const size_t n_vec)
{
  const size_t stride = (size_t)gridDim.x * kThreads;
  for (size_t i = (size_t)blockIdx.x * kThreads + threadIdx.x; i < n_vec; i += stride) {
    const vec4_t v = in[i];
    if constexpr (NONTEMPORAL) __builtin_nontemporal_store(v, out + i);
    else out[i] = v;
  }
}

enum Placement { kInPlace, kSwapped, kPermuted, kWriteOnlySwapped };

// Block b of the row-major block grid sits at block row b / blocks_per_row, block column b % blocks_per_row.
// kInPlace: written where it was read.  kSwapped: written at (block column, block row), the placement of a
// transposition (the 64 x 64 elements inside the block keep their order: this probe moves, it does not
// transpose).  kPermuted: written where it was read, but the blocks are visited in the order
// b -> (b * odd) mod number of blocks (a power of two).  kWriteOnlySwapped: no loads.
template<int PLACEMENT>
__global__ void __launch_bounds__(kThreads)
probe_blocks(const char* __restrict__ in, char* __restrict__ out, const size_t pitch, const size_t num_blocks,
             const int blocks_per_row)
{
  const int lane = threadIdx.x & 63;
  const size_t wave = (size_t)blockIdx.x * (kThreads / 64) + (threadIdx.x >> 6);
  const size_t waves = (size_t)gridDim.x * (kThreads / 64);
  const int seg = lane >> 4;                // four 256-byte segments per dwordx4 instruction
  const int off = (lane & 15) * 16;
  for (size_t b0 = wave; b0 < num_blocks; b0 += waves) {
    const size_t b = (PLACEMENT == kPermuted) ? ((b0 * 0x9E3779B1ull) & (num_blocks - 1)) : b0;
    const size_t brow = b / blocks_per_row, bcol = b % blocks_per_row;
    const char* src = in + brow * kBlockRows * pitch + bcol * kSegBytes;
    char* dst = (PLACEMENT == kSwapped || PLACEMENT == kWriteOnlySwapped)
                    ? out + bcol * kBlockRows * pitch + brow * kSegBytes
                    : out + brow * kBlockRows * pitch + bcol * kSegBytes;
    vec4_t v[kBlockRows / 4];
#pragma unroll
    for (int i = 0; i < kBlockRows / 4; ++i) {
      if constexpr (PLACEMENT == kWriteOnlySwapped) v[i] = vec4_t{0x3f800000u, 0x3f800000u, 0x3f800000u, 0x3f800000u};
      else v[i] = *(const vec4_t*)(src + (size_t)(i * 4 + seg) * pitch + off);
    }
#pragma unroll
    for (int i = 0; i < kBlockRows / 4; ++i) *(vec4_t*)(dst + (size_t)(i * 4 + seg) * pitch + off) = v[i];
  }
}

// The transposition itself without a DMA object and without any synchronisation between wavefronts:
// every wavefront brings its own block into a private LDS tile (rows padded to 272 B), reads it back
// row per lane, transposes 4 x 4 words inside each quad of lanes and writes dwordx4.  out = in^T.
__device__ __forceinline__ vec4_t probe_quad_transpose(const vec4_t a, const int lane)
{
  auto mv = [](const unsigned v, auto ctrl) { return (unsigned)__builtin_amdgcn_update_dpp(0, (int)v, decltype(ctrl)::value, 0xf, 0xf, false); };
  typedef std::integral_constant<int, 0x4E> pairs;   // quad_perm [2, 3, 0, 1]
  typedef std::integral_constant<int, 0xB1> lanes;   // quad_perm [1, 0, 3, 2]
  const bool upper = (lane & 2) != 0, odd = (lane & 1) != 0;
  const unsigned p0 = mv(a[0], pairs()), p1 = mv(a[1], pairs()), p2 = mv(a[2], pairs()), p3 = mv(a[3], pairs());
  const vec4_t b = {upper ? p2 : a[0], upper ? p3 : a[1], upper ? a[2] : p0, upper ? a[3] : p1};
  const unsigned q0 = mv(b[0], lanes()), q1 = mv(b[1], lanes()), q2 = mv(b[2], lanes()), q3 = mv(b[3], lanes());
  return vec4_t{odd ? q1 : b[0], odd ? b[1] : q0, odd ? q3 : b[2], odd ? b[3] : q2};
}

__global__ void __launch_bounds__(kThreads)
probe_transpose_private(const char* __restrict__ in, char* __restrict__ out, const size_t pitch, const size_t num_blocks,
                        const int blocks_per_row)
{
  constexpr int kLdsRow = kSegBytes + 16;
  __shared__ __attribute__((aligned(16))) char tiles[kThreads / 64][kBlockRows * kLdsRow];
  const int lane = threadIdx.x & 63;
  char* tile = tiles[threadIdx.x >> 6];
  const size_t wave = (size_t)blockIdx.x * (kThreads / 64) + (threadIdx.x >> 6);
  const size_t waves = (size_t)gridDim.x * (kThreads / 64);
  const int seg = lane >> 4, off = (lane & 15) * 16;
  for (size_t b = wave; b < num_blocks; b += waves) {
    const size_t brow = b / blocks_per_row, bcol = b % blocks_per_row;
    const char* src = in + brow * kBlockRows * pitch + bcol * kSegBytes;
    vec4_t v[kBlockRows / 4];
#pragma unroll
    for (int i = 0; i < kBlockRows / 4; ++i) v[i] = *(const vec4_t*)(src + (size_t)(i * 4 + seg) * pitch + off);
#pragma unroll
    for (int i = 0; i < kBlockRows / 4; ++i) *(vec4_t*)(tile + (i * 4 + seg) * kLdsRow + off) = v[i];
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    const vec4_t* row = (const vec4_t*)(tile + lane * kLdsRow);
#pragma unroll
    for (int j = 0; j < kBlockRows / 4; ++j) v[j] = row[j];
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    // lane 4q + i now gets rows 4q .. 4q+3 of block column 4j + i: four words of output row 4j + i
    char* dst = out + (bcol * kBlockRows + (lane & 3)) * pitch + brow * kSegBytes + (size_t)(lane & ~3) * 4;
#pragma unroll
    for (int j = 0; j < kBlockRows / 4; ++j) *(vec4_t*)(dst + (size_t)(4 * j) * pitch) = probe_quad_transpose(v[j], lane);
  }
}

}  // namespace

extern "C" long long cudadma_probe_memory(int mode, const void* d_src, void* d_dst, size_t bytes, int workgroups,
                                          void* stream)
{
  if (mode < 0 || mode >= CUDADMA_PROBE_MODES) {
    cudadma_host::set_error("no probe mode %d", mode);
    return CUDADMA_ERANGE;
  }
  CUDADMA_REQUIRE(bytes > 0 && (bytes % 16) == 0, "bytes must be a positive multiple of 16");
  CUDADMA_REQUIRE(workgroups > 0 && workgroups <= 65536, "workgroups must lie in 1..65536");
  const bool reads = mode != CUDADMA_PROBE_WRITE && mode != CUDADMA_PROBE_WRITE_NONTEMPORAL &&
                     mode != CUDADMA_PROBE_WRITE_BLOCKS_SWAPPED;
  const bool writes = mode != CUDADMA_PROBE_READ;
  CUDADMA_REQUIRE((!reads || d_src != nullptr) && (!writes || d_dst != nullptr), "NULL pointer");
  CUDADMA_REQUIRE((!reads || cudadma_host::aligned_to(d_src, 16)) && (!writes || cudadma_host::aligned_to(d_dst, 16)),
                  "pointers must be 16-byte aligned");
  hipStream_t s = (hipStream_t)stream;
  const dim3 grid((unsigned)workgroups), block(kThreads);
  const size_t n_vec = bytes / 16;
  const bool blocks = mode >= CUDADMA_PROBE_BLOCKS_IN_PLACE;
  size_t pitch = 0, num_blocks = 0;
  int blocks_per_row = 0;
  if (blocks) {
    // bytes = 4 n^2 with n a power of two of at least 64: the block count is then a power of two as well
    size_t n = 64;
    while (4 * n * n < bytes) n *= 2;
    CUDADMA_REQUIRE(4 * n * n == bytes, "the block modes need bytes = 4 n^2 with n a power of two >= 64 (got %zu)", bytes);
    pitch = 4 * n;
    blocks_per_row = (int)(pitch / kSegBytes);
    num_blocks = bytes / ((size_t)kBlockRows * kSegBytes);
  }
  const char* in = (const char*)d_src;
  char* out = (char*)d_dst;
  switch (mode) {
    case CUDADMA_PROBE_READ: hipLaunchKernelGGL(probe_read, grid, block, 0, s, (const vec4_t*)d_src, (vec4_t*)d_dst, n_vec); break;
    case CUDADMA_PROBE_WRITE: hipLaunchKernelGGL(probe_write<false>, grid, block, 0, s, (vec4_t*)d_dst, n_vec); break;
    case CUDADMA_PROBE_WRITE_NONTEMPORAL: hipLaunchKernelGGL(probe_write<true>, grid, block, 0, s, (vec4_t*)d_dst, n_vec); break;
    case CUDADMA_PROBE_COPY: hipLaunchKernelGGL(probe_copy<false>, grid, block, 0, s, (const vec4_t*)d_src, (vec4_t*)d_dst, n_vec); break;
    case CUDADMA_PROBE_COPY_NONTEMPORAL: hipLaunchKernelGGL(probe_copy<true>, grid, block, 0, s, (const vec4_t*)d_src, (vec4_t*)d_dst, n_vec); break;
    case CUDADMA_PROBE_BLOCKS_IN_PLACE: hipLaunchKernelGGL(probe_blocks<kInPlace>, grid, block, 0, s, in, out, pitch, num_blocks, blocks_per_row); break;
    case CUDADMA_PROBE_BLOCKS_SWAPPED: hipLaunchKernelGGL(probe_blocks<kSwapped>, grid, block, 0, s, in, out, pitch, num_blocks, blocks_per_row); break;
    case CUDADMA_PROBE_BLOCKS_PERMUTED: hipLaunchKernelGGL(probe_blocks<kPermuted>, grid, block, 0, s, in, out, pitch, num_blocks, blocks_per_row); break;
    case CUDADMA_PROBE_WRITE_BLOCKS_SWAPPED: hipLaunchKernelGGL(probe_blocks<kWriteOnlySwapped>, grid, block, 0, s, in, out, pitch, num_blocks, blocks_per_row); break;
    default: hipLaunchKernelGGL(probe_transpose_private, grid, block, 0, s, in, out, pitch, num_blocks, blocks_per_row); break;
  }
  CUDADMA_HIP_CHECK(hipGetLastError());
  return (long long)((reads ? bytes : 0) + (writes ? bytes : 0));
}
