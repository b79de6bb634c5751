/* CPU oracle: see oracle.h.  Plain C + OpenMP; TEST INFRASTRUCTURE ONLY. */
#include "oracle.h"

#include <math.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

int oracle_num_threads(void)
{
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}

/* ------------------------------------------------------------------ inputs */

/* Steele, Lea, Flood: "Fast splittable pseudorandom number generators" (2014),
 * the splitmix64 output function applied to x + golden gamma.  x = 0 gives the
 * generator's well-known first output for seed 0, 0xE220A8397B1DCDAF. */
uint64_t oracle_splitmix64(uint64_t x)
{
  uint64_t z = x + 0x9E3779B97F4A7C15ull;
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  return z ^ (z >> 31);
}

uint32_t oracle_hash32(uint64_t seed, uint64_t i) { return (uint32_t)(oracle_splitmix64(seed + i) >> 32); }

static inline float uniform_pm1(uint32_t h) { return (float)(h >> 8) * (1.0f / 8388608.0f) - 1.0f; }

void oracle_fill_uniform(float* dst, size_t n, uint64_t seed)
{
#pragma omp parallel for schedule(static)
  for (long long i = 0; i < (long long)n; ++i) dst[i] = uniform_pm1(oracle_hash32(seed, (uint64_t)i));
}

/* Input of the reference's known-answer tests:
 * src/tests/test_sequential/cudaDMA_test_sequential_v2.cu:416-418 */
void oracle_fill_ramp(float* dst, size_t n)
{
  for (size_t i = 0; i < n; ++i) dst[i] = (float)i;
}

/* Element indices uniform over [0, n_records); one position in ten (beyond the
 * first 1024) repeats the draw of a position up to 1024 places back. */
void oracle_fill_indices(int32_t* dst, size_t n, uint32_t n_records, uint64_t seed)
{
#pragma omp parallel for schedule(static)
  for (long long i = 0; i < (long long)n; ++i) {
    uint64_t j = (uint64_t)i;
    const uint32_t r = oracle_hash32(seed ^ 0x5bd1e995u, (uint64_t)i);
    if (i > 1024 && (r % 10u) == 0u) j = (uint64_t)i - 1u - ((r / 10u) % 1024u);
    dst[i] = (int32_t)(oracle_hash32(seed, j) % n_records);
  }
}

/* A permutation of [0, 2^log2_n): an odd multiplier, an added constant and a right xor-shift are
 * each one-to-one on log2_n bits.  States the generator the scatter workload draws its distinct
 * indices from (no counterpart in the reference, whose tests draw non-overlapping offsets with
 * srand/rand, src/tests/test_indirect/cudaDMA_test_indirect_v2.cu:721-760). */
void oracle_fill_permutation(int32_t* dst, int log2_n, uint64_t seed)
{
  const uint64_t n = (uint64_t)1 << log2_n, mask = n - 1;
  const uint64_t k0 = oracle_splitmix64(seed), k1 = oracle_splitmix64(seed + 1);
  const int h = (log2_n + 1) / 2;
#pragma omp parallel for schedule(static)
  for (long long i = 0; i < (long long)n; ++i) {
    uint64_t x = (uint64_t)i;
    x = (x * ((k0 & 0xffffffffu) | 1u) + (k0 >> 32)) & mask;
    x ^= x >> h;
    x = (x * ((k1 & 0xffffffffu) | 1u) + (k1 >> 32)) & mask;
    x ^= x >> h;
    x = (x * 0x9E3779B1u) & mask;
    dst[i] = (int32_t)x;
  }
}

uint16_t oracle_f32_to_bf16(float v)
{
  uint32_t u;
  memcpy(&u, &v, 4);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40u); /* quiet NaN */
  u += 0x7fffu + ((u >> 16) & 1u);                                            /* round to nearest even */
  return (uint16_t)(u >> 16);
}

float oracle_bf16_to_f32(uint16_t v)
{
  uint32_t u = (uint32_t)v << 16;
  float f;
  memcpy(&f, &u, 4);
  return f;
}

/* normal(0,1) by Box-Muller on two hashes, rounded to bf16 */
void oracle_fill_normal_bf16(uint16_t* dst, size_t n, uint64_t seed)
{
#pragma omp parallel for schedule(static)
  for (long long i = 0; i < (long long)n; ++i) {
    const double u1 = ((double)(oracle_hash32(seed, 2ull * (uint64_t)i) >> 8) + 1.0) / 16777216.0;
    const double u2 = (double)(oracle_hash32(seed, 2ull * (uint64_t)i + 1ull) >> 8) / 16777216.0;
    dst[i] = oracle_f32_to_bf16((float)(sqrt(-2.0 * log(u1)) * cos(6.283185307179586476925286766559 * u2)));
  }
}

/* -------------------------------------------------------- transfer patterns */

/* CudaDMASequential: dst[0..B) = src[0..B)
 * include/cudaDMAv2.h:1380-1400 (every byte offset below BYTES_PER_ELMT is
 * owned by exactly one thread), :1810-1841 (load at offset, store at the same offset). */
void oracle_sequential(const void* src, void* dst, size_t bytes)
{
  const unsigned char* s = (const unsigned char*)src;
  unsigned char* d = (unsigned char*)dst;
  for (size_t i = 0; i < bytes; ++i) d[i] = s[i];
}

/* CudaDMAStrided: NUM_ELMTS rows of BYTES_PER_ELMT bytes, independent strides.
 * include/cudaDMAv2.h:3098-3107 (row r starts at r*src_stride / r*dst_stride),
 * :8381-8393 and :8561-8573 (load_strided / store_strided walk both sides in step). */
void oracle_strided(const void* src, void* dst, int elmt_bytes, int num_elmts, int src_stride, int dst_stride)
{
  const unsigned char* s = (const unsigned char*)src;
  unsigned char* d = (unsigned char*)dst;
  for (int r = 0; r < num_elmts; ++r)
    for (int j = 0; j < elmt_bytes; ++j)
      d[(size_t)r * dst_stride + j] = s[(size_t)r * src_stride + j];
}

/* The swizzled LDS layout of CudaDMAStrided's STORE_LDS_SWIZZLE / STORE_LDS_DIRECT_SWIZZLE
 * qualifiers (an addition of this library, no reference lines): the same rows as
 * oracle_strided, with the chunks of destination row r permuted by XOR with key(r):
 *   span  = largest power of two dividing the chunks per row, at most 256 / chunk
 *   key   = the low log2(span) bits of r / (rows per 256-byte bank line), bit-reversed,
 *           rows per bank line = max(1, 256 / (span * chunk)). */
static int swizzle_key(int row, int chunks, int chunk)
{
  int span = 256 / chunk;
  while (span > 1 && (chunks % span) != 0) span >>= 1;
  if (chunks <= 0) span = 1;
  int rows_per_line = 256 / (span * chunk);
  if (rows_per_line < 1) rows_per_line = 1;
  int v = row / rows_per_line, key = 0;
  for (int bit = 1; bit < span; bit <<= 1) {
    key = (key << 1) | (v & 1);
    v >>= 1;
  }
  return key;
}

void oracle_strided_swizzled(const void* src, void* dst, int elmt_bytes, int num_elmts, int src_stride, int dst_stride,
                             int chunk)
{
  const unsigned char* s = (const unsigned char*)src;
  unsigned char* d = (unsigned char*)dst;
  const int chunks = elmt_bytes / chunk;
  for (int r = 0; r < num_elmts; ++r) {
    const int key = swizzle_key(r, chunks, chunk);
    for (int c = 0; c < chunks; ++c)
      for (int b = 0; b < chunk; ++b)
        d[(size_t)r * dst_stride + (size_t)((c ^ key) * chunk) + b] = s[(size_t)r * src_stride + (size_t)c * chunk + b];
  }
}

/* CudaDMAIndirect<GATHER=true>: row r comes from element index[r] of the source;
 * rows land max(alt_stride, elmt_bytes) apart.
 * include/cudaDMAv2.h:9940-9957 (offset = index_ptr[...]; src_ptr + offset*BYTES_PER_ELMT),
 * :9406 (SELECT_STRIDE). */
void oracle_gather(const int32_t* index, const void* src, void* dst, int elmt_bytes, int num_elmts, int alt_stride)
{
  const unsigned char* s = (const unsigned char*)src;
  unsigned char* d = (unsigned char*)dst;
  const int stride = alt_stride > elmt_bytes ? alt_stride : elmt_bytes;
  for (int r = 0; r < num_elmts; ++r)
    for (int j = 0; j < elmt_bytes; ++j)
      d[(size_t)r * stride + j] = s[(size_t)index[r] * elmt_bytes + j];
}

/* CudaDMAIndirect<GATHER=false>: row r of the (dense) source goes to element index[r].
 * include/cudaDMAv2.h:10199-10217. */
void oracle_scatter(const int32_t* index, const void* src, void* dst, int elmt_bytes, int num_elmts, int alt_stride)
{
  const unsigned char* s = (const unsigned char*)src;
  unsigned char* d = (unsigned char*)dst;
  const int stride = alt_stride > elmt_bytes ? alt_stride : elmt_bytes;
  for (int r = 0; r < num_elmts; ++r)
    for (int j = 0; j < elmt_bytes; ++j)
      d[(size_t)index[r] * elmt_bytes + j] = s[(size_t)r * stride + j];
}

/* cudaDMAHalo: ring of ghost cells around a dimx x dimy tile; origins at the
 * first interior cell; source pitch `pitch` cells, destination pitch dimx+2R cells.
 * include/cudaDMA.h:3616 (row width), :3718-3727 (pitches, top/bottom offsets),
 * :3746-3749 (side strips). */
void oracle_halo(const void* src_origin, void* dst_origin, int elmt_bytes, int radius, int corners,
                 int dimx, int dimy, int pitch)
{
  oracle_halo_pitched(src_origin, dst_origin, elmt_bytes, radius, corners, dimx, dimy, pitch, dimx + 2 * radius);
}

/* The same ring with the destination row pitch given in cells (>= dimx+2R): the layout the build's
 * CudaDMAHalo offers next to the reference's fixed one; dst_pitch = dimx+2R is the reference's. */
void oracle_halo_pitched(const void* src_origin, void* dst_origin, int elmt_bytes, int radius, int corners,
                         int dimx, int dimy, int pitch, int dst_pitch)
{
  const unsigned char* s = (const unsigned char*)src_origin;
  unsigned char* d = (unsigned char*)dst_origin;
  const ptrdiff_t sp = (ptrdiff_t)pitch * elmt_bytes;
  const ptrdiff_t dp = (ptrdiff_t)dst_pitch * elmt_bytes;
  const ptrdiff_t x0 = corners ? -(ptrdiff_t)radius * elmt_bytes : 0;
  const ptrdiff_t x1 = (ptrdiff_t)dimx * elmt_bytes + (corners ? (ptrdiff_t)radius * elmt_bytes : 0);
  for (int r = 0; r < radius; ++r) {
    const ptrdiff_t top = (ptrdiff_t)(r - radius), bot = (ptrdiff_t)(dimy + r);
    for (ptrdiff_t x = x0; x < x1; ++x) {
      d[top * dp + x] = s[top * sp + x];
      d[bot * dp + x] = s[bot * sp + x];
    }
  }
  for (int y = 0; y < dimy; ++y)
    for (ptrdiff_t x = 0; x < (ptrdiff_t)radius * elmt_bytes; ++x) {
      d[y * dp - (ptrdiff_t)radius * elmt_bytes + x] = s[y * sp - (ptrdiff_t)radius * elmt_bytes + x];
      d[y * dp + (ptrdiff_t)dimx * elmt_bytes + x] = s[y * sp + (ptrdiff_t)dimx * elmt_bytes + x];
    }
}

/* The reference's own halo checker, on bytes:
 * src/tests/test_halo/cudaDMA_test_halo.cu:91-164. */
int oracle_halo_check(const void* idata, const void* odata, int elmt_bytes, int radius, int corners,
                      int dimx, int dimy, int pitch)
{
  const unsigned char* in = (const unsigned char*)idata;
  const unsigned char* out = (const unsigned char*)odata;
  const size_t es = (size_t)elmt_bytes;
  const size_t opitch = (size_t)(dimx + 2 * radius);
  const int row_cells = dimx + (corners ? 2 * radius : 0);
  const size_t row_skip = corners ? 0 : (size_t)radius;
  for (int i = 0; i < radius; ++i) { /* top rows */
    const unsigned char* s = in + ((size_t)i * pitch + row_skip) * es;
    const unsigned char* d = out + ((size_t)i * opitch + row_skip) * es;
    if (memcmp(s, d, (size_t)row_cells * es) != 0) return 0;
  }
  for (int i = 0; i < radius; ++i) { /* bottom rows */
    const unsigned char* s = in + ((size_t)(radius + dimy + i) * pitch + row_skip) * es;
    const unsigned char* d = out + ((size_t)(radius + dimy + i) * opitch + row_skip) * es;
    if (memcmp(s, d, (size_t)row_cells * es) != 0) return 0;
  }
  for (int i = 0; i < dimy; ++i) { /* left and right panels */
    const unsigned char* s = in + (size_t)(radius + i) * pitch * es;
    const unsigned char* d = out + (size_t)(radius + i) * opitch * es;
    if (memcmp(s, d, (size_t)radius * es) != 0) return 0;
    if (memcmp(s + (size_t)(radius + dimx) * es, d + (size_t)(radius + dimx) * es, (size_t)radius * es) != 0) return 0;
  }
  return 1;
}

/* ----------------------------------------------------------------- workloads */

/* Config 1: tiled copy through LDS; as a whole, out == in. */
void oracle_copy(const float* in, float* out, size_t n)
{
#pragma omp parallel for schedule(static)
  for (long long i = 0; i < (long long)n; ++i) out[i] = in[i];
}

/* Config 2: out = in^T for an n x n row-major matrix.  Two levels of blocking: 256 x 256
 * tiles keep the pages touched on both sides within the reach of the TLB, and inside a tile
 * 16 x 16 blocks go through a local buffer so that every cache line of the input is read
 * once and every cache line of the output is written once and whole (with a power-of-two
 * row pitch the rows of a block fall into the same cache set: a line must not be revisited). */
void oracle_transpose(const float* in, float* out, int n)
{
  enum { T = 256, B = 16 };
  const int nt = (n + T - 1) / T;
#pragma omp parallel for collapse(2) schedule(static)
  for (int tr = 0; tr < nt; ++tr)
    for (int tc = 0; tc < nt; ++tc) {
      const int r_end = (tr * T + T < n) ? tr * T + T : n, c_end = (tc * T + T < n) ? tc * T + T : n;
      for (int r0 = tr * T; r0 < r_end; r0 += B)
        for (int c0 = tc * T; c0 < c_end; c0 += B) {
          float tmp[B][B];
          const int nr = (r_end - r0 < B) ? r_end - r0 : B, nc = (c_end - c0 < B) ? c_end - c0 : B;
          for (int r = 0; r < nr; ++r)
            for (int c = 0; c < nc; ++c) tmp[r][c] = in[(size_t)(r0 + r) * n + (size_t)(c0 + c)];
          for (int c = 0; c < nc; ++c)
            for (int r = 0; r < nr; ++r) out[(size_t)(c0 + c) * n + (size_t)(r0 + r)] = tmp[r][c];
        }
    }
}

/* Config 3, record check: out[i] = table[idx[i]] */
void oracle_gather_copy(const float* table, const int32_t* idx, float* out, size_t n_idx, int rec_floats)
{
#pragma omp parallel for schedule(static)
  for (long long i = 0; i < (long long)n_idx; ++i)
    memcpy(out + (size_t)i * rec_floats, table + (size_t)idx[i] * rec_floats, (size_t)rec_floats * sizeof(float));
}

/* The scatter workload: table[idx[i]] = records[i] (addressing of include/cudaDMAv2.h:10199-10217
 * with the dense side packed).  Indices are distinct, so the iterations are independent. */
void oracle_scatter_copy(const float* records, const int32_t* idx, float* table, size_t n_idx, int rec_floats)
{
#pragma omp parallel for schedule(static)
  for (long long i = 0; i < (long long)n_idx; ++i)
    memcpy(table + (size_t)idx[i] * rec_floats, records + (size_t)i * rec_floats, (size_t)rec_floats * sizeof(float));
}

/* Config 3, headline consumer: out[t][j] = sum over the recs_per_tile records of
 * tile t of word j, added in ascending record order starting from record 0. */
void oracle_gather_rowsum(const float* table, const int32_t* idx, float* out, size_t n_idx, int rec_floats,
                          int recs_per_tile)
{
  const long long tiles = (long long)(n_idx / (size_t)recs_per_tile);
#pragma omp parallel for schedule(static)
  for (long long t = 0; t < tiles; ++t)
    for (int j = 0; j < rec_floats; ++j) {
      float acc = table[(size_t)idx[t * recs_per_tile] * rec_floats + j];
      for (int r = 1; r < recs_per_tile; ++r)
        acc = acc + table[(size_t)idx[t * recs_per_tile + r] * rec_floats + j];
      out[t * rec_floats + j] = acc;
    }
}

/* Config 4: 8th-order, 25-point star stencil (second derivative in each axis).
 * `in` is a (nx+2p) x (ny+2p) x (nz+2p) array (x fastest) with p = radius_pad >= 4;
 * `out` is nx x ny x nz.  Fixed evaluation order:
 *   acc = c0 * centre; for r = 1..4: acc = fma(c[r], ((xm + xp) + (ym + yp)) + (zm + zp), acc)
 * with every other operation rounded on its own (no contraction). */
void oracle_stencil25(const float* in, float* out, int nx, int ny, int nz, int radius_pad)
{
  const float c0 = (float)(3.0 * (-205.0 / 72.0));
  const float c[5] = {0.0f, (float)(8.0 / 5.0), (float)(-1.0 / 5.0), (float)(8.0 / 315.0), (float)(-1.0 / 560.0)};
  const int p = radius_pad;
  const size_t px = (size_t)nx + 2 * p, py = (size_t)ny + 2 * p;
#pragma omp parallel for collapse(2) schedule(static)
  for (int z = 0; z < nz; ++z)
    for (int y = 0; y < ny; ++y)
      for (int x = 0; x < nx; ++x) {
        const size_t o = ((size_t)(z + p) * py + (size_t)(y + p)) * px + (size_t)(x + p);
        float acc = c0 * in[o];
        for (int r = 1; r <= 4; ++r) {
          const float sx = in[o - r] + in[o + r];
          const float sy = in[o - r * px] + in[o + r * px];
          const float sz = in[o - r * px * py] + in[o + r * px * py];
          acc = fmaf(c[r], (sx + sy) + sz, acc);
        }
        out[((size_t)z * ny + y) * nx + x] = acc;
      }
}

/* Config 5: C = A * B, A m x k and B k x n row-major bf16, fp32 products of the
 * rounded inputs accumulated in fp32 in ascending k. */
void oracle_gemm_bf16(const uint16_t* a, const uint16_t* b, float* c, int m, int n, int k)
{
#pragma omp parallel for schedule(static)
  for (int i = 0; i < m; ++i) {
    float* crow = c + (size_t)i * n;
    for (int j = 0; j < n; ++j) crow[j] = 0.0f;
    for (int kk = 0; kk < k; ++kk) {
      const float av = oracle_bf16_to_f32(a[(size_t)i * k + kk]);
      const uint16_t* brow = b + (size_t)kk * n;
      for (int j = 0; j < n; ++j) crow[j] += av * oracle_bf16_to_f32(brow[j]);
    }
  }
}

float oracle_gemm_bf16_entry(const uint16_t* a, const uint16_t* b, int n, int k, int row, int col)
{
  float acc = 0.0f;
  for (int kk = 0; kk < k; ++kk)
    acc += oracle_bf16_to_f32(a[(size_t)row * k + kk]) * oracle_bf16_to_f32(b[(size_t)kk * n + col]);
  return acc;
}

/* ---- consumers of the reference's example programs ---- */

/* saxpy (src/examples/saxpy/saxpy_cudaDMA_kernel.cu:55-59, gold loop saxpy_cudaDMA.cu:66-72).
 * The device compiler of the reference contracts a*x+y into one fused operation; the
 * oracle states that rounding explicitly. */
void oracle_saxpy(float a, const float* x, float* y, size_t n)
{
#pragma omp parallel for schedule(static)
  for (size_t i = 0; i < n; ++i) y[i] = fmaf(a, x[i], y[i]);
}

/* sgemv, "n" form (src/examples/sgemv/sgemv_dma.cu:140-175; host check :752-771): thread `i`
 * walks row i of a column-major matrix, res += A[i + j*lda] * x[j] for ascending j starting
 * from 0.0f, one fused multiply-add per term, then y[i] = alpha * res. */
void oracle_sgemv(int n, int m, float alpha, const float* a, int lda, const float* x, float* y)
{
#pragma omp parallel for schedule(static)
  for (int i = 0; i < n; ++i) {
    float res = 0.0f;
    for (int j = 0; j < m; ++j) res = fmaf(a[(size_t)i + (size_t)j * lda], x[j], res);
    y[i] = alpha * res;
  }
}

/* 2-D cross average of the stencil example (src/examples/stencil/stencil_math.h:52-84), on
 * float2 elements (two independent components).  Order of the additions: centre, then the
 * -x arm for d = 1..reach, the +x arm, the -y arm, the +y arm; the sum is divided by
 * 4*radius + 1.  The reference's loops run d < RADIUS, i.e. reach = radius - 1, while the
 * divisor stays 4*radius + 1; callers pass reach = radius - 1 to state exactly that.
 * Layout (cudaDMA_stencil2D.cu:86-101): (dimx+2r) x (dimy+2r) x (dimz+2r) elements, row
 * stride dimx+2r, slice stride (dimy+2r)*(dimx+2r); slices r .. r+dimz-1 are processed and
 * only interior points of dst are written. */
void oracle_stencil2d(const float* src, float* dst, int dimx, int dimy, int dimz, int radius, int reach)
{
  const size_t row = (size_t)dimx + 2 * radius;
  const size_t slice = ((size_t)dimy + 2 * radius) * row;
  const float div = (float)(4 * radius + 1);
#pragma omp parallel for collapse(2) schedule(static)
  for (int z = 0; z < dimz; ++z)
    for (int y = 0; y < dimy; ++y)
      for (int x = 0; x < dimx; ++x) {
        const size_t o = (size_t)(z + radius) * slice + (size_t)(y + radius) * row + (size_t)(x + radius);
        for (int c = 0; c < 2; ++c) {
          float acc = src[2 * o + c];
          for (int d = 1; d <= reach; ++d) acc += src[2 * (o - d) + c];
          for (int d = 1; d <= reach; ++d) acc += src[2 * (o + d) + c];
          for (int d = 1; d <= reach; ++d) acc += src[2 * (o - d * row) + c];
          for (int d = 1; d <= reach; ++d) acc += src[2 * (o + d * row) + c];
          dst[2 * o + c] = acc / div;
        }
      }
}
