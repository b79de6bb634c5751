/* CPU oracle for the hipDMA transfer patterns and the five benchmark workloads.
 *
 * TEST INFRASTRUCTURE ONLY.  Nothing that ships (the headers under include/,
 * libcudadma_amd.so, the cudadma_amd package) links, loads or calls this
 * library; only tests/, __graft_entry__.smoke() and the cpu_baseline leg of
 * bench.py do, as the checker.
 *
 * Every transfer function restates, as a plain loop over bytes, what one DMA
 * object of the reference moves; the citation names the reference lines the
 * statement is taken from.  The reference cannot be compiled here (CUDA with
 * inline PTX), so each function is pinned in tests/test_oracle.py against the
 * expectations of the reference's own tests (ramp input + exact compare,
 * check_halo), against library routines it must reduce to (memcpy, numpy
 * slicing / take / transpose / matmul) and against brute-force byte maps.
 * Parity status: all functions below are pinned that way; none is "parity
 * unpinned".
 */
#ifndef HIPDMA_ORACLE_H
#define HIPDMA_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

int oracle_num_threads(void);

/* ---- seeded, counter-based inputs ---- */
uint64_t oracle_splitmix64(uint64_t x);
uint32_t oracle_hash32(uint64_t seed, uint64_t i);            /* splitmix64(seed + i) >> 32 */
void oracle_fill_uniform(float* dst, size_t n, uint64_t seed);/* (h >> 8) * 2^-23 - 1, in [-1,1) */
void oracle_fill_ramp(float* dst, size_t n);                  /* dst[i] = (float)i, as the reference tests */
void oracle_fill_indices(int32_t* dst, size_t n, uint32_t n_records, uint64_t seed);
void oracle_fill_permutation(int32_t* dst, int log2_n, uint64_t seed);  /* of [0, 2^log2_n) */
void oracle_fill_normal_bf16(uint16_t* dst, size_t n, uint64_t seed);
uint16_t oracle_f32_to_bf16(float v);
float oracle_bf16_to_f32(uint16_t v);

/* ---- transfer patterns (one DMA object, one transfer) ---- */
void oracle_sequential(const void* src, void* dst, size_t bytes);
void oracle_strided(const void* src, void* dst, int elmt_bytes, int num_elmts, int src_stride, int dst_stride);
/* strided transfer into swizzled LDS rows: chunk c (of `chunk` bytes) of row r lands at chunk
 * c ^ key(r) of the destination row; key(r) = bit-reversed low bits of r / (rows per 256-byte
 * bank line), as many bits as the row has aligned chunks (at most 256 bytes' worth).  No
 * counterpart in the reference: it states the layout of the STORE_LDS_SWIZZLE qualifiers of
 * include/hipdma/base.hpp.  elmt_bytes must be a multiple of chunk. */
void oracle_strided_swizzled(const void* src, void* dst, int elmt_bytes, int num_elmts, int src_stride, int dst_stride,
                             int chunk);
void oracle_gather(const int32_t* index, const void* src, void* dst, int elmt_bytes, int num_elmts, int alt_stride);
void oracle_scatter(const int32_t* index, const void* src, void* dst, int elmt_bytes, int num_elmts, int alt_stride);
void oracle_halo(const void* src_origin, void* dst_origin, int elmt_bytes, int radius, int corners,
                 int dimx, int dimy, int pitch);
void oracle_halo_pitched(const void* src_origin, void* dst_origin, int elmt_bytes, int radius, int corners,
                         int dimx, int dimy, int pitch, int dst_pitch);
/* 1 when odata holds the ring of idata; both point at the top-left of the padded tile */
int oracle_halo_check(const void* idata, const void* odata, int elmt_bytes, int radius, int corners,
                      int dimx, int dimy, int pitch);

/* ---- benchmark workloads (OpenMP) ---- */
void oracle_copy(const float* in, float* out, size_t n);
void oracle_transpose(const float* in, float* out, int n);
void oracle_gather_copy(const float* table, const int32_t* idx, float* out, size_t n_idx, int rec_floats);
void oracle_scatter_copy(const float* records, const int32_t* idx, float* table, size_t n_idx, int rec_floats);
void oracle_gather_rowsum(const float* table, const int32_t* idx, float* out, size_t n_idx, int rec_floats,
                          int recs_per_tile);
void oracle_stencil25(const float* in, float* out, int nx, int ny, int nz, int radius_pad);
void oracle_gemm_bf16(const uint16_t* a, const uint16_t* b, float* c, int m, int n, int k);
/* one entry of the product, for spot checks at full size */
float oracle_gemm_bf16_entry(const uint16_t* a, const uint16_t* b, int n, int k, int row, int col);

/* ---- consumers of the reference's example programs ---- */
/* y[i] = fma(a, x[i], y[i])  (src/examples/saxpy/saxpy_cudaDMA_kernel.cu:55-59) */
void oracle_saxpy(float a, const float* x, float* y, size_t n);
/* y[i] = alpha * sum_j A[i + j*lda] * x[j], A column-major n x m, ascending j, fused multiply-add
 * (src/examples/sgemv/sgemv_dma.cu:140-175) */
void oracle_sgemv(int n, int m, float alpha, const float* a, int lda, const float* x, float* y);
/* two-component 2-D cross average of every z slice (src/examples/stencil/stencil_math.h:27-87);
 * buffers are padded by `radius` on every side of all three dimensions
 * (src/examples/stencil/cudaDMA_stencil2D.cu:86-101); `reach` neighbours per arm are summed */
void oracle_stencil2d(const float* src, float* dst, int dimx, int dimy, int dimz, int radius, int reach);

#ifdef __cplusplus
}
#endif
#endif
