/* C ABI of libcudadma_amd.so: the host drivers around the hipDMA device header.
 *
 * The reference is a header; what its repository binds it to are the host
 * programs of src/tests, src/perf and src/examples.  Each entry point below
 * stands for one of the src/perf and src/examples programs' run functions (the
 * counterpart of src/tests is cudadma_amd_harness.h, a library of its own), takes plain device pointers
 * and sizes, launches on the given HIP stream (NULL = default stream) and
 * returns 0 or a negative CUDADMA_E* code; cudadma_last_error() gives the text.
 * Nothing here allocates device memory.
 */
#ifndef CUDADMA_AMD_H
#define CUDADMA_AMD_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define CUDADMA_OK            0
#define CUDADMA_EINVAL       -1   /* bad argument (size, alignment, variant, null pointer) */
#define CUDADMA_ELAUNCH      -2   /* HIP reported a launch or runtime error */
#define CUDADMA_ERANGE       -3   /* case index or variant out of range */

const char* cudadma_last_error(void);
/* Number of compute units of the current device (used to size persistent grids). */
int cudadma_device_cus(void);

/* The transfer patterns of the DMA objects. */
enum {
  CUDADMA_PATTERN_SEQUENTIAL = 0,
  CUDADMA_PATTERN_STRIDED    = 1,
  CUDADMA_PATTERN_GATHER     = 2,
  CUDADMA_PATTERN_SCATTER    = 3,
  CUDADMA_PATTERN_HALO       = 4
};

/* The failure record of the handshake.  A wait that runs into the poll limit (HIPDMA_SPIN_LIMIT of
 * include/hipdma/base.hpp; the reference's named barriers would hang instead, its DEBUG_CUDADMA build asserts,
 * include/cudaDMAv2.h:1564-1576) lets its kernel finish and records the fact on the device.  This call waits
 * for `stream` to drain and returns, summed over every kernel of the library that ran on the current device
 * since the last clear: *status_bits = CUDADMA_STATUS_* bits, *waits_given_up = wavefronts whose wait gave up.
 * clear != 0 resets the record.  Either pointer may be NULL.  Allocates nothing.  A non-zero record means the
 * outputs of the kernels since the last clear are void. */
#define CUDADMA_STATUS_WAIT_GAVE_UP 1u
int cudadma_device_status(unsigned* status_bits, unsigned* waits_given_up, int clear, void* stream);
/* Number of translation units whose record cudadma_device_status() reads. */
int cudadma_device_status_sources(void);

/* ------------------------------------------------------------------------
 * Host-side planner.  cudadma_diagnose prints what the static diagnose()
 * members of the objects print (include/cudaDMAv2.h:1402-1458, :3208-3493,
 * :9417-9698).  cudadma_plan_map replays, on the host and with the very code
 * the device objects use, which DMA thread moves which bytes: map[d] receives
 * the source byte offset that lands on destination byte d (-1 = untouched),
 * both relative to the transfer's pointers shifted by src_origin / dst_origin.
 * Returns the number of destination bytes written more than once (0 for a
 * sound plan) or a negative error, e.g. when a thread would step outside
 * [0, map_len).  Needs no GPU.
 * ---------------------------------------------------------------------- */
typedef struct cudadma_plan_query {
  int pattern;            /* CUDADMA_PATTERN_*                                   */
  int alignment, bytes_per_thread, bytes_per_elmt, dma_threads, num_elmts;
  int src_stride;         /* strided; scatter: dense-side stride                 */
  int dst_stride;         /* strided; gather: dense-side stride                  */
  int radius, corners, dimx, dimy, pitch;   /* halo                              */
  const int* index;       /* gather / scatter: num_elmts element indices         */
  int dst_pitch;          /* halo: destination row pitch in cells, 0 = dimx + 2*radius */
} cudadma_plan_query_t;

int cudadma_plan_map(const cudadma_plan_query_t* q, long long src_origin, long long dst_origin,
                     int* map, size_t map_len, int* steps_out);
/* The same replay without the map: the lowest and highest byte offsets (relative to the transfer's pointers)
 * that any DMA thread reads and writes; extents[0..3] = src_min, src_end, dst_min, dst_end (end = one past the
 * last byte; all 0 for an empty transfer).  Returns 0 or a negative error. */
int cudadma_plan_extents(const cudadma_plan_query_t* q, long long extents[4]);
int cudadma_diagnose(int pattern, int alignment, int bytes_per_thread, int bytes_per_elmt, int dma_threads,
                     int num_elmts, int full_template, int verbose);

/* ------------------------------------------------------------------------
 * Benchmark workloads.  Each launches one persistent-grid kernel built from the
 * DMA objects; `variant` picks the buffering idiom, as the none / single /
 * double / manual kernels of src/perf/sequential/perf_sequential.cu:52-223 and
 * the five stencil kernels of src/examples/stencil do.  Variant 0 is the one the
 * benchmark reports.  cudadma_num_variants(workload) tells how many exist.
 * ---------------------------------------------------------------------- */
enum {
  CUDADMA_WORKLOAD_SEQUENTIAL = 0,
  CUDADMA_WORKLOAD_STRIDED    = 1,
  CUDADMA_WORKLOAD_GATHER     = 2,
  CUDADMA_WORKLOAD_HALO       = 3,
  CUDADMA_WORKLOAD_GEMM       = 4,
  CUDADMA_WORKLOAD_SCATTER    = 5
};
int cudadma_num_variants(int workload);
/* One-line description of a variant ("" when out of range, and for a variant that this build of the library
 * does not hold: kernels that only serve the parameter sweeps are compiled with make EXTRA=-DHIPDMA_SWEEP_VARIANTS). */
const char* cudadma_variant_name(int workload, int variant);
/* The values the knob "transpose_split" accepts in this build: writes up to `capacity` of them to `codes`
 * (may be NULL) and returns how many there are. */
int cudadma_transpose_splits(int* codes, int capacity);
/* Tuning knob: workgroups resident per compute unit for the persistent grids
 * (0 restores each kernel's default).  Returns the previous value. */
int cudadma_set_workgroups_per_cu(int value);
/* Further integer knobs by name (0 restores the default); returns the previous
 * value or CUDADMA_EINVAL for an unknown name:
 *   "transpose_band"  tile rows per band of the config 2 tile order
 *   "transpose_workgroups"  workgroups to launch for config 2, whatever the per-CU knob says
 *   "transpose_split"  config 2, variant 10: 100 x DMA wavefronts + 10 x compute wavefronts + tiles requested ahead
 *                      (1 or 2; with 3 + 1 wavefronts also 3 .. 7: the tile requested in halves or quarters, 1.5, 1.25, 1.5,
 *                      1.75 and 0.75 tiles in flight; 8, also with 2 + 2: the next tile requested as soon as the loads of
 *                      the current one have returned)
 *   "stencil_zchunk"     output planes one workgroup marches through in config 4
 *   "stencil_xcd_remap"  config 4 numbers its workgroups so that each XCD gets a slab of the grid over its whole width;
 *                        4 asks for compact blocks of the tile grid instead (2 x 4 blocks), 2 turns the numbering off
 *   "stencil_ring"       halo objects on the DMA wavefront of config 4's warp-specialised kernels: 8 or 12 */
int cudadma_set_tuning(const char* name, int value);

/* Seeded inputs generated on the device; bit-identical to the host statement
 * h(i) = splitmix64(seed + i) >> 32, value = (h >> 8) * 2^-23 - 1. */
int cudadma_fill_uniform(float* d_dst, size_t n, uint64_t seed, void* stream);
/* normal(0,1) values as bf16 bit patterns (the inputs of config 5): Box-Muller on the hashes 2i and 2i+1,
 * sqrt(-2 ln u1) * cos(2 pi u2) with u1 = ((h(2i) >> 8) + 1) / 2^24 and u2 = (h(2i+1) >> 8) / 2^24 in double
 * precision, rounded to float, then to bf16 (nearest even). */
int cudadma_fill_normal_bf16(uint16_t* d_dst, size_t n, uint64_t seed, void* stream);
/* Element indices uniform over [0, n_records), one in ten repeating an earlier draw. */
int cudadma_fill_indices(int32_t* d_dst, size_t n, uint32_t n_records, uint64_t seed, void* stream);

/* A seeded permutation of [0, 2^log2_n), 1 <= log2_n <= 31: distinct element indices for the
 * scatter.  With mask = 2^log2_n - 1, h = (log2_n + 1) / 2, k0 = splitmix64(seed) and
 * k1 = splitmix64(seed + 1), entry i is x after
 *   x = i;  x = (x * (lo32(k0) | 1) + hi32(k0)) & mask;  x ^= x >> h;
 *           x = (x * (lo32(k1) | 1) + hi32(k1)) & mask;  x ^= x >> h;
 *           x = (x * 0x9E3779B1) & mask
 * (an odd multiplier, an added constant and a right xor-shift are each one-to-one on log2_n bits). */
int cudadma_fill_permutation(int32_t* d_dst, int log2_n, uint64_t seed, void* stream);

/* Calibration kernel: grid-stride dwordx4 copy with no LDS and no DMA object.
 * bytes must be a multiple of 16. */
int cudadma_plain_copy(const void* d_src, void* d_dst, size_t bytes, void* stream);

/* Config 1 (perf_sequential.cu:255-361): copy `bytes` (a multiple of 16 KiB) in
 * 16 KiB tiles through LDS; 128 DMA + 128 compute threads per workgroup. */
int cudadma_sequential_copy(const float* d_in, float* d_out, size_t bytes, int variant, void* stream);

/* Config 2: d_out = transpose(d_in) for an n x n float matrix, n a multiple of
 * 64; CudaDMAStrided pulls 64 rows x 256 B tiles, consumers write them transposed. */
int cudadma_strided_transpose(const float* d_in, float* d_out, int n, int variant, void* stream);

/* Config 3: records of 128 B; n_idx a multiple of 32.  CudaDMAIndirect gathers
 * 32 records per LDS tile.
 *   copy  : d_out[i] = d_table[d_idx[i]]                     (n_idx * 128 B)
 *   rowsum: d_out[t][j] = sum_{r<32} d_table[d_idx[32t+r]][j] (n_idx/32 * 128 B) */
int cudadma_gather_copy(const float* d_table, const int32_t* d_idx, float* d_out,
                        size_t n_records, size_t n_idx, int variant, void* stream);
int cudadma_gather_rowsum(const float* d_table, const int32_t* d_idx, float* d_out,
                          size_t n_records, size_t n_idx, int variant, void* stream);

/* The opposite direction of config 3, LDS -> global (include/cudaDMAv2.h:10199-10217; the
 * reference has no test or program of it): d_table[d_idx[i]] = d_records[i] for i < n_idx,
 * records of 128 B, n_idx a multiple of 32.  The compute wavefronts fill LDS tiles of 32
 * records, the DMA wavefronts scatter them with CudaDMAIndirect<false>.  d_idx[i] must lie
 * in [0, n_records); records of the table that no index names are left untouched; when an
 * index repeats, which of its records ends up in the table is unspecified. */
int cudadma_scatter_copy(const float* d_records, const int32_t* d_idx, float* d_table,
                         size_t n_records, size_t n_idx, int variant, void* stream);

/* Config 4 (src/examples/stencil/cudaDMA_stencil2D.cu:100-240): 8th-order
 * 25-point star stencil.  d_in is (nx+8) x (ny+8) x (nz+8) floats, x fastest;
 * d_out is nx x ny x nz.  nx, ny multiples of 32.  CudaDMAHalo brings the ring
 * of each 32x32 tile, plane by plane along z.  Variants 6 and 7 are variants 0 and 1
 * with tiles of 64 x 16 cells and need nx a multiple of 64 and ny a multiple of 16. */
int cudadma_halo_stencil(const float* d_in, float* d_out, int nx, int ny, int nz, int variant, void* stream);

/* Config 5 (no GEMM in the reference; nearest: src/examples/sgemv/sgemv_dma.cu:329-388):
 * C = A * B with A m x k and B k x n row-major bf16 (as uint16 bit patterns), C m x n
 * float, fp32 accumulation on the matrix cores.  m, n and k multiples of 128.
 * In the warp-specialised variants four DMA wavefronts stage the A and B tiles of one K step
 * through CudaDMAStrided and four or eight compute wavefronts multiply.  variant 0 picks the largest workgroup tile that divides the
 * problem and leaves no compute unit without a tile; 1: 128 x 128; 2: 128 x 256 (n a multiple of
 * 256); 3: 256 x 128 (m a multiple of 256); 4: 256 x 128 with the tiles brought in by
 * global_load_lds into swizzled LDS rows; 5: 256 x 256 with eight compute wavefronts (m and n
 * multiples of 256); 6: the same tile with K steps of 32 brought into four swizzled LDS stages by
 * global_load_lds; 7: variant 6 with A transfers of two K steps (rows of 128 B, whole cache
 * lines) into two buffers of their own; 8: the 256 x 256 tile without warp specialisation: four
 * wavefronts that each issue their share of the direct-to-LDS loads (the form of CudaDMAStrided
 * that is not warp-specialised) between the matrix instructions of their 128 x 128 block; 9:
 * variant 8 with A transfers of two K steps in a ring of three buffers. */
int cudadma_gemm_bf16(const uint16_t* d_a, const uint16_t* d_b, float* d_c, int m, int n, int k,
                      int variant, void* stream);

/* ---- read-bandwidth probe with run-time parameters ------------------------------------
 * src/perf/sequential/perf_sequential.cu:52-228 with the macros of params_directed.h as
 * arguments: every workgroup brings loop_iters consecutive elements of elmt_bytes into
 * LDS with CudaDMASequential (run-time size and thread count), one compute wavefront
 * standing for the consumer.  buffering picks the kernel shape of the reference's four.
 * Returns the bytes read (workgroups * elmt_bytes * loop_iters) or a negative CUDADMA_E*
 * code.  d_sums may be NULL (pure probe, nothing is written, as in the reference); otherwise
 * it holds one zero-initialised word per workgroup, to which the 32-bit words that arrived
 * in LDS are added.
 * load_qualifier / store_qualifier are the template arguments of the objects' fully qualified calls
 * (execute_dma<true, LOAD_QUAL, STORE_QUAL>, include/cudaDMAv2.h:1460-1562; the reference's probe uses the
 * defaults, perf_sequential.cu:67): CUDADMA_LOAD_CACHE_ALL or _STREAMING (non-temporal loads), and how the
 * bytes reach LDS: CUDADMA_STORE_WRITE_BACK (a generic store, the reference's default), CUDADMA_STORE_LDS
 * (ds_write_b128) or CUDADMA_STORE_LDS_DIRECT (global_load_lds, no register staging).  Other values are refused
 * with CUDADMA_ERANGE.  The objects' BYTES_PER_THREAD is 64: four dwordx4 in flight per DMA thread. */
enum {
  CUDADMA_BUFFERING_NONE   = 0,  /* not warp-specialised, two workgroup barriers per element */
  CUDADMA_BUFFERING_SINGLE = 1,  /* one buffer, one object                                    */
  CUDADMA_BUFFERING_DOUBLE = 2,  /* two buffers, two objects on disjoint DMA wavefronts       */
  CUDADMA_BUFFERING_MANUAL = 3   /* two buffers, two objects on the same DMA wavefronts       */
};
/* values of enum CudaDMALoadQualifier / CudaDMAStoreQualifier of the device header (include/cudaDMAv2.h:50-63,
 * plus the LDS stores this library adds) */
enum {
  CUDADMA_LOAD_CACHE_ALL       = 0,
  CUDADMA_LOAD_CACHE_STREAMING = 2,
  CUDADMA_STORE_WRITE_BACK     = 0,
  CUDADMA_STORE_LDS            = 4,
  CUDADMA_STORE_LDS_DIRECT     = 5
};
long long cudadma_perf_sequential(const void* d_src, size_t src_bytes, unsigned* d_sums, int elmt_bytes,
                                  int dma_wavefronts, int buffering, int loop_iters, int workgroups,
                                  int load_qualifier, int store_qualifier, void* stream);

/* ---- streaming yardsticks ------------------------------------------------------------------
 * Kernels without LDS and without a DMA object (grid-stride dwordx4 accesses) that show what read-only,
 * write-only and copy-shaped streams reach on the device at a given launch shape, and the vendor's own
 * device-to-device copy: what the patterns' figures are read against.  No counterpart in the reference.
 * `bytes` is the size of each buffer (a multiple of 16).  Write-only modes store the float 1.0.
 * Returns the bytes read plus the bytes written, or a negative CUDADMA_E* code. */
enum {
  CUDADMA_PROBE_READ                 = 0,  /* d_dst may be NULL                                    */
  CUDADMA_PROBE_WRITE                = 1,  /* d_src may be NULL                                    */
  CUDADMA_PROBE_WRITE_NONTEMPORAL    = 2,
  CUDADMA_PROBE_COPY                 = 3,
  CUDADMA_PROBE_COPY_NONTEMPORAL     = 4,  /* non-temporal loads and stores                        */
  CUDADMA_PROBE_VENDOR_COPY          = 5,  /* hipMemcpyDtoDAsync; `workgroups` is ignored          */
  CUDADMA_PROBE_READ_NONTEMPORAL     = 6,  /* d_dst may be NULL                                    */
  CUDADMA_PROBE_MODES                = 7
};
long long cudadma_probe_memory(int mode, const void* d_src, void* d_dst, size_t bytes, int workgroups, void* stream);

/* Clock probe: one wavefront runs `iterations` dependent fused multiply-adds between two readings of the shader clock
 * counter (s_memtime) and of the constant 100 MHz counter (s_memrealtime).  d_ticks[0] and d_ticks[1] receive the two
 * differences: d_ticks[0] / d_ticks[1] x 100 MHz is the shader clock during the launch, and d_ticks[0] / iterations
 * the cycles per dependent instruction (a constant of the chip).  Used to tell a clock ramp from a memory-side effect
 * when the first launches after an idle phase run slow.  No counterpart in the reference. */
int cudadma_probe_clock(uint64_t* d_ticks, int iterations, void* stream);

/* ---- yardsticks with the patterns' own addresses -----------------------------------------------
 * The memory accesses of the gather, the scatter and the tile transposition with nothing but loads and stores
 * between them and memory (no LDS, no DMA object, no handshake), on the patterns' own buffers: what each pattern's
 * figure is read against.  No counterpart in the reference.  `workgroups` workgroups of 256 threads share the work
 * round-robin.  Returns the algorithmic bytes moved, or a negative CUDADMA_E* code.
 *   GATHER_XOR  d_in: table of n_records records of 128 B; d_idx: n element indices (n a multiple of 32);
 *               d_out[t][j] = xor over r < 32 of the 32-bit words table[d_idx[32 t + r]][j]: n / 32 rows of 128 B.
 *               Moves what cudadma_gather_rowsum moves: n * 132 + n / 32 * 128 bytes.
 *   SCATTER     d_in: n records of 128 B; d_out: table of n_records records; table[d_idx[i]] = records[i].
 *               Moves what cudadma_scatter_copy moves: n * 260 bytes.
 *   TILE_READ   d_in: n x n floats (n a multiple of 64); reads its 64 x 64 tiles in the order in which
 *               cudadma_strided_transpose takes them (workgroup b: tiles b, b + workgroups, ...; tile t lies in
 *               tile row t mod (n / 64), tile column t / (n / 64)); d_out receives 16 bytes per workgroup: the xor
 *               of the 16-byte chunks of its tiles.  n * n * 4 bytes.
 *   TILE_WRITE  d_out: n x n floats; writes, in the same order, the output tiles of the transposition (source tile
 *               (row ty, column tx) lands on rows 64 tx.., columns 64 ty..); element (r, c) receives the 32-bit
 *               pattern r * n + c.  n * n * 4 bytes.  d_in and d_idx are ignored.
 *   TILE_COPY   both halves together without the transposition inside a tile:
 *               d_out[64 tx + r][64 ty + c] = d_in[64 ty + r][64 tx + c].  2 * n * n * 4 bytes.
 *   MASKED_READ d_in: a buffer of n bytes (a power of two, 256-byte aligned); n_records: a bit mask over the index of
 *               its 256-byte granules.  Reads the granules whose index has even parity under the mask (half of the
 *               buffer: n / 2 bytes); d_out receives 16 bytes per workgroup, the xor of the 16-byte chunks it read.
 *               When the parity of those address bits picks half of the memory channels, the rate halves: a probe
 *               for the address hash of the part.  d_idx is ignored.
 * Two knobs of cudadma_set_tuning shape TILE_WRITE and TILE_COPY: "probe_piece_bytes" (256, 512, 1024, 2048 or
 * 4096; default 256, one tile) is the length of the piece of an output row that a workgroup writes per turn
 * (TILE_COPY then reads pieces of as many source tiles per turn), "probe_xcd_group" = 1 gives the workgroups of
 * one XCD neighbouring pieces instead of every eighth one. */
enum {
  CUDADMA_PATTERN_PROBE_GATHER_XOR = 0,
  CUDADMA_PATTERN_PROBE_SCATTER    = 1,
  CUDADMA_PATTERN_PROBE_TILE_READ  = 2,
  CUDADMA_PATTERN_PROBE_TILE_WRITE = 3,
  CUDADMA_PATTERN_PROBE_TILE_COPY  = 4,
  CUDADMA_PATTERN_PROBE_MASKED_READ = 5,
  CUDADMA_PATTERN_PROBE_MODES      = 6
};
long long cudadma_probe_pattern(int mode, const void* d_in, const int32_t* d_idx, void* d_out, size_t n,
                                size_t n_records, int workgroups, void* stream);

/* ---- the reference's example programs on the wave64 objects --------------------------
 * The kernels behind these are written against the DMA classes alone (the first-
 * generation names of include/cudaDMA.h for saxpy and sgemv, the current ones for the
 * stencil); the reference has them as stand-alone programs with compile-time sizes,
 * here sizes are arguments and the launch geometry is fixed per example. */
enum {
  CUDADMA_EXAMPLE_SAXPY     = 0,
  CUDADMA_EXAMPLE_SGEMV     = 1,
  CUDADMA_EXAMPLE_STENCIL2D = 2
};
int cudadma_example_num_variants(int example);
const char* cudadma_example_variant_name(int example, int variant);

/* y = a*x + y in place, one fused multiply-add per element
 * (src/examples/saxpy/saxpy_cudaDMA_kernel.cu:55-61, :270-315, :322-418; driver
 * saxpy_cudaDMA.cu:76-175).  Variants 0/1 use no DMA object, 2/3 stage x and y through
 * LDS with cudaDMASequential.  n a multiple of 1024 floats except for variant 0. */
int cudadma_example_saxpy(int variant, float a, const float* d_x, float* d_y, long long n, void* stream);

/* y = alpha * A x, A column-major n x m with leading dimension lda, accumulated in
 * ascending column order with fused multiply-add (src/examples/sgemv/sgemv_dma.cu:140-175,
 * :262-325, :329-388, :392-470; host check :752-771).  m a multiple of 256 (variant 0),
 * 512 (variant 1) or 32 (variants 2, 3, which also need lda >= n rounded up to 128 and
 * 16-byte aligned columns). */
int cudadma_example_sgemv(int variant, int n, int m, float alpha, const float* d_a, int lda, const float* d_x,
                          float* d_y, void* stream);

/* The 2-D cross average of every z slice of a float2 volume in its five buffering
 * styles (src/examples/stencil/cudaDMA_stencil2D.cu:99-204, stencil_math.h:27-87).
 * d_src and d_dst hold (dimx+8) x (dimy+8) x (dimz+8) float2 elements (radius 4 padding on
 * every side, x fastest); only interior points of d_dst are written.  full_cross = 0
 * sums three neighbours per arm as the reference's loops do, 1 sums all four; the divisor
 * is 17 either way.  dimx a multiple of 32, dimy of 4; dimz even for variants 1, 2, 4. */
int cudadma_example_stencil2d(int variant, const float* d_src, float* d_dst, int dimx, int dimy, int dimz,
                              int full_cross, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* CUDADMA_AMD_H */
