/* C ABI of libcudadma_amd_harness.so: the known-answer harness and the self-tests of the hipDMA device
 * header, the counterpart of the reference's test programs under src/tests.  Test equipment, kept out of
 * libcudadma_amd.so (which it links against for the error text and the failure record): several hundred
 * instantiations of the DMA objects, one per combination of template parameters and call style.
 * Conventions as in cudadma_amd.h: plain device pointers and sizes, a HIP stream (NULL = default stream),
 * 0 or a negative CUDADMA_E* code, text from cudadma_last_error(); nothing here allocates device memory.
 */
#ifndef CUDADMA_AMD_HARNESS_H
#define CUDADMA_AMD_HARNESS_H

#include "cudadma_amd.h"

#ifdef __cplusplus
extern "C" {
#endif

/* ------------------------------------------------------------------------
 * Known-answer harness: one workgroup moves data global -> LDS with one DMA
 * object and copies the whole LDS buffer back out, as the kernels
 * special_xfer_* / nonspec_xfer_* of
 * src/tests/test_sequential/cudaDMA_test_sequential_v2.cu:52-395,
 * src/tests/test_strided/cudaDMA_test_strided_v2.cu:52-536,
 * src/tests/test_indirect/cudaDMA_test_indirect_v2.cu:52-548 and dma_ld_test of
 * src/tests/test_halo/cudaDMA_test_halo.cu:180-231 do.  Every compiled
 * combination of template parameters is one case.
 * ---------------------------------------------------------------------- */

/* Transfer call styles (cudaDMA_test_strided_v2.cu:693-812 runs the same set). */
enum {
  CUDADMA_CALL_UNQUALIFIED  = 0,  /* execute_dma(src,dst)                                  */
  CUDADMA_CALL_GLOBAL       = 1,  /* execute_dma<true>(src,dst)                            */
  CUDADMA_CALL_QUALIFIED    = 2,  /* execute_dma<true,LOAD_CACHE_STREAMING,STORE_LDS>      */
  CUDADMA_CALL_LDS_DIRECT   = 3,  /* execute_dma<true,LOAD_CACHE_ALL,STORE_LDS_DIRECT>     */
  /* strided cases whose rows are whole chunks: the chunks of LDS row r are permuted, chunk c
   * at position c ^ key(r) (hipdma::swizzled_chunk in include/hipdma/base.hpp: key = bit-reversed
   * low bits of the row number, as many bits as the row has aligned chunks, at most 256 bytes) */
  CUDADMA_CALL_LDS_SWIZZLE  = 4,  /* execute_dma<true,LOAD_CACHE_ALL,STORE_LDS_SWIZZLE>        */
  CUDADMA_CALL_LDS_DIRECT_SWIZZLE = 5, /* execute_dma<true,LOAD_CACHE_ALL,STORE_LDS_DIRECT_SWIZZLE> */
  /* The qualifier matrix (enums of include/cudaDMAv2.h:50-63): every load qualifier with a source known to be
   * global (Q_) and with a generic source (QG_), every store qualifier of the reference.  The QG_ styles are also
   * accepted with reverse = 1, where the store qualifier acts on global memory. */
  CUDADMA_CALL_Q_GLOBAL_CG      = 6,   /* <true,  LOAD_CACHE_GLOBAL,    STORE_CACHE_GLOBAL>        */
  CUDADMA_CALL_Q_LASTUSE_CS     = 7,   /* <true,  LOAD_CACHE_LAST_USE,  STORE_CACHE_STREAMING>     */
  CUDADMA_CALL_Q_VOLATILE_WT    = 8,   /* <true,  LOAD_CACHE_VOLATILE,  STORE_CACHE_WRITE_THROUGH> */
  CUDADMA_CALL_Q_STREAMING_WB   = 9,   /* <true,  LOAD_CACHE_STREAMING, STORE_WRITE_BACK>          */
  CUDADMA_CALL_QG_GLOBAL_CS     = 10,  /* <false, LOAD_CACHE_GLOBAL,    STORE_CACHE_STREAMING>     */
  CUDADMA_CALL_QG_STREAMING_WT  = 11,  /* <false, LOAD_CACHE_STREAMING, STORE_CACHE_WRITE_THROUGH> */
  CUDADMA_CALL_QG_LASTUSE_CG    = 12,  /* <false, LOAD_CACHE_LAST_USE,  STORE_CACHE_GLOBAL>        */
  CUDADMA_CALL_QG_VOLATILE_WB   = 13,  /* <false, LOAD_CACHE_VOLATILE,  STORE_WRITE_BACK>          */
  /* the direct-to-LDS path with the load qualifier in the instruction's cache-policy bits */
  CUDADMA_CALL_LDS_DIRECT_SC1   = 14,  /* <true,  LOAD_CACHE_GLOBAL,    STORE_LDS_DIRECT>          */
  CUDADMA_CALL_LDS_DIRECT_NT    = 15,  /* <true,  LOAD_CACHE_STREAMING, STORE_LDS_DIRECT>          */
  /* gather and scatter cases only: prefetch_index() + start_xfer_async_prefetched() / execute_dma_prefetched()
   * (an addition of this library to CudaDMAIndirect); with two_phase the index words of the next repetition are
   * requested between the two phases of the current one.  Generic source, so also accepted with reverse = 1. */
  CUDADMA_CALL_INDEX_AHEAD      = 16,
  CUDADMA_CALL_STYLES           = 17
};

typedef struct cudadma_case {
  int pattern;            /* CUDADMA_PATTERN_*                                        */
  int warp_specialized;   /* DO_SYNC                                                  */
  int level;              /* how many trailing template parameters are compile-time   */
  int alignment;          /* ALIGNMENT                                                */
  int bytes_per_thread;   /* BYTES_PER_THREAD                                         */
  int bytes_per_elmt;     /* BYTES_PER_ELMT (halo: bytes of one cell)                 */
  int dma_threads;        /* DMA_THREADS                                              */
  int num_elmts;          /* NUM_ELMTS (strided / indirect)                           */
  int radius;             /* halo only                                                */
  int corners;            /* halo only                                                */
  int dimx, dimy;         /* halo only: tile size in cells                            */
} cudadma_case_t;

typedef struct cudadma_run {
  const void* d_in;       /* device input                                             */
  void* d_out;            /* device output: reps * lds_bytes                          */
  const int* d_index;     /* device element indices (gather / scatter), else NULL     */
  int lds_bytes;          /* size of the LDS buffer, copied out whole after each rep  */
  int src_offset_bytes;   /* added to d_in before the transfer (ALIGN_OFFSET)         */
  int dst_offset_bytes;   /* added to the LDS buffer before the transfer              */
  int src_stride;         /* strided: source stride; scatter: dense-side stride       */
  int dst_stride;         /* strided: destination stride; gather: dense-side stride   */
  int pitch;              /* halo: source row pitch in cells                          */
  int call_style;         /* CUDADMA_CALL_*                                           */
  int two_phase;          /* start_xfer_async + wait_xfer_finish instead of execute   */
  int reps;               /* transfers run back to back through the same LDS buffer   */
  int rep_src_bytes;      /* source advance per rep                                   */
  int rep_index_elmts;    /* index advance per rep                                    */
  int reverse;            /* 1: the object moves LDS -> global.  The workgroup first copies
                             lds_bytes from d_in (+ rep * rep_src_bytes) into LDS, the object then
                             moves from LDS + src_offset_bytes to d_out + rep * out_bytes +
                             dst_offset_bytes.  Needs generic pointers on both sides
                             (include/cudaDMAv2.h:107-114,553-558): CUDADMA_CALL_UNQUALIFIED or one of
                             the CUDADMA_CALL_QG_* styles.                                         */
  int out_bytes;          /* reverse only: bytes of d_out one rep may touch            */
  /* Other values for the parameters that the case's level hands to the constructor at run time
   * (0 keeps the case's own), so that one compiled case can be swept the way the reference's
   * param_sweep_v2.py recompiles its test (src/tests/test_strided/param_sweep_v2.py:51-75):
   *   rt_bytes_per_elmt  level 1 of sequential / strided / indirect (a multiple of 4)
   *   rt_dma_threads     levels 1-2 of those, levels 0-1 of halo (a multiple of 64)
   *   rt_num_elmts       levels 1-3 of strided / indirect
   *   rt_dimx, rt_dimy   levels 0-2 of halo
   * A value for a parameter that the case fixes at compile time is refused. */
  int rt_bytes_per_elmt, rt_dma_threads, rt_num_elmts, rt_dimx, rt_dimy;
  /* halo: destination row pitch in cells handed to the constructor (0 = the reference's dimx + 2*radius,
   * include/cudaDMA.h:3718-3719); at least dimx + 2*radius and a multiple of ALIGNMENT in bytes */
  int dst_pitch;
  /* Sizes of the caller's buffers, so that a wrong value above is refused on the host instead of turning
   * into out-of-range accesses on the device: before the launch the transfer is replayed on the host with
   * the device objects' own index arithmetic (gather / scatter: after copying the index list back), and
   * the call fails with CUDADMA_ERANGE when any byte falls outside d_in, d_out or the LDS window. */
  size_t in_bytes;        /* bytes readable at d_in                                        */
  size_t out_capacity;    /* bytes writable at d_out: >= reps * (reverse ? out_bytes : lds_bytes) */
  int index_elmts;        /* ints readable at d_index                                      */
} cudadma_run_t;

int cudadma_num_cases(void);
int cudadma_get_case(int case_id, cudadma_case_t* out);
int cudadma_run_case(int case_id, const cudadma_run_t* run, void* stream);

/* Failure handling of the handshake (the reference deadlocks on unbalanced calls,
 * include/cudaDMAv2.h:1329-1347): launches one workgroup whose DMA and compute threads wait for
 * signals that never come, with the poll limit lowered to 256.  Both sides must give up and the
 * kernel must end; d_flags[0] (DMA side) and d_flags[1] (compute side) are then 1 and
 * cudadma_device_status() reports CUDADMA_STATUS_WAIT_GAVE_UP with a count of 2 wavefronts. */
int cudadma_selftest_bounded_wait(int* d_flags, void* stream);

/* Global memory handed across the handshake in both directions (the reference's bar.sync / bar.arrive order
 * all memory of the block, include/cudaDMAv2.h:65-75): per phase the compute wavefront writes 8 KiB to
 * d_scratch, two DMA wavefronts move them to d_scratch + 8 KiB with CudaDMASequential's generic-pointer
 * calls, the compute wavefront reads them back.  d_scratch: 16 KiB, 16-byte aligned; *d_wrong (zeroed)
 * receives the number of words read back wrong.  The _lds_only twin is the same kernel built with
 * HIPDMA_LDS_ONLY_FENCE. */
int cudadma_selftest_global_handoff(unsigned* d_scratch, int* d_wrong, int phases, void* stream);
int cudadma_selftest_global_handoff_lds_only(unsigned* d_scratch, int* d_wrong, int phases, void* stream);

/* No counterpart in the reference.  cudadma_selftest_global_handoff() for callers that cannot allocate device
 * memory (code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc): the same kernel with
 * its 16 KiB of staging memory in a device array of the library instead of d_scratch, so the caller passes only the
 * (zeroed) word for the result.  Calls no hipMalloc, hipFree or other allocating routine.  The need for staging memory
 * is those 16 KiB whatever the arguments; what bounds the call is `phases`, refused beyond CUDADMA_NOALLOC_MAX_PHASES
 * with CUDADMA_EINVAL.  The array exists once per device (16 KiB held until the process ends) and keeps the last
 * call's contents, which no call depends on; two calls that overlap on one device (different streams, or threads)
 * share it and race: run them one after the other.  The first call on a device looks the array's address up
 * (hipGetSymbolAddress) and should therefore happen outside a graph capture. */
#define CUDADMA_NOALLOC_MAX_PHASES (1 << 20)
int cudadma_selftest_global_handoff_noalloc(int* d_wrong, int phases, void* stream);

/* The split wait that only exists here (peek_dma_finish() + wait_for_dma_finish(peeked),
 * include/hipdma/base.hpp): one workgroup hands a 64-word buffer from a DMA wavefront to a
 * compute wavefront `phases` times, the DMA side early on even and late on odd phases.
 * d_out (two zeroed ints): [0] = words the compute side saw wrong (must be 0), [1] = phases in
 * which the peek already found the buffer full. */
int cudadma_selftest_split_wait(int* d_out, int phases, void* stream);

/* All sixteen dmaIDs at once: sixteen sync-only objects guard sixteen LDS slots, two DMA wavefronts
 * fill slot (phase mod 16) with the phase's token and may run sixteen phases ahead, one compute
 * wavefront checks every token.  d_out (one zeroed int) receives the number of wrong tokens. */
int cudadma_selftest_all_ids(int* d_out, int phases, void* stream);

/* ---- known-answer cases for the first-generation class names -------------------------
 * One transfer per case by cudaDMASequential / cudaDMAStrided / cudaDMAIndirect as declared in
 * include/cudaDMA.h:644-3580 (every constructor form), into a 16 KiB LDS window that holds the
 * byte 0xA5 everywhere else; the whole window is copied to d_out.  The reference has no test
 * of these classes beyond its examples; the expectation is the closed form of each pattern. */
typedef struct {
  int pattern;            /* CUDADMA_PATTERN_*                                               */
  int warp_specialized;   /* 1: 64 compute threads + dma_threads DMA threads; 0: all transfer */
  int bytes_per_elmt;     /* bytes of the transfer (sequential) or of one element             */
  int num_elmts;
  int src_stride;         /* bytes; strided source, or dense source of a scatter               */
  int dst_stride;         /* bytes; strided destination, or dense destination of a gather      */
  int dma_threads;
  int block_threads;
  int window_bytes;       /* size of d_out                                                     */
} cudadma_v1_case_t;
int cudadma_v1_num_cases(void);
int cudadma_v1_get_case(int case_id, cudadma_v1_case_t* out);
const char* cudadma_v1_case_text(int case_id);       /* the declaration the case exercises */
int cudadma_v1_run_case(int case_id, const void* d_in, const int* d_index, void* d_out, void* stream);

#ifdef __cplusplus
}
#endif

#endif /* CUDADMA_AMD_HARNESS_H */
