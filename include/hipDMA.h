// hipDMA: wavefront-specialised DMA objects for AMD CDNA4 (gfx950).
//
// Header-only.  Provides CudaDMASequential, CudaDMAStrided, CudaDMAIndirect and
// CudaDMAHalo with the template parameters and calls of include/cudaDMAv2.h
// (DO_SYNC, ALIGNMENT, BYTES_PER_THREAD, BYTES_PER_ELMT, DMA_THREADS, NUM_ELMTS;
// execute_dma, start_xfer_async, wait_xfer_finish, start_async_dma,
// wait_for_dma_finish, wait_for_dma_start, finish_async_dma, owns_this_thread),
// rebuilt around 64-lane wavefronts, dwordx4 / direct-to-LDS loads and an
// LDS-counter handshake instead of named barriers.
//
// What a kernel written for the CUDA header has to change:
//   * include this file (or the forwarding cudaDMAv2.h next to it);
//   * make the compute and DMA thread counts multiples of 64 instead of 32 and
//     start the DMA threads at a multiple of 64;
//   * construct every warp-specialised object in all threads of the workgroup,
//     before the code branches on owns_this_thread().
//
// What exists here and not in the CUDA header:
//   * store qualifiers STORE_LDS, STORE_LDS_DIRECT, STORE_LDS_SWIZZLE, STORE_LDS_DIRECT_SWIZZLE and
//     hipdma::swizzled_chunk() for readers of swizzled rows (base.hpp, strided.hpp);
//   * CudaDMAHalo with the v2 template parameters and two-phase calls (halo.hpp);
//   * peek_dma_finish() + wait_for_dma_finish(peeked), the wait in two halves (base.hpp);
//   * CudaDMAStrided::issue_direct() / issue_direct_part() + hipdma::wait_direct_loads<N>() and the
//     wait_for_dma_start_direct() / finish_async_dma_direct() hand-off, for kernels that keep several
//     direct-to-LDS transfers in flight or spread the loads of one between other instructions
//     (strided.hpp, base.hpp);
//   * hipdma::GroupBarrier, a barrier among some of the workgroup's wavefronts (base.hpp);
//   * CudaDMAIndirect::prefetch_index() + start_xfer_async_prefetched() / execute_dma_prefetched(): the index
//     words of a transfer requested ahead of it, for several objects on the same DMA threads (indirect.hpp);
//   * a destination pitch as the last constructor argument of CudaDMAHalo (halo.hpp);
//   * a failure record: a handshake wait that gives up sets HIPDMA_STATUS_WAIT_GAVE_UP in a device word that
//     hipdma::read_status() returns to the host (base.hpp);
//   * HIPDMA_SPIN_LIMIT, HIPDMA_LDS_ONLY_FENCE, DEBUG_CUDADMA build switches (base.hpp).
#pragma once

#include "hipdma/base.hpp"
#include "hipdma/mem.hpp"
#include "hipdma/sequential.hpp"
#include "hipdma/grid.hpp"
#include "hipdma/strided.hpp"
#include "hipdma/indirect.hpp"
#include "hipdma/halo.hpp"
#include "hipdma/v1.hpp"
