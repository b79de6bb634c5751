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
#pragma once

#include "hipdma/base.hpp"
#include "hipdma/mem.hpp"
#include "hipdma/sequential.hpp"
#include "hipdma/grid.hpp"
#include "hipdma/strided.hpp"
#include "hipdma/indirect.hpp"
#include "hipdma/halo.hpp"
#include "hipdma/v1.hpp"
