// The stencil kernels of workloads_stencil.hip once more with tiles of 64 x 16 cells instead of 32 x 32: a tile
// row is 256 contiguous bytes in memory instead of 128, sixteen lanes share it instead of eight, the ring has 160
// chunks instead of 128 (three per DMA thread).  Reached through cudadma_halo_stencil variants 6 and 7.
#define STENCIL_TX 64
#define STENCIL_TY 16
#define STENCIL_WIDE_TILES 1
#include "workloads_stencil.hip"
