// Forwarding header: lets a kernel that says #include "cudaDMAv2.h" build
// against hipDMA unchanged.  WARP_SIZE is what such kernels size their thread
// groups with (include/cudaDMAv2.h:22); on gfx950 a wavefront has 64 lanes.
#pragma once

#include "hipDMA.h"

#ifndef WARP_SIZE
#define WARP_SIZE HIPDMA_WAVE_SIZE
#endif
