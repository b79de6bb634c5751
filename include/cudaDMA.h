// Forwarding header: kernels written against the first-generation interface
// (cudaDMASequential, cudaDMAStrided, cudaDMAIndirect, cudaDMAHalo,
// cudaDMACustom of include/cudaDMA.h) keep their include line.
#pragma once

#include "hipDMA.h"

#ifndef WARP_SIZE
#define WARP_SIZE HIPDMA_WAVE_SIZE
#endif
