// Registers this translation unit's copy of the DMA objects' failure record with the library, so that
// cudadma_device_status() finds it.  Every .hip file that instantiates DMA objects includes this header.
#pragma once

#include "common.hpp"
#include "../../include/hipDMA.h"

namespace {
const cudadma_host::StatusRegistrar g_status_registrar(&hipdma::status_words_address, __FILE__);
}
