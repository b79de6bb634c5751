// Global-memory hand-off across the handshake with the header's default (all address spaces) fences.
#define HANDOFF_ENTRY cudadma_selftest_global_handoff
#include "selftest_handoff.inc"
