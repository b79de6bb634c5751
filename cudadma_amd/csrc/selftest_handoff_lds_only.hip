// The same kernel built with HIPDMA_LDS_ONLY_FENCE: on gfx950 both builds wait the same way (the wavefronts of
// a workgroup share one vector L1 that serves requests in issue order); the switch only frees the compiler to
// move global accesses across a hand-off, so this build documents what the hardware does, not a guarantee.
#define HIPDMA_LDS_ONLY_FENCE
#define HANDOFF_ENTRY cudadma_selftest_global_handoff_lds_only
#include "selftest_handoff.inc"
