// Sliding-window forward / fused backward kernels specialised for kernel size 31.
#define NPLM_K 31
#ifdef NPLM_SWEEP
// extra (dtype, VEC, U, launch-bounds) variants for the geometry sweeps
#define NPLM_SWEEP_FWD                                                                     \
    NPLM_FWD(true, 2, 16, 256) NPLM_FWD(true, 2, 4, 256)
#define NPLM_SWEEP_BWD                                                                     \
    NPLM_BWD(true, 1, 16, 256) NPLM_BWD(true, 1, 4, 256) NPLM_BWD(true, 1, 2, 256) NPLM_BWD(true, 2, 4, 256)
#endif
#include "dwconv_inst.inc"
