// Sliding-window forward / fused backward kernels specialised for kernel size 7.
#define NPLM_K 7
#ifdef NPLM_SWEEP
// extra (dtype, VEC, U, launch-bounds) variants for the geometry sweeps
#define NPLM_SWEEP_FWD                                                                     \
    NPLM_FWD(true, 8, 2, 256) NPLM_FWD(true, 8, 8, 256) NPLM_FWD(true, 4, 4, 256)          \
    NPLM_FWD(true, 4, 16, 256) NPLM_FWD(true, 8, 4, 512) NPLM_FWD(true, 4, 8, 512)
#define NPLM_SWEEP_BWD                                                                     \
    NPLM_BWD(true, 8, 2, 256) NPLM_BWD(true, 8, 4, 256) NPLM_BWD(true, 4, 2, 512)          \
    NPLM_BWD(true, 4, 4, 512) NPLM_BWD(true, 4, 4, 256) NPLM_BWD(true, 4, 8, 256)          \
    NPLM_BWD(true, 2, 4, 512) NPLM_BWD(true, 2, 16, 512) NPLM_BWD(true, 2, 8, 1024)
#endif
#include "dwconv_inst.inc"
