// LDS-staged forward / fused backward kernels specialised for kernel size 7.
#define NPLM_K 7
#ifdef NPLM_SWEEP
// extra (dtype, VEC, rows per wave, row groups, wave-columns, loader waves, buffers) variants for the sweeps
#define NPLM_SWEEP_LFWD                                                                                 \
    NPLM_LFWD(true, 4, 8, 2, 4, 4, 2) NPLM_LFWD(true, 4, 8, 2, 4, 4, 3) NPLM_LFWD(true, 4, 8, 2, 4, 2, 3) \
    NPLM_LFWD(true, 8, 8, 2, 2, 2, 3) NPLM_LFWD(true, 8, 8, 2, 2, 4, 3) NPLM_LFWD(true, 4, 4, 2, 4, 4, 3) \
    NPLM_LFWD(true, 4, 6, 2, 4, 4, 3) NPLM_LFWD(true, 8, 4, 4, 2, 4, 3) NPLM_LFWD(true, 4, 8, 2, 4, 8, 3)
#define NPLM_SWEEP_LBWD NPLM_LBWD(true, 4, 8, 2, 4, 4, 2) NPLM_LBWD(true, 2, 16, 1, 8, 4, 2) NPLM_LBWD(true, 4, 4, 2, 4, 4, 2) \
    NPLM_LBWD(true, 2, 8, 1, 8, 4, 2)
#endif
#include "dwconv_lds_inst.inc"
