// LDS-staged forward / fused backward kernels specialised for kernel size 31.
#define NPLM_K 31
#ifdef NPLM_SWEEP
#define NPLM_SWEEP_LFWD NPLM_LFWD(true, 2, 8, 3, 4, 4, 2) NPLM_LFWD(true, 2, 10, 3, 4, 4, 2)
#endif
#include "dwconv_lds_inst.inc"
