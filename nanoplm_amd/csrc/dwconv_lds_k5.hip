// LDS-staged forward / fused backward kernels specialised for kernel size 5.
#define NPLM_K 5
#include "dwconv_lds_inst.inc"
