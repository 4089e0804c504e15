// LDS-staged forward / fused backward kernels specialised for kernel size 3.
#define NPLM_K 3
#include "dwconv_lds_inst.inc"
