// LDS-staged forward / fused backward kernels specialised for kernel size 9.
#define NPLM_K 9
#include "dwconv_lds_inst.inc"
