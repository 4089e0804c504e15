// LDS-staged forward kernel specialised for kernel size 15 (the fused backward is built for K <= 9 only).
#define NPLM_K 15
#include "dwconv_lds_inst.inc"
