// Sliding-window forward / fused backward kernels specialised for kernel size 15.
#define NPLM_K 15
#include "dwconv_inst.inc"
