// Sliding-window forward / fused backward kernels specialised for kernel size 7.
#define NPLM_K 7
#include "dwconv_inst.inc"
