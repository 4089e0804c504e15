// Sliding-window forward / fused backward kernels specialised for kernel size 5.
#define NPLM_K 5
#include "dwconv_inst.inc"
