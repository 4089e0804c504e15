// Sliding-window forward / fused backward kernels specialised for kernel size 31.
#define NPLM_K 31
#include "dwconv_inst.inc"
