// Single-function elementwise kernels (see nk_eltwise.h, rows_single_kernel): element type float.
#define NK_T float
#include "nk_eltwise_single.inc"
