// Single-function elementwise kernels (see nk_eltwise.h, rows_single_kernel): element type double.
#define NK_T double
#include "nk_eltwise_single.inc"
