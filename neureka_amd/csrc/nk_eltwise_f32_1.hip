// Elementwise kernel family: element type float, function set 1 (see nk_eltwise.h).
#define NK_T float
#define NK_FUNSET 1
#include "nk_eltwise_family.inc"
