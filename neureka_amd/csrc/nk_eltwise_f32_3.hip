// Elementwise kernel family: element type float, function set 3 (see nk_eltwise.h).
#define NK_T float
#define NK_FUNSET 3
#include "nk_eltwise_family.inc"
