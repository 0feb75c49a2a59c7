// Elementwise kernel family: element type float, function set 0 (see nk_eltwise.h).
#define NK_T float
#define NK_FUNSET 0
#include "nk_eltwise_family.inc"
