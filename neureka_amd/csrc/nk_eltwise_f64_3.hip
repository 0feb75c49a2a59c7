// Elementwise kernel family: element type double, function set 3 (see nk_eltwise.h).
#define NK_T double
#define NK_FUNSET 3
#include "nk_eltwise_family.inc"
