#define CUMO_T sfloat
#define CUMO_C float
#include "ew_extra_float.inc"
