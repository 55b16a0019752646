#define CUMO_T dfloat
#define CUMO_C double
#include "ew_extra_float.inc"
