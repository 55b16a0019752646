#define CUMO_T dfloat
#define CUMO_C double
#include "ew_math_float.inc"
