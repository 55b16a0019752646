#define CUMO_T dfloat
#define CUMO_C double
#include "ew_arith_float.inc"
