#define CUMO_T dfloat
#define CUMO_C double
#define CUMO_PART 1
#define CUMO_DOUBLE 1
#include "reduce_float.inc"
