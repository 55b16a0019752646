#define CUMO_T dfloat
#define CUMO_C double
#define CUMO_PART 2
#define CUMO_DOUBLE 1
#include "reduce_float.inc"
