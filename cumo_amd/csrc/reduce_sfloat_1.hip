#define CUMO_T sfloat
#define CUMO_C float
#define CUMO_PART 1
#include "reduce_float.inc"
