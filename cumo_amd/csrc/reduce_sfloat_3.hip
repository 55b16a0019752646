#define CUMO_T sfloat
#define CUMO_C float
#define CUMO_PART 3
#include "reduce_float.inc"
