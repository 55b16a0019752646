#define CUMO_T sfloat
#define CUMO_C float
#define CUMO_PART 2
#include "reduce_float.inc"
