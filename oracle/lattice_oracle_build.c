/* Builds both precisions of the scalar oracle into one library (see lattice_oracle.c). */
#define ORC_REAL float
#define ORC_SUFFIX _f32
#define ORC_IS_FLOAT 1
#include "lattice_oracle.c"
#undef ORC_REAL
#undef ORC_SUFFIX
#undef ORC_IS_FLOAT

#define ORC_REAL double
#define ORC_SUFFIX _f64
#define ORC_IS_FLOAT 0
#include "lattice_oracle.c"
