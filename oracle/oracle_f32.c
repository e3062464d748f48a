/* float instantiation of the CPU oracle (test infrastructure only; see oracle.h). */
#define REAL float
#define FN(name) name##_f32
#define R_EXP expf
#define R_SQRT sqrtf
#define R_LOG1P log1pf
#include "oracle_impl.h"
