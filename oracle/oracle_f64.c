/* double instantiation of the CPU oracle (test infrastructure only; see oracle.h). */
#define REAL double
#define FN(name) name##_f64
#define R_EXP exp
#define R_SQRT sqrt
#define R_LOG1P log1p
#include "oracle_impl.h"
