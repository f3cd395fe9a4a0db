/*
 * TEST INFRASTRUCTURE ONLY -- CPU oracle for the SRWM and delta-rule recurrences,
 * built for float and double from one body (fastweight_oracle_impl.h, which
 * carries the citations of the reference files it follows).  The product never
 * links or loads this library; tests, the smoke check and the bench's CPU
 * baseline leg do.
 */
#include <math.h>
#include <stddef.h>
#include <stdlib.h>

#define REAL double
#define SUFFIX f64
#include "fastweight_oracle_impl.h"
#undef REAL
#undef SUFFIX

#define REAL float
#define SUFFIX f32
#include "fastweight_oracle_impl.h"
#undef REAL
#undef SUFFIX
