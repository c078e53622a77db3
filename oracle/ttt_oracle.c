/* CPU restatement (plain C + OpenMP) of the reference's TTT-Linear / TTT-MLP inner models.
 * TEST INFRASTRUCTURE ONLY: used by the tests as a second checker and by the benchmark as the
 * host-CPU baseline; the product library never links or calls it.
 * Built by oracle/Makefile into oracle/_build/libttt_oracle.so. */
#include <math.h>
#include <stddef.h>
#include <stdlib.h>
#include <string.h>

#define REAL float
#define SUF f32
#include "ttt_oracle_body.inc"
#undef REAL
#undef SUF

#define REAL double
#define SUF f64
#include "ttt_oracle_body.inc"
#undef REAL
#undef SUF
