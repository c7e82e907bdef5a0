/*
 * TEST INFRASTRUCTURE ONLY -- never linked into, imported by or called from the
 * shipped library. CPU restatement (plain C, optional OpenMP) of the algorithms
 * behind pytorch-loss's LabelSmoothSoftmaxCE / FocalLoss / LargeMarginSoftmax /
 * LovaszSoftmax and the ops next to them (OHEM relabelling, one-hot, Taylor softmax,
 * soft dice, channel layer norm), used by the tests as the parity checker and by the benchmark's
 * cpu_baseline leg. Every function in oracle_body.inc cites the reference lines
 * it follows and is pinned by tests/test_oracle_*.py without the reference (library
 * routines, closed forms, brute force, known answers worked by hand). Built by
 * oracle/build.py into oracle/liboracle.so.
 *
 * Each function exists as <name>_f32 (the arithmetic type of the shipped path)
 * and <name>_f64 (a higher-precision check on the fp32 restatement itself).
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>

#define REAL float
#define FN(name) name##_f32
#define EXP expf
#define LOG logf
#define LOG1P log1pf
#define POW powf
#define FABS fabsf
#define SQRT sqrtf
#include "oracle_body.inc"
#undef REAL
#undef FN
#undef EXP
#undef LOG
#undef LOG1P
#undef POW
#undef FABS
#undef SQRT

#define REAL double
#define FN(name) name##_f64
#define EXP exp
#define LOG log
#define LOG1P log1p
#define POW pow
#define FABS fabs
#define SQRT sqrt
#include "oracle_body.inc"

int oracle_abi_version(void) { return 1; }
