/*
 * TEST INFRASTRUCTURE ONLY.  CPU oracle for the GPT-2 training kernels: a
 * scalar C restatement of what the reference's task bodies compute.  Only the
 * tests, the smoke check and the benchmark's CPU-baseline leg may load this
 * library; nothing in the product path does.
 *
 * Built as oracle/_build/libcs_oracle.so by oracle/Makefile.  Every function
 * exists twice: name_f32 works in float (ATen's opmath type for float, half
 * and bfloat16 storage), name_f64 in double.
 */
#define _GNU_SOURCE
#include <math.h>
#include <stdint.h>
#include <stdlib.h>

#define CAT_(a, b) a##b
#define CAT(a, b) CAT_(a, b)

#define REAL float
#define FN(name) CAT(name, _f32)
#define SQRT sqrtf
#define ERF erff
#define TANH tanhf
#define EXP expf
#include "cs_oracle_body.h"
#undef REAL
#undef FN
#undef SQRT
#undef ERF
#undef TANH
#undef EXP

#define REAL double
#define FN(name) CAT(name, _f64)
#define SQRT sqrt
#define ERF erf
#define TANH tanh
#define EXP exp
#include "cs_oracle_body.h"

int oracle_abi_version(void) { return 1; }
