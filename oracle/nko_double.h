/* Prefix of the oracle's double-precision build (test infrastructure; see nuka_oracle.h).
 *
 * Force-included ahead of every source (-include nko_double.h): the same restatement of the reference's algorithm
 * with every scalar, array and interface member a double and the rounding unit of its convergence tests that of
 * double.  What it computes is the answer the single-precision algorithm approximates; tests measure how far the
 * device's results and the single-precision oracle's lie from it.  The system headers come first so that only the
 * oracle's own text is affected. */
#ifndef NKO_DOUBLE_H_
#define NKO_DOUBLE_H_

#include <float.h>
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

typedef float nko_f32;   /* words that hold bit patterns (row flags, shape table entries, residual keys) stay 32 bits wide */
#define NKO_DOUBLE 1
#define float double
#undef FLT_EPSILON
#define FLT_EPSILON DBL_EPSILON
#define fabsf fabs
#define fmaxf fmax
#define fminf fmin
#define fmaf fma
#define sqrtf sqrt
#define powf pow
#define hypotf hypot
#define sinf sin
#define cosf cos
#define nextafterf nextafter

#endif
