/*
 * TEST INFRASTRUCTURE ONLY - CPU oracle for the DeepJ HIP backend.
 * Nothing in the shipped library links or loads this code.
 *
 * Restatement of java.util.Random as specified by the JDK Javadoc (the class
 * is not part of the reference tree; its algorithm is fixed by that spec):
 * 48-bit LCG, next(bits), nextInt, nextInt(bound), nextFloat, nextDouble and
 * the Marsaglia polar nextGaussian with its cached second value.  The
 * reference draws every seeded weight through it:
 *   src/main/java/io/github/kirstenali/deepj/tensor/cpu/CpuBackend.java:148-152
 */
#ifndef DEEPJ_ORACLE_JRANDOM_H
#define DEEPJ_ORACLE_JRANDOM_H

#include <stdint.h>

typedef struct {
    uint64_t seed;       /* 48-bit LCG state */
    int have_next;       /* haveNextNextGaussian */
    double next_next;    /* nextNextGaussian */
} jrandom;

void    jr_init(jrandom *r, int64_t seed);
int32_t jr_next(jrandom *r, int bits);
int32_t jr_next_int(jrandom *r);
int32_t jr_next_int_bound(jrandom *r, int32_t bound);
float   jr_next_float(jrandom *r);
double  jr_next_double(jrandom *r);
double  jr_next_gaussian(jrandom *r);

/* fdlibm __ieee754_log, which is what StrictMath.log evaluates. */
double  fdlibm_log(double x);

#endif
