/*
 * TEST INFRASTRUCTURE ONLY - CPU oracle (see jrandom.h).
 *
 * java.util.Random per the JDK specification, plus the fdlibm logarithm that
 * StrictMath.log is defined to be (freely distributable algorithm, Sun
 * Microsystems 1993; restated here, compiled with -ffp-contract=off so no
 * multiply-add is fused, as Java's strict floating point requires).
 */
#include "jrandom.h"

#include <math.h>
#include <string.h>

#define JR_MULT 0x5DEECE66DULL
#define JR_ADD  0xBULL
#define JR_MASK ((1ULL << 48) - 1)

void jr_init(jrandom *r, int64_t seed) {
    r->seed = ((uint64_t)seed ^ JR_MULT) & JR_MASK;
    r->have_next = 0;
    r->next_next = 0.0;
}

int32_t jr_next(jrandom *r, int bits) {
    r->seed = (r->seed * JR_MULT + JR_ADD) & JR_MASK;
    return (int32_t)(uint32_t)(r->seed >> (48 - bits));
}

int32_t jr_next_int(jrandom *r) { return jr_next(r, 32); }

int32_t jr_next_int_bound(jrandom *r, int32_t bound) {
    /* bound must be > 0 (Java throws IllegalArgumentException otherwise). */
    int32_t v = jr_next(r, 31);
    int32_t m = bound - 1;
    if ((bound & m) == 0) {
        return (int32_t)(((int64_t)bound * (int64_t)v) >> 31);
    }
    for (;;) {
        int32_t u = v;
        v = u % bound;
        /* Java int arithmetic wraps: u - v + m < 0 detects the biased tail. */
        uint32_t w = (uint32_t)u - (uint32_t)v + (uint32_t)m;
        if ((int32_t)w >= 0) return v;
        v = jr_next(r, 31);
    }
}

float jr_next_float(jrandom *r) {
    return (float)jr_next(r, 24) / (float)(1 << 24);
}

double jr_next_double(jrandom *r) {
    int64_t hi = (int64_t)jr_next(r, 26);
    int64_t lo = (int64_t)jr_next(r, 27);
    return (double)((hi << 27) + lo) * 0x1.0p-53;
}

double jr_next_gaussian(jrandom *r) {
    if (r->have_next) {
        r->have_next = 0;
        return r->next_next;
    }
    double v1, v2, s;
    do {
        v1 = 2 * jr_next_double(r) - 1;
        v2 = 2 * jr_next_double(r) - 1;
        s = v1 * v1 + v2 * v2;
    } while (s >= 1 || s == 0);
    double multiplier = sqrt(-2 * fdlibm_log(s) / s);   /* StrictMath.sqrt is correctly rounded */
    r->next_next = v2 * multiplier;
    r->have_next = 1;
    return v1 * multiplier;
}

/* ------------------------------------------------------------------ */
/* fdlibm e_log.c                                                      */
/* ------------------------------------------------------------------ */

static const double
    ln2_hi = 6.93147180369123816490e-01,
    ln2_lo = 1.90821492927058770002e-10,
    two54  = 1.80143985094819840000e+16,
    Lg1 = 6.666666666666735130e-01,
    Lg2 = 3.999999999940941908e-01,
    Lg3 = 2.857142874366239149e-01,
    Lg4 = 2.222219843214978396e-01,
    Lg5 = 1.818357216161805012e-01,
    Lg6 = 1.531383769920937332e-01,
    Lg7 = 1.479819860511658591e-01;

static inline int32_t hi_word(double x) {
    uint64_t u; memcpy(&u, &x, 8); return (int32_t)(u >> 32);
}
static inline uint32_t lo_word(double x) {
    uint64_t u; memcpy(&u, &x, 8); return (uint32_t)u;
}
static inline double with_hi(double x, int32_t hi) {
    uint64_t u; memcpy(&u, &x, 8);
    u = (u & 0xffffffffULL) | ((uint64_t)(uint32_t)hi << 32);
    memcpy(&x, &u, 8); return x;
}

double fdlibm_log(double x) {
    static const double zero = 0.0;
    double hfsq, f, s, z, R, w, t1, t2, dk;
    int32_t k, hx, i, j;
    uint32_t lx;

    hx = hi_word(x);
    lx = lo_word(x);

    k = 0;
    if (hx < 0x00100000) {                       /* x < 2**-1022 */
        if (((hx & 0x7fffffff) | lx) == 0) return -two54 / zero;   /* log(+-0) = -inf */
        if (hx < 0) return (x - x) / zero;                         /* log(-#) = NaN */
        k -= 54; x *= two54;                                       /* subnormal: scale up */
        hx = hi_word(x);
    }
    if (hx >= 0x7ff00000) return x + x;
    k += (hx >> 20) - 1023;
    hx &= 0x000fffff;
    i = (hx + 0x95f64) & 0x100000;
    x = with_hi(x, hx | (i ^ 0x3ff00000));       /* normalize x or x/2 */
    k += (i >> 20);
    f = x - 1.0;
    if ((0x000fffff & (2 + hx)) < 3) {           /* |f| < 2**-20 */
        if (f == zero) {
            if (k == 0) return zero;
            dk = (double)k;
            return dk * ln2_hi + dk * ln2_lo;
        }
        R = f * f * (0.5 - 0.33333333333333333 * f);
        if (k == 0) return f - R;
        dk = (double)k;
        return dk * ln2_hi - ((R - dk * ln2_lo) - f);
    }
    s = f / (2.0 + f);
    dk = (double)k;
    z = s * s;
    i = hx - 0x6147a;
    w = z * z;
    j = 0x6b851 - hx;
    t1 = w * (Lg2 + w * (Lg4 + w * Lg6));
    t2 = z * (Lg1 + w * (Lg3 + w * (Lg5 + w * Lg7)));
    i |= j;
    R = t2 + t1;
    if (i > 0) {
        hfsq = 0.5 * f * f;
        if (k == 0) return f - (hfsq - s * (hfsq + R));
        return dk * ln2_hi - ((hfsq - (s * (hfsq + R) + dk * ln2_lo)) - f);
    }
    if (k == 0) return f - s * (f - R);
    return dk * ln2_hi - ((s * (f - R) - dk * ln2_lo) - f);
}
