// java.util.Random on the host, so that a layer can be initialised with the very numbers a Java run of the reference
// draws: RandomUtils keeps one java.util.Random (RandomUtils.getInstance / setSeed, J/common/utils/RandomUtils.java:18-28)
// and RandomUtils.normal_ fills a tensor with (float)(std * nextGaussian() + mean), element after element
// (RandomUtils.java:697-703) - the initialiser of LlamaMLPLayer's three weights (LlamaMLPLayer.initLayers,
// J/engine/nn/layer/llama/LlamaMLPLayer.java:68-90: linear1, linear2, linear3, each normal_(n, 0.01f, 0.02f)).
// The generator is the one the Java SE specification of java.util.Random fixes: a 48-bit linear congruential generator
// (multiplier 0x5DEECE66D, increment 0xB), next(bits) = top bits of the state, nextDouble from 26 + 27 bits,
// nextGaussian by the polar method with the second value kept for the next call.  nextGaussian calls StrictMath.sqrt
// (correctly rounded everywhere) and StrictMath.log, which the specification ties to the fdlibm algorithm
// (__ieee754_log: argument reduction to [sqrt(2)/2, sqrt(2)], degree-14 polynomial in s = f/(2+f)); that algorithm is
// restated below, because the C library's log is a different one and differs from it in the last place on about 7 %
// of the arguments (new Random(42).nextGaussian() is 1.1419053154730547 with fdlibm's, one unit in the last place
// more with glibc's).  This file is compiled with -ffp-contract=off (every operation rounds once, as in Java).
// No GPU code in this file.
#include <math.h>
#include <string.h>

#include "omega_hip.h"

static double fdlibm_log(double x)
{
    static const double ln2_hi = 6.93147180369123816490e-01, ln2_lo = 1.90821492927058770002e-10,
                        two54 = 1.80143985094819840000e+16, Lg1 = 6.666666666666735130e-01,
                        Lg2 = 3.999999999940941908e-01, Lg3 = 2.857142874366239149e-01, Lg4 = 2.222219843214978396e-01,
                        Lg5 = 1.818357216161805012e-01, Lg6 = 1.531383769920937332e-01, Lg7 = 1.479819860511658591e-01;
    double hfsq, f, s, z, R, w, t1, t2, dk;
    int32_t k = 0, hx, i, j;
    uint64_t u;
    memcpy(&u, &x, 8);
    hx = (int32_t)(u >> 32);
    if (hx < 0x00100000) {  // x < 2^-1022: zero, negative or subnormal
        if (((hx & 0x7fffffff) | (uint32_t)u) == 0) return -two54 / 0.0;
        if (hx < 0) return (x - x) / 0.0;
        k -= 54;
        x *= two54;
        memcpy(&u, &x, 8);
        hx = (int32_t)(u >> 32);
    }
    if (hx >= 0x7ff00000) return x + x;
    k += (hx >> 20) - 1023;
    hx &= 0x000fffff;
    i = (hx + 0x95f64) & 0x100000;
    u = (u & 0xffffffffULL) | ((uint64_t)(uint32_t)(hx | (i ^ 0x3ff00000)) << 32);  // x or x/2 in [sqrt(2)/2, sqrt(2)]
    memcpy(&x, &u, 8);
    k += (i >> 20);
    f = x - 1.0;
    if ((0x000fffff & (2 + hx)) < 3) {  // |f| < 2^-20
        if (f == 0.0) {
            if (k == 0) return 0.0;
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

static const int64_t JR_MULT = 0x5DEECE66DLL, JR_MASK = (1LL << 48) - 1;

static int32_t jr_next(omega_jrandom *r, int bits)
{
    r->state = (int64_t)(((uint64_t)r->state * (uint64_t)JR_MULT + 0xBULL) & (uint64_t)JR_MASK);
    return (int32_t)(r->state >> (48 - bits));
}

extern "C" {

void omega_jrandom_seed(omega_jrandom *r, int64_t seed)
{
    r->state = (seed ^ JR_MULT) & JR_MASK;
    r->have_next_gaussian = 0;
    r->next_gaussian = 0.0;
}

int32_t omega_jrandom_next_int(omega_jrandom *r) { return jr_next(r, 32); }

double omega_jrandom_next_double(omega_jrandom *r)
{
    const int64_t hi = (int64_t)jr_next(r, 26) << 27;
    return (double)(hi + jr_next(r, 27)) * 0x1.0p-53;
}

double omega_jrandom_next_gaussian(omega_jrandom *r)
{
    if (r->have_next_gaussian) {
        r->have_next_gaussian = 0;
        return r->next_gaussian;
    }
    double v1, v2, s;
    do {
        v1 = 2 * omega_jrandom_next_double(r) - 1;
        v2 = 2 * omega_jrandom_next_double(r) - 1;
        s = v1 * v1 + v2 * v2;
    } while (s >= 1 || s == 0);
    const double multiplier = sqrt(-2 * fdlibm_log(s) / s);
    r->next_gaussian = v2 * multiplier;
    r->have_next_gaussian = 1;
    return v1 * multiplier;
}

void omega_jrandom_normal(omega_jrandom *r, float *out, size_t n, float mean, float std)
{
    for (size_t i = 0; i < n; ++i) out[i] = (float)((double)std * omega_jrandom_next_gaussian(r) + (double)mean);
}

}  // extern "C"
