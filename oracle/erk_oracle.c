/*
 * TEST INFRASTRUCTURE ONLY.  Scalar CPU oracle for the batch-parallel adaptive
 * explicit Runge-Kutta solve loop of torchode (Dopri5 / Tsit5 with the integral
 * and PID step size controllers) on the built-in right-hand sides.
 *
 * It is a checker: only tests/, __graft_entry__.smoke() and the CPU-baseline
 * leg of bench.py load it.  The product library never links or calls it.
 *
 * The loop is restated literally: every sample of the batch is stepped in
 * every iteration until all have finished or one has failed (finished samples
 * take zero-length steps), evaluation points are tracked with a [B,E] pending
 * mask, and the batch-uniform f-evaluation counter advances by 6 per iteration.
 * Arithmetic follows the association that ATen's CPU kernels use at the
 * reference's call sites (documented next to each function in
 * erk_oracle_impl.h), with explicit fma() and floating point contraction
 * switched off at compile time.
 *
 * Deviations from an ATen evaluation, both on purpose and both harmless at
 * the stated tolerances:
 *   - pow() is oracle_pow_core below, a fixed sequence of IEEE double
 *     operations (so that an independent implementation can reproduce it
 *     bit for bit), not the vectorised library pow ATen calls;
 *   - Tsit5's dense output weights come from an exact rational expansion.
 *
 * Reference sites (torchode source tree):
 *   loop                adjoints.py:50-309
 *   RK step             single_step_methods/runge_kutta.py:226-279
 *   tableaux            single_step_methods/dopri5.py:11-44, tsit5.py:74-114
 *   dense weights       single_step_methods/tsit5.py:11-50
 *   quartic build/eval  tsit5.py:123-139, dopri5.py:53-60, interpolation.py:25-40,138-175
 *   controllers         step_size_controllers.py:170-181, 260-490, 554-835
 *
 * Pinning: every function here is checked in tests/test_oracle_pins.py against
 * closed forms / library special cases and against oracle/torch_loop.py (the
 * same loop issued as ATen operations).
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#include "erk_oracle.h"

/* ------------------------------------------------------------------------- */
/* pow(x, p) for x >= 0 as a fixed sequence of double operations:            */
/*   x = m 2^e, m in [1/sqrt2, sqrt2);  s = (m-1)/(m+1);                      */
/*   ln m = 2 s + s^3 (2/3 + 2 s^2/5 + ... + 2 s^18/21)                        */
/*   y = p (e + ln m / ln 2);  n = rint(y);  r = (y - n) ln 2                  */
/*   result = ldexp(sum_{i<=13} r^i / i!, n)                                   */
/* Relative error about 2e-15 for |y| < 20.                                   */
/* ------------------------------------------------------------------------- */
double oracle_pow_core(double x, double p) {
    if (p == 0.0) return 1.0;
    if (x != x || p != p) return NAN;
    if (x == 1.0) return 1.0;
    if (x < 0.0) return NAN;
    if (x == 0.0) return p > 0.0 ? 0.0 : INFINITY;
    if (isinf(x)) return p > 0.0 ? INFINITY : 0.0;
    if (isinf(p)) return ((x < 1.0) == (p > 0.0)) ? 0.0 : INFINITY;

    uint64_t bits;
    memcpy(&bits, &x, 8);
    int e = (int)((bits >> 52) & 0x7ff);
    if (e == 0) { /* subnormal: renormalise */
        x = x * 18014398509481984.0; /* 2^54 */
        memcpy(&bits, &x, 8);
        e = (int)((bits >> 52) & 0x7ff) - 54;
    }
    e -= 1023;
    bits = (bits & 0x000fffffffffffffULL) | 0x3ff0000000000000ULL;
    double m;
    memcpy(&m, &bits, 8);
    if (m > 1.4142135623730951) {
        m = m * 0.5;
        e += 1;
    }
    double s = (m - 1.0) / (m + 1.0);
    double z = s * s;
    double q = 2.0 / 21.0;
    q = fma(q, z, 2.0 / 19.0);
    q = fma(q, z, 2.0 / 17.0);
    q = fma(q, z, 2.0 / 15.0);
    q = fma(q, z, 2.0 / 13.0);
    q = fma(q, z, 2.0 / 11.0);
    q = fma(q, z, 2.0 / 9.0);
    q = fma(q, z, 2.0 / 7.0);
    q = fma(q, z, 2.0 / 5.0);
    q = fma(q, z, 2.0 / 3.0);
    double s3 = s * z;
    double lnm = fma(s3, q, 2.0 * s);
    double l2 = fma(lnm, 1.4426950408889634, (double)e);
    double y = p * l2;
    if (y > 1100.0) return INFINITY;
    if (y < -1100.0) return 0.0;
    double n = rint(y);
    double r = (y - n) * 0.6931471805599453;
    double v = 1.0 / 6227020800.0;
    v = fma(v, r, 1.0 / 479001600.0);
    v = fma(v, r, 1.0 / 39916800.0);
    v = fma(v, r, 1.0 / 3628800.0);
    v = fma(v, r, 1.0 / 362880.0);
    v = fma(v, r, 1.0 / 40320.0);
    v = fma(v, r, 1.0 / 5040.0);
    v = fma(v, r, 1.0 / 720.0);
    v = fma(v, r, 1.0 / 120.0);
    v = fma(v, r, 1.0 / 24.0);
    v = fma(v, r, 1.0 / 6.0);
    v = fma(v, r, 0.5);
    v = fma(v, r, 1.0);
    v = fma(v, r, 1.0);
    return ldexp(v, (int)n);
}

/* ------------------------------------------------------------------------- */
/* Butcher tableaux (float64, cast per use)                                   */
/* ------------------------------------------------------------------------- */
static oracle_tableau g_tab[2];
static int g_tab_ready = 0;

static void build_tableaux(void) {
    oracle_tableau *d = &g_tab[ORACLE_METHOD_DOPRI5], *t = &g_tab[ORACLE_METHOD_TSIT5];
    memset(g_tab, 0, sizeof(g_tab));
    /* Dormand-Prince 5(4), dopri5.py:11-44 */
    {
        const double c[7] = {0.0, 1.0 / 5, 3.0 / 10, 4.0 / 5, 8.0 / 9, 1.0, 1.0};
        const double a[7][7] = {
            {0},
            {1.0 / 5},
            {3.0 / 40, 9.0 / 40},
            {44.0 / 45, -56.0 / 15, 32.0 / 9},
            {19372.0 / 6561, -25360.0 / 2187, 64448.0 / 6561, -212.0 / 729},
            {9017.0 / 3168, -355.0 / 33, 46732.0 / 5247, 49.0 / 176, -5103.0 / 18656},
            {35.0 / 384, 0, 500.0 / 1113, 125.0 / 192, -2187.0 / 6784, 11.0 / 84},
        };
        const double b[7] = {35.0 / 384, 0, 500.0 / 1113, 125.0 / 192, -2187.0 / 6784, 11.0 / 84, 0.0};
        const double bl[7] = {1951.0 / 21600, 0, 22642.0 / 50085, 451.0 / 720, -12231.0 / 42400, 649.0 / 6300, 1.0 / 60};
        const double mid[7] = {6025192743.0 / 30085553152.0 / 2,    0,
                               51252292925.0 / 65400821598.0 / 2,   -2691868925.0 / 45128329728.0 / 2,
                               187940372067.0 / 1594534317056.0 / 2, -1776094331.0 / 19743644256.0 / 2,
                               11237099.0 / 235043384.0 / 2};
        memcpy(d->c, c, sizeof(c));
        memcpy(d->a, a, sizeof(a));
        memcpy(d->b, b, sizeof(b));
        for (int s = 0; s < 7; ++s) d->b_err[s] = b[s] - bl[s];
        memcpy(d->b_other[0], mid, sizeof(mid));
        d->n_other = 1;
    }
    /* Tsitouras 5(4), tsit5.py:74-114 */
    {
        const double c[7] = {0.0, 0.161, 0.327, 0.9, 0.9800255409045097, 1.0, 1.0};
        const double b[7] = {0.09646076681806523, 0.01, 0.4798896504144996, 1.379008574103742,
                             -3.290069515436081,  2.324710524099774, 0.0};
        const double a[7][7] = {
            {0},
            {0.161},
            {-0.008480655492356989, 0.335480655492357},
            {2.8971530571054935, -6.359448489975075, 4.3622954328695815},
            {5.325864828439257, -11.748883564062828, 7.4955393428898365, -0.09249506636175525},
            {5.86145544294642, -12.92096931784711, 8.159367898576159, -0.071584973281401, -0.02826905039406838},
            {0.09646076681806523, 0.01, 0.4798896504144996, 1.379008574103742, -3.290069515436081, 2.324710524099774},
        };
        const double be[7] = {0.00178001105222577714, 0.0008164344596567469, -0.007880878010261995, 0.1447110071732629,
                              -0.5823571654525552,    0.45808210592918697,   -1.0 / 66};
        /* theta^2..theta^4 monomial coefficients of the seven dense-output basis
         * polynomials (tsit5.py:27-35), expanded in exact rational arithmetic. */
        const double w[3][7] = {
            {-2.763706197274826, 0.13169999999999998, 3.930296236894751, -12.411077166933676, 37.50931341651104,
             -27.896526289197286, 1.5},
            {2.9132554618219126, -0.2234, -5.941033872131505, 30.33818863028232, -88.1789048947664, 65.09189467479366,
             -4.0},
            {-1.0530884977290216, 0.1017, 2.490627285651253, -16.548102889244902, 47.37952196281928,
             -34.87065786149661, 2.5},
        };
        memcpy(t->c, c, sizeof(c));
        memcpy(t->a, a, sizeof(a));
        memcpy(t->b, b, sizeof(b));
        memcpy(t->b_err, be, sizeof(be));
        memcpy(t->b_other, w, sizeof(w));
        t->n_other = 3;
    }
    g_tab_ready = 1;
}

const oracle_tableau *oracle_get_tableau(int method) {
    if (!g_tab_ready) build_tableaux();
    if (method != ORACLE_METHOD_DOPRI5 && method != ORACLE_METHOD_TSIT5) return NULL;
    return &g_tab[method];
}

/* ------------------------------------------------------------------------- */
/* float32 and float64 instantiations                                         */
/* ------------------------------------------------------------------------- */
#define REAL float
#define SFX(n) n##_f32
#define R_FMA(a, b, c) fmaf((a), (b), (c))
#define R_SQRT(a) sqrtf(a)
#define R_ABS(a) fabsf(a)
#define R_ISFINITE(a) isfinite(a)
#include "erk_oracle_impl.h"
#undef REAL
#undef SFX
#undef R_FMA
#undef R_SQRT
#undef R_ABS
#undef R_ISFINITE

#define REAL double
#define SFX(n) n##_f64
#define R_FMA(a, b, c) fma((a), (b), (c))
#define R_SQRT(a) sqrt(a)
#define R_ABS(a) fabs(a)
#define R_ISFINITE(a) isfinite(a)
#include "erk_oracle_impl.h"
