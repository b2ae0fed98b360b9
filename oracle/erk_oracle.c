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
 * Third-party arithmetic: the reference's pow runs in ATen, which calls the
 * SLEEF library's vectorised pow (vendored in PyTorch 2.10's third_party/sleef).
 * Its published algorithm is restated below and reproduces torch.pow bit for
 * bit (tests/test_oracle_pins.py).  Remaining deliberate deviation: Tsit5's
 * dense output weights come from an exact rational expansion (the reference
 * expands in floating point with sympy; last-ulp differences at most).
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
/* pow.  ATen's CPU kernels evaluate tensor ** scalar with the vectorised pow  */
/* of the SLEEF library (Sleef_powf*_u10 / Sleef_powd*_u10, FMA variants):     */
/* pow(x, y) = expk(logk(|x|) * y) in double-word arithmetic.  The published   */
/* algorithm is restated here operation by operation (every product, sum and   */
/* fused multiply-add is one IEEE operation in the working type), so that the  */
/* oracle reproduces ATen's results bit for bit and an independent             */
/* implementation can reproduce the oracle's.  Special cases are restated for  */
/* x >= 0 or NaN, which is all the solver produces.                            */
/* ------------------------------------------------------------------------- */
#define DW_DEFINE(T, P, FMA)                                                                                        \
    typedef struct { T x, y; } P##2;                                                                                \
    static inline P##2 P##mk(T x, T y) { P##2 r = {x, y}; return r; }                                               \
    static inline T P##fmapn(T x, T y, T z) { return FMA(x, y, -z); }                                               \
    static inline T P##fmanp(T x, T y, T z) { return FMA(-x, y, z); }                                               \
    static inline P##2 P##add2_s_s(T x, T y) { T s = x + y; T v = s - x; return P##mk(s, (x - (s - v)) + (y - v)); } \
    static inline P##2 P##add2_d_s(P##2 x, T y) { T s = x.x + y; T v = s - x.x; T t = (x.x - (s - v)) + (y - v); return P##mk(s, t + x.y); } \
    static inline P##2 P##add_s_d(T x, P##2 y) { T s = x + y.x; return P##mk(s, ((x - s) + y.x) + y.y); }            \
    static inline P##2 P##add_d_d(P##2 x, P##2 y) { T s = x.x + y.x; return P##mk(s, (((x.x - s) + y.x) + x.y) + y.y); } \
    static inline P##2 P##add2_d_d(P##2 x, P##2 y) { T s = x.x + y.x; T v = s - x.x; T t = (x.x - (s - v)) + (y.x - v); return P##mk(s, t + (x.y + y.y)); } \
    static inline P##2 P##scale(P##2 d, T s) { return P##mk(d.x * s, d.y * s); }                                    \
    static inline P##2 P##normalize(P##2 t) { T s = t.x + t.y; return P##mk(s, (t.x - s) + t.y); }                  \
    static inline P##2 P##div(P##2 n, P##2 d) {                                                                     \
        T t = (T)1 / d.x; T s = n.x * t; T u = P##fmapn(t, n.x, s);                                                 \
        T v = P##fmanp(d.y, t, P##fmanp(d.x, t, (T)1));                                                             \
        return P##mk(s, FMA(s, v, FMA(n.y, t, u)));                                                                 \
    }                                                                                                               \
    static inline P##2 P##squ(P##2 x) { T s = x.x * x.x; return P##mk(s, FMA(x.x + x.x, x.y, P##fmapn(x.x, x.x, s))); } \
    static inline P##2 P##mul_d_s(P##2 x, T y) { T s = x.x * y; return P##mk(s, FMA(x.y, y, P##fmapn(x.x, y, s))); }  \
    static inline P##2 P##mul_d_d(P##2 x, P##2 y) { T s = x.x * y.x; return P##mk(s, FMA(x.x, y.y, FMA(x.y, y.x, P##fmapn(x.x, y.x, s)))); }

DW_DEFINE(float, df, fmaf)
DW_DEFINE(double, dd, fma)

/* ---- float ---- */
static inline float f_pow2i(int q) { int32_t i = (int32_t)(q + 0x7f) << 23; float f; memcpy(&f, &i, 4); return f; }
static inline float f_ldexp2k(float d, int e) { return d * f_pow2i(e >> 1) * f_pow2i(e - (e >> 1)); }

static df2 f_logk(float d) {
    int o = d < 1.17549435e-38f;
    if (o) d = d * ((float)(INT64_C(1) << 32) * (float)(INT64_C(1) << 32));
    float d43 = d * (1.0f / 0.75f);
    int32_t bits;
    memcpy(&bits, &d43, 4);
    int e = ((bits >> 23) & 0xff) - 0x7f;
    memcpy(&bits, &d, 4);
    bits -= e << 23; /* d * 2^-e by exponent arithmetic */
    float m;
    memcpy(&m, &bits, 4);
    if (o) e -= 64;
    df2 x = dfdiv(dfadd2_s_s(-1.0f, m), dfadd2_s_s(1.0f, m));
    df2 x2 = dfsqu(x);
    float t = 0.240320354700088500976562f;
    t = fmaf(t, x2.x, 0.285112679004669189453125f);
    t = fmaf(t, x2.x, 0.400007992982864379882812f);
    df2 c = dfmk(0.66666662693023681640625f, 3.69183861259614332084311e-09f);
    df2 s = dfmul_d_s(dfmk(0.69314718246459960938f, -1.904654323148236017e-09f), (float)e);
    s = dfadd_d_d(s, dfscale(x, 2.0f));
    s = dfadd_d_d(s, dfmul_d_d(dfmul_d_d(x2, x), dfadd2_d_d(dfmul_d_s(x2, t), c)));
    return s;
}

static float f_expk(df2 d) {
    float u = (d.x + d.y) * 1.442695040888963407359924681001892137426645954152985934135449406931f;
    float fq = rintf(u);
    int q = (int)fq;
    df2 s = dfadd2_d_s(d, fq * -0.693145751953125f);
    s = dfadd2_d_s(s, fq * -1.428606765330187045e-06f);
    s = dfnormalize(s);
    u = 0.00136324646882712841033936f;
    u = fmaf(u, s.x, 0.00836596917361021041870117f);
    u = fmaf(u, s.x, 0.0416710823774337768554688f);
    u = fmaf(u, s.x, 0.166665524244308471679688f);
    u = fmaf(u, s.x, 0.499999850988388061523438f);
    df2 t = dfadd_d_d(s, dfmul_d_s(dfsqu(s), u));
    t = dfadd_s_d(1.0f, t);
    u = t.x + t.y;
    u = f_ldexp2k(u, q);
    if (d.x < -104.0f) u = 0.0f;
    return u;
}

float oracle_powf(float x, float y) {
    if (y == 0.0f || x == 1.0f) return 1.0f;
    if (x != x || y != y) return NAN;
    if (x < 0.0f) return NAN; /* not produced by the solver (negative base, non-integer exponent) */
    if (isinf(x) || x == 0.0f) return (((x == 0.0f) ? -y : y) < 0.0f) ? 0.0f : INFINITY;
    if (isinf(y)) { float efx = (y < 0 ? -1.0f : 1.0f) * (x - 1.0f); return efx < 0 ? 0.0f : (efx == 0 ? 1.0f : INFINITY); }
    float r = f_expk(dfmul_d_s(f_logk(x), y));
    return (r != r) ? INFINITY : r;
}

/* ---- double ---- */
static inline double d_pow2i(int q) { int64_t i = (int64_t)(q + 0x3ff) << 52; double f; memcpy(&f, &i, 8); return f; }
static inline double d_ldexp2k(double d, int e) { return d * d_pow2i(e >> 1) * d_pow2i(e - (e >> 1)); }

static dd2 d_logk(double d) {
    int o = d < 2.2250738585072014e-308;
    if (o) d = d * ((double)(INT64_C(1) << 32) * (double)(INT64_C(1) << 32));
    double d43 = d * (1.0 / 0.75);
    int64_t bits;
    memcpy(&bits, &d43, 8);
    int e = (int)((bits >> 52) & 0x7ff) - 0x3ff;
    memcpy(&bits, &d, 8);
    bits -= (int64_t)e << 52;
    double m;
    memcpy(&m, &bits, 8);
    if (o) e -= 64;
    dd2 x = dddiv(ddadd2_s_s(-1.0, m), ddadd2_s_s(1.0, m));
    dd2 x2 = ddsqu(x);
    double z = x2.x, z2 = z * z, z4 = z2 * z2, z8 = z4 * z4;
    /* Estrin evaluation of a degree-8 polynomial in z */
    double p01 = fma(z, 0.285714285714249172087875, 0.400000000000000077715612);
    double p23 = fma(z, 0.181818180850050775676507, 0.222222222230083560345903);
    double p45 = fma(z, 0.13332981086846273921509, 0.153846227114512262845736);
    double p67 = fma(z, 0.103239680901072952701192, 0.117754809412463995466069);
    double lo = fma(z2, p23, p01), hi = fma(z2, p67, p45);
    double t = fma(z8, 0.116255524079935043668677, fma(z4, hi, lo));
    dd2 c = ddmk(0.666666666666666629659233, 3.80554962542412056336616e-17);
    dd2 s = ddmul_d_s(ddmk(0.693147180559945286226764, 2.319046813846299558417771e-17), (double)e);
    s = ddadd_d_d(s, ddscale(x, 2.0));
    x = ddmul_d_d(x2, x);
    s = ddadd_d_d(s, ddmul_d_d(x, c));
    x = ddmul_d_d(x2, x);
    s = ddadd_d_d(s, ddmul_d_s(x, t));
    return s;
}

static double d_expk(dd2 d) {
    double u = (d.x + d.y) * 1.442695040888963407359924681001892137426645954152985934135449406931;
    double dq = rint(u);
    int q = (int)dq;
    dd2 s = ddadd2_d_s(d, dq * -.69314718055966295651160180568695068359375);
    s = ddadd2_d_s(s, dq * -.28235290563031577122588448175013436025525412068e-12);
    s = ddnormalize(s);
    double z = s.x, z2 = z * z, z4 = z2 * z2, z8 = z4 * z4;
    double p01 = fma(z, 0.166666666666666740681535, 0.500000000000000999200722);
    double p23 = fma(z, 0.00833333333332371417601081, 0.0416666666665409524128449);
    double p45 = fma(z, 0.000198412698809069797676111, 0.0013888888939977128960529);
    double p67 = fma(z, 2.75572496725023574143864e-06, 2.48014973989819794114153e-05);
    double p89 = fma(z, 2.51069683420950419527139e-08, 2.76286166770270649116855e-07);
    double lo = fma(z2, p23, p01), hi = fma(z2, p67, p45);
    u = fma(z8, p89, fma(z4, hi, lo));
    dd2 t = ddadd_s_d(1.0, s);
    t = ddadd_d_d(t, ddmul_d_s(ddsqu(s), u));
    u = t.x + t.y;
    u = d_ldexp2k(u, q);
    if (d.x < -1000.0) u = 0.0;
    return u;
}

double oracle_pow(double x, double y) {
    if (y == 0.0 || x == 1.0) return 1.0;
    if (x != x || y != y) return NAN;
    if (x < 0.0) return NAN;
    if (isinf(x) || x == 0.0) return (((x == 0.0) ? -y : y) < 0.0) ? 0.0 : INFINITY;
    if (isinf(y)) { double efx = (y < 0 ? -1.0 : 1.0) * (x - 1.0); return efx < 0 ? 0.0 : (efx == 0 ? 1.0 : INFINITY); }
    double r = d_expk(ddmul_d_s(d_logk(x), y));
    return (r != r) ? INFINITY : r;
}

void oracle_powf_array(const float *x, float y, float *out, int64_t n) { for (int64_t i = 0; i < n; ++i) out[i] = oracle_powf(x[i], y); }
void oracle_pow_array(const double *x, double y, double *out, int64_t n) { for (int64_t i = 0; i < n; ++i) out[i] = oracle_pow(x[i], y); }

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
            {2.9132554618219126, -0.2234, -5.941033872131505, 30.338188630282318, -88.1789048947664, 65.09189467479368,
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
#define R_POW(x, p) oracle_powf((x), (float)(p))
#include "erk_oracle_impl.h"
#undef R_POW
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
#define R_POW(x, p) oracle_pow((x), (double)(p))
#include "erk_oracle_impl.h"

/* tensor ** python_float, elementwise (the dispatch of rpow above) */
void oracle_rpowf_array(const float *x, double p, float *out, int64_t n) { for (int64_t i = 0; i < n; ++i) out[i] = rpow_f32(x[i], p); }
void oracle_rpow_array(const double *x, double p, double *out, int64_t n) { for (int64_t i = 0; i < n; ++i) out[i] = rpow_f64(x[i], p); }
