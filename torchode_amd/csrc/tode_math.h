// Device-side arithmetic shared by the persistent and per-step kernels.
//
// Everything here is written so that the result of every floating point
// operation is fixed by IEEE-754: products and sums are fused only where
// fma_() is spelled out (the translation unit is compiled with
// -ffp-contract=off), divisions and square roots are the correctly rounded
// ones, and pow is a fixed sequence of double operations.  The association of
// each formula follows what ATen's CPU kernels compute at the corresponding
// torchode call site, which is what makes results comparable bit for bit with
// a CPU evaluation of the reference.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace tode {

template <typename T> __device__ __forceinline__ T fma_(T a, T b, T c);
template <> __device__ __forceinline__ float fma_<float>(float a, float b, float c) { return __builtin_fmaf(a, b, c); }
template <> __device__ __forceinline__ double fma_<double>(double a, double b, double c) { return __builtin_fma(a, b, c); }

template <typename T> __device__ __forceinline__ T sqrt_(T a);
template <> __device__ __forceinline__ float sqrt_<float>(float a) { return __builtin_sqrtf(a); }
template <> __device__ __forceinline__ double sqrt_<double>(double a) { return __builtin_sqrt(a); }

template <typename T> __device__ __forceinline__ T abs_(T a);
template <> __device__ __forceinline__ float abs_<float>(float a) { return __builtin_fabsf(a); }
template <> __device__ __forceinline__ double abs_<double>(double a) { return __builtin_fabs(a); }

template <typename T> __device__ __forceinline__ bool finite_(T a) { return abs_(a) < __builtin_huge_val(); }

// torch.maximum / torch.minimum / torch.clamp: NaN in any operand gives NaN.  Written as
// max/min plus one unordered-compare select so that it stays straight-line code.
template <typename T> __device__ __forceinline__ T nan_();
template <> __device__ __forceinline__ float nan_<float>() { return __builtin_nanf(""); }
template <> __device__ __forceinline__ double nan_<double>() { return __builtin_nan(""); }
__device__ __forceinline__ float hwmax(float a, float b) { return __builtin_fmaxf(a, b); }
__device__ __forceinline__ double hwmax(double a, double b) { return __builtin_fmax(a, b); }
__device__ __forceinline__ float hwmin(float a, float b) { return __builtin_fminf(a, b); }
__device__ __forceinline__ double hwmin(double a, double b) { return __builtin_fmin(a, b); }
template <typename T> __device__ __forceinline__ T tmax(T a, T b) { return __builtin_isunordered(a, b) ? nan_<T>() : hwmax(a, b); }
template <typename T> __device__ __forceinline__ T tmin(T a, T b) { return __builtin_isunordered(a, b) ? nan_<T>() : hwmin(a, b); }
template <typename T> __device__ __forceinline__ T tclamp(T x, T lo, T hi) { return tmin(tmax(x, lo), hi); }

// pow(x, p) for x >= 0:  x = m 2^e with m in [1/sqrt2, sqrt2), s = (m-1)/(m+1),
// ln m = 2s + s^3 (2/3 + 2 s^2/5 + ... + 2 s^18/21), y = p (e + ln m / ln 2),
// n = rint(y), r = (y-n) ln 2, result = ldexp(sum_{i<=13} r^i/i!, n).
// Relative error about 2e-15 for |y| < 20.
__device__ __forceinline__ double pow_core(double x, double p) {
    if (p == 0.0) return 1.0;
    if (x != x || p != p) return __builtin_nan("");
    if (x == 1.0) return 1.0;
    if (x < 0.0) return __builtin_nan("");
    if (x == 0.0) return p > 0.0 ? 0.0 : __builtin_huge_val();
    if (x == __builtin_huge_val()) return p > 0.0 ? __builtin_huge_val() : 0.0;
    if (__builtin_fabs(p) == __builtin_huge_val()) return ((x < 1.0) == (p > 0.0)) ? 0.0 : __builtin_huge_val();

    uint64_t bits = (uint64_t)__double_as_longlong(x);
    int e = (int)((bits >> 52) & 0x7ff);
    if (e == 0) {
        x = x * 18014398509481984.0;
        bits = (uint64_t)__double_as_longlong(x);
        e = (int)((bits >> 52) & 0x7ff) - 54;
    }
    e -= 1023;
    bits = (bits & 0x000fffffffffffffULL) | 0x3ff0000000000000ULL;
    double m = __longlong_as_double((long long)bits);
    if (m > 1.4142135623730951) {
        m = m * 0.5;
        e += 1;
    }
    double s = (m - 1.0) / (m + 1.0);
    double z = s * s;
    double q = 2.0 / 21.0;
    q = __builtin_fma(q, z, 2.0 / 19.0);
    q = __builtin_fma(q, z, 2.0 / 17.0);
    q = __builtin_fma(q, z, 2.0 / 15.0);
    q = __builtin_fma(q, z, 2.0 / 13.0);
    q = __builtin_fma(q, z, 2.0 / 11.0);
    q = __builtin_fma(q, z, 2.0 / 9.0);
    q = __builtin_fma(q, z, 2.0 / 7.0);
    q = __builtin_fma(q, z, 2.0 / 5.0);
    q = __builtin_fma(q, z, 2.0 / 3.0);
    double s3 = s * z;
    double lnm = __builtin_fma(s3, q, 2.0 * s);
    double l2 = __builtin_fma(lnm, 1.4426950408889634, (double)e);
    double y = p * l2;
    if (y > 1100.0) return __builtin_huge_val();
    if (y < -1100.0) return 0.0;
    double n = __builtin_rint(y);
    double r = (y - n) * 0.6931471805599453;
    double v = 1.0 / 6227020800.0;
    v = __builtin_fma(v, r, 1.0 / 479001600.0);
    v = __builtin_fma(v, r, 1.0 / 39916800.0);
    v = __builtin_fma(v, r, 1.0 / 3628800.0);
    v = __builtin_fma(v, r, 1.0 / 362880.0);
    v = __builtin_fma(v, r, 1.0 / 40320.0);
    v = __builtin_fma(v, r, 1.0 / 5040.0);
    v = __builtin_fma(v, r, 1.0 / 720.0);
    v = __builtin_fma(v, r, 1.0 / 120.0);
    v = __builtin_fma(v, r, 1.0 / 24.0);
    v = __builtin_fma(v, r, 1.0 / 6.0);
    v = __builtin_fma(v, r, 0.5);
    v = __builtin_fma(v, r, 1.0);
    v = __builtin_fma(v, r, 1.0);
    return __builtin_ldexp(v, (int)n);
}

// The two halves of pow_core for arguments that need none of its special cases:
// log2_normal(x) for a positive, finite, normal x, and exp2_of(y) for |y| <= 1016.
// pow_core(x, p) == exp2_of(p * log2_normal(x)) bit for bit on that domain, which lets
// a caller reuse one logarithm for several exponents.
__device__ __forceinline__ double log2_normal(double x) {
    const unsigned hi = (unsigned)__double2hiint(x);
    int e = (int)((hi >> 20) & 0x7ff) - 1023;
    double m = __hiloint2double((int)((hi & 0x000fffffu) | 0x3ff00000u), __double2loint(x));
    const bool big = m > 1.4142135623730951;
    m = big ? m * 0.5 : m;
    e = big ? e + 1 : e;
    double s = (m - 1.0) / (m + 1.0);
    double z = s * s;
    double q = 2.0 / 21.0;
    q = __builtin_fma(q, z, 2.0 / 19.0);
    q = __builtin_fma(q, z, 2.0 / 17.0);
    q = __builtin_fma(q, z, 2.0 / 15.0);
    q = __builtin_fma(q, z, 2.0 / 13.0);
    q = __builtin_fma(q, z, 2.0 / 11.0);
    q = __builtin_fma(q, z, 2.0 / 9.0);
    q = __builtin_fma(q, z, 2.0 / 7.0);
    q = __builtin_fma(q, z, 2.0 / 5.0);
    q = __builtin_fma(q, z, 2.0 / 3.0);
    double s3 = s * z;
    double lnm = __builtin_fma(s3, q, 2.0 * s);
    return __builtin_fma(lnm, 1.4426950408889634, (double)e);
}

__device__ __forceinline__ double exp2_of(double y) {
    double n = __builtin_rint(y);
    double r = (y - n) * 0.6931471805599453;
    double v = 1.0 / 6227020800.0;
    v = __builtin_fma(v, r, 1.0 / 479001600.0);
    v = __builtin_fma(v, r, 1.0 / 39916800.0);
    v = __builtin_fma(v, r, 1.0 / 3628800.0);
    v = __builtin_fma(v, r, 1.0 / 362880.0);
    v = __builtin_fma(v, r, 1.0 / 40320.0);
    v = __builtin_fma(v, r, 1.0 / 5040.0);
    v = __builtin_fma(v, r, 1.0 / 720.0);
    v = __builtin_fma(v, r, 1.0 / 120.0);
    v = __builtin_fma(v, r, 1.0 / 24.0);
    v = __builtin_fma(v, r, 1.0 / 6.0);
    v = __builtin_fma(v, r, 0.5);
    v = __builtin_fma(v, r, 1.0);
    v = __builtin_fma(v, r, 1.0);
    return __builtin_ldexp(v, (int)n);
}

// Tensor ** python_float: the exponent is rounded to the tensor dtype first.
template <typename T> __device__ __forceinline__ T rpow(T x, double p) { return (T)pow_core((double)x, (double)(T)p); }

// ---------------------------------------------------------------------------
// Butcher tableaux, float64 literals cast to the working type where used
// (torchode single_step_methods/dopri5.py:11-44, tsit5.py:74-114).
// ---------------------------------------------------------------------------
struct Dopri5Tab {
    static constexpr int n_other = 1;
    static constexpr double c[7] = {0.0, 1.0 / 5, 3.0 / 10, 4.0 / 5, 8.0 / 9, 1.0, 1.0};
    static constexpr double a[7][7] = {
        {0},
        {1.0 / 5},
        {3.0 / 40, 9.0 / 40},
        {44.0 / 45, -56.0 / 15, 32.0 / 9},
        {19372.0 / 6561, -25360.0 / 2187, 64448.0 / 6561, -212.0 / 729},
        {9017.0 / 3168, -355.0 / 33, 46732.0 / 5247, 49.0 / 176, -5103.0 / 18656},
        {35.0 / 384, 0, 500.0 / 1113, 125.0 / 192, -2187.0 / 6784, 11.0 / 84},
    };
    // b - b_low, subtracted in float64 (runge_kutta.py:84-88)
    static constexpr double b_err[7] = {35.0 / 384 - 1951.0 / 21600,
                                        0.0 - 0.0,
                                        500.0 / 1113 - 22642.0 / 50085,
                                        125.0 / 192 - 451.0 / 720,
                                        -2187.0 / 6784 - -12231.0 / 42400,
                                        11.0 / 84 - 649.0 / 6300,
                                        0.0 - 1.0 / 60};
    // mid-point weights
    static constexpr double w[3][7] = {{6025192743.0 / 30085553152.0 / 2, 0, 51252292925.0 / 65400821598.0 / 2,
                                        -2691868925.0 / 45128329728.0 / 2, 187940372067.0 / 1594534317056.0 / 2,
                                        -1776094331.0 / 19743644256.0 / 2, 11237099.0 / 235043384.0 / 2},
                                       {0},
                                       {0}};
};

struct Tsit5Tab {
    static constexpr int n_other = 3;
    static constexpr double c[7] = {0.0, 0.161, 0.327, 0.9, 0.9800255409045097, 1.0, 1.0};
    static constexpr double a[7][7] = {
        {0},
        {0.161},
        {-0.008480655492356989, 0.335480655492357},
        {2.8971530571054935, -6.359448489975075, 4.3622954328695815},
        {5.325864828439257, -11.748883564062828, 7.4955393428898365, -0.09249506636175525},
        {5.86145544294642, -12.92096931784711, 8.159367898576159, -0.071584973281401, -0.02826905039406838},
        {0.09646076681806523, 0.01, 0.4798896504144996, 1.379008574103742, -3.290069515436081, 2.324710524099774},
    };
    static constexpr double b_err[7] = {0.00178001105222577714, 0.0008164344596567469, -0.007880878010261995,
                                        0.1447110071732629,     -0.5823571654525552,    0.45808210592918697,
                                        -1.0 / 66};
    // theta^2, theta^3, theta^4 monomial coefficients of the seven dense-output basis
    // polynomials of the Tsitouras pair (tsit5.py:27-35), expanded in exact rational
    // arithmetic and rounded once.
    static constexpr double w[3][7] = {
        {-2.763706197274826, 0.13169999999999998, 3.930296236894751, -12.411077166933676, 37.50931341651104,
         -27.896526289197286, 1.5},
        {2.9132554618219126, -0.2234, -5.941033872131505, 30.33818863028232, -88.1789048947664, 65.09189467479366,
         -4.0},
        {-1.0530884977290216, 0.1017, 2.490627285651253, -16.548102889244902, 47.37952196281928, -34.87065786149661,
         2.5},
    };
};

// ---------------------------------------------------------------------------
// Controller parameters in the working type
// ---------------------------------------------------------------------------
template <typename T> struct CtrlParams {
    T atol, rtol;              // float32-rounded tolerances
    T safety, fmin, fmax;      // factor clipping
    T dt_min, dt_max;
    double e1, e2, e3;         // pow exponents: ratio, prev, prev_prev
    int has_dt_min, has_dt_max;
    int skip2, skip3;          // exponent is +-0: the factor is exactly 1
};

// rms_norm over F register values (step_size_controllers.py:170-181); ATen's CPU
// vector_norm fuses the chain for F <= 3 and rounds the squares first for F >= 4.
template <typename T, int F> __device__ __forceinline__ T rms(const T (&v)[F]) {
    const T sf = (T)__builtin_sqrt((double)F);
    T acc = 0;
#pragma unroll
    for (int f = 0; f < F; ++f) {
        T x = v[f] / sf;
        if (F <= 3)
            acc = fma_(x, x, acc);
        else {
            T sq = x * x;
            acc = acc + sq;
        }
    }
    return sqrt_(acc);
}

// sum_s round(dt*w_s) * k_s, products rounded before they are added
// (einsum "b, s, sbf -> bf" on the small-matrix path, F <= 57).  The weights are
// row ROW of Tab::w, or Tab::b_err for ROW < 0; they are named by template
// arguments so that the float64 -> T conversion happens at compile time.
template <typename T, int F, typename Tab, int ROW>
__device__ __forceinline__ void weighted_k(T dt, const T (&k)[7][F], T (&out)[F]) {
#pragma unroll
    for (int f = 0; f < F; ++f) out[f] = 0;
#pragma unroll
    for (int s = 0; s < 7; ++s) {
        constexpr int R = ROW < 0 ? 0 : ROW;
        const T ws = ROW < 0 ? (T)Tab::b_err[s] : (T)Tab::w[R][s];
        T p = dt * ws;
#pragma unroll
        for (int f = 0; f < F; ++f) {
            T pk = p * k[s][f];
            out[f] = out[f] + pk;
        }
    }
}

// Error ratio (step_size_controllers.py:393-401, 738-746).
template <typename T, int F>
__device__ __forceinline__ T error_ratio(const CtrlParams<T> &cp, const T (&y0)[F], const T (&y1)[F], const T (&err)[F]) {
    T q[F];
#pragma unroll
    for (int f = 0; f < F; ++f) {
        T m = tmax(abs_(y0[f]), abs_(y1[f]));
        T eb = fma_(cp.rtol, m, cp.atol);
        q[f] = abs_(err[f]) / eb;
    }
    return tmax(rms<T, F>(q), (T)1e-38);
}

// dt factor (step_size_controllers.py:289-294, 598-620).
template <typename T, int CTRL> __device__ __forceinline__ T dt_factor(const CtrlParams<T> &cp, T ratio, T prev, T prev_prev) {
    T factor = cp.safety * rpow<T>(ratio, cp.e1);
    if (CTRL == 1) {
        T f2 = cp.skip2 ? (T)1 : rpow<T>(prev, cp.e2);
        T f3 = cp.skip3 ? (T)1 : rpow<T>(prev_prev, cp.e3);
        factor = factor * f2;
        factor = factor * f3;
    }
    return tclamp(factor, cp.fmin, cp.fmax);
}

// dt_min / dt_max enforcement and status (step_size_controllers.py:406-422, 751-767).
template <typename T> __device__ __forceinline__ int limit_dt(const CtrlParams<T> &cp, T ratio, T &dt_next) {
    int status = finite_(ratio) ? 0 : 4;
    if (cp.has_dt_min || cp.has_dt_max) {
        T mag = abs_(dt_next);
        T c = mag;
        if (cp.has_dt_min) c = tmax(c, cp.dt_min);
        if (cp.has_dt_max) c = tmin(c, cp.dt_max);
        T sg = (dt_next > 0) ? (T)1 : ((dt_next < 0) ? (T)-1 : dt_next);
        dt_next = sg * c;
        if (cp.has_dt_min && mag < cp.dt_min) status = 2;
    }
    return status;
}

// Quartic coefficients of the dense output, lowest power first.
// Tsit5: tsit5.py:123-139.  Dopri5: dopri5.py:53-60 -> interpolation.py:138-170.
template <typename T, int F, int METHOD>
__device__ __forceinline__ void quartic(T dt, const T (&y0)[F], const T (&y1)[F], const T (&k)[7][F], T (&q)[5][F]) {
    if (METHOD == 1) {
#pragma unroll
        for (int f = 0; f < F; ++f) {
            q[0][f] = y0[f];
            q[1][f] = dt * k[0][f];
        }
        weighted_k<T, F, Tsit5Tab, 0>(dt, k, q[2]);
        weighted_k<T, F, Tsit5Tab, 1>(dt, k, q[3]);
        weighted_k<T, F, Tsit5Tab, 2>(dt, k, q[4]);
    } else {
        T ymid[F];
        weighted_k<T, F, Dopri5Tab, 0>(dt, k, ymid);
#pragma unroll
        for (int f = 0; f < F; ++f) {
            T f0 = dt * k[0][f], f1 = dt * k[6][f];
            T ym = y0[f] + ymid[f];
            T df = f1 - f0;
            T sy = y1[f] + y0[f];
            T a = (T)2 * df;
            a = fma_((T)-8, sy, a);
            a = fma_((T)16, ym, a);
            T b = (T)5 * f0;
            b = fma_((T)-3, f1, b);
            b = fma_((T)18, y0[f], b);
            b = fma_((T)14, y1[f], b);
            b = fma_((T)-32, ym, b);
            T c = fma_((T)-4, f0, f1);
            c = fma_((T)-11, y0[f], c);
            c = fma_((T)-5, y1[f], c);
            c = fma_((T)16, ym, c);
            q[0][f] = y0[f];
            q[1][f] = f0;
            q[2][f] = c;
            q[3][f] = b;
            q[4][f] = a;
        }
    }
}

// Horner on x = (t - t0) / ((t0 + dt) - t0), interpolation.py:25-40.
template <typename T, int F> __device__ __forceinline__ void quartic_eval(const T (&q)[5][F], T t0, T dt, T t, T (&out)[F]) {
    T t1 = t0 + dt;
    T den = t1 - t0;
    if (!(abs_(den) > (T)0)) den = (T)1;
    T x = (t - t0) / den;
#pragma unroll
    for (int f = 0; f < F; ++f) {
        T y = q[4][f];
        y = fma_(y, x, q[3][f]);
        y = fma_(y, x, q[2][f]);
        y = fma_(y, x, q[1][f]);
        y = fma_(y, x, q[0][f]);
        out[f] = y;
    }
}

}  // namespace tode
