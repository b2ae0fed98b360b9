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

// A sample that has finished on t_end keeps stepping in the reference's later iterations with dt = 0, which is seen in
// the status of those steps alone: a success as long as their error ratio is finite.  With dt = 0 every stage is
// evaluated at y itself, so every stage derivative is k0 again, the stage sums are a_i1 k0 + a_i2 k0 + ..., and the
// step's result and error estimate are y and 0 -- provided no such sum overflows (0 * inf is NaN).  The tableaus'
// |a_ij| sum to less than 32 per row: a value and derivative that pass this test cannot produce anything but status 0.
template <typename T> __device__ __forceinline__ bool settles_(T y, T k0) {
    return finite_(y) && abs_(k0) <= (T)(sizeof(T) == 4 ? 0x1p+122 : 0x1p+1018);  // (the largest finite value / 64; false for NaN)
}

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

// ---------------------------------------------------------------------------
// pow.  The reference's `tensor ** python_float` is evaluated by ATen's CPU kernels with
// the SLEEF library's vectorised pow (u10, FMA variants): pow(x, y) = expk(logk(|x|) * y)
// in double-word arithmetic.  That published algorithm is written out here operation by
// operation -- every sum, product and fma below is one IEEE operation in the working
// type -- which makes the device result identical, bit for bit, to what the reference
// computes on the host.  logk() and expk() are exposed separately so that a caller can
// reuse one logarithm for several exponents.  Special cases are covered for x >= 0 or
// NaN, which is all the step size controllers produce.
// ---------------------------------------------------------------------------
template <typename T> struct DW { T x, y; };  // unevaluated sum x + y, |y| <= ulp(x)/2

template <typename T> __device__ __forceinline__ DW<T> dw(T x, T y) { return DW<T>{x, y}; }
template <typename T> __device__ __forceinline__ T fmapn(T x, T y, T z) { return fma_(x, y, -z); }
template <typename T> __device__ __forceinline__ T fmanp(T x, T y, T z) { return fma_(-x, y, z); }
template <typename T> __device__ __forceinline__ DW<T> dw_add2(T x, T y) {
    T s = x + y, v = s - x;
    return dw(s, (x - (s - v)) + (y - v));
}
template <typename T> __device__ __forceinline__ DW<T> dw_add2(DW<T> x, T y) {
    T s = x.x + y, v = s - x.x;
    T t = (x.x - (s - v)) + (y - v);
    return dw(s, t + x.y);
}
template <typename T> __device__ __forceinline__ DW<T> dw_add(T x, DW<T> y) {
    T s = x + y.x;
    return dw(s, ((x - s) + y.x) + y.y);
}
template <typename T> __device__ __forceinline__ DW<T> dw_add(DW<T> x, DW<T> y) {
    T s = x.x + y.x;
    return dw(s, (((x.x - s) + y.x) + x.y) + y.y);
}
template <typename T> __device__ __forceinline__ DW<T> dw_add2(DW<T> x, DW<T> y) {
    T s = x.x + y.x, v = s - x.x;
    T t = (x.x - (s - v)) + (y.x - v);
    return dw(s, t + (x.y + y.y));
}
template <typename T> __device__ __forceinline__ DW<T> dw_scale(DW<T> d, T s) { return dw(d.x * s, d.y * s); }
template <typename T> __device__ __forceinline__ DW<T> dw_normalize(DW<T> t) {
    T s = t.x + t.y;
    return dw(s, (t.x - s) + t.y);
}
template <typename T> __device__ __forceinline__ DW<T> dw_div(DW<T> n, DW<T> d) {
    T t = (T)1 / d.x;
    T s = n.x * t;
    T u = fmapn(t, n.x, s);
    T v = fmanp(d.y, t, fmanp(d.x, t, (T)1));
    return dw(s, fma_(s, v, fma_(n.y, t, u)));
}
template <typename T> __device__ __forceinline__ DW<T> dw_squ(DW<T> x) {
    T s = x.x * x.x;
    return dw(s, fma_(x.x + x.x, x.y, fmapn(x.x, x.x, s)));
}
template <typename T> __device__ __forceinline__ DW<T> dw_mul(DW<T> x, T y) {
    T s = x.x * y;
    return dw(s, fma_(x.y, y, fmapn(x.x, y, s)));
}
template <typename T> __device__ __forceinline__ DW<T> dw_mul(DW<T> x, DW<T> y) {
    T s = x.x * y.x;
    return dw(s, fma_(x.x, y.y, fma_(x.y, y.x, fmapn(x.x, y.x, s))));
}

// ---- float ----
__device__ __forceinline__ float pow2i(float, int q) { return __int_as_float((q + 0x7f) << 23); }
__device__ __forceinline__ double pow2i(double, int q) { return __longlong_as_double((long long)(q + 0x3ff) << 52); }
template <typename T> __device__ __forceinline__ T ldexp2k(T d, int e) { return d * pow2i(T(0), e >> 1) * pow2i(T(0), e - (e >> 1)); }

// log of a positive finite d as a double-word
__device__ __forceinline__ DW<float> logk(float d) {
    const bool o = d < 1.17549435e-38f;
    d = o ? d * 18446744073709551616.0f : d;  // 2^64
    const float d43 = d * (1.0f / 0.75f);
    int e = ((__float_as_int(d43) >> 23) & 0xff) - 0x7f;
    const float m = __int_as_float(__float_as_int(d) - (e << 23));  // d * 2^-e
    e = o ? e - 64 : e;
    DW<float> x = dw_div(dw_add2(-1.0f, m), dw_add2(1.0f, m));
    DW<float> x2 = dw_squ(x);
    float t = 0.240320354700088500976562f;
    t = fma_(t, x2.x, 0.285112679004669189453125f);
    t = fma_(t, x2.x, 0.400007992982864379882812f);
    const DW<float> c = dw(0.66666662693023681640625f, 3.69183861259614332084311e-09f);
    DW<float> s = dw_mul(dw(0.69314718246459960938f, -1.904654323148236017e-09f), (float)e);
    s = dw_add(s, dw_scale(x, 2.0f));
    s = dw_add(s, dw_mul(dw_mul(x2, x), dw_add2(dw_mul(x2, t), c)));
    return s;
}

// exp of a double-word
__device__ __forceinline__ float expk(DW<float> d) {
    float u = (d.x + d.y) * 1.442695040888963407359924681001892137426645954152985934135449406931f;
    const float fq = __builtin_rintf(u);
    const int q = (int)fq;
    DW<float> s = dw_add2(d, fq * -0.693145751953125f);
    s = dw_add2(s, fq * -1.428606765330187045e-06f);
    s = dw_normalize(s);
    u = 0.00136324646882712841033936f;
    u = fma_(u, s.x, 0.00836596917361021041870117f);
    u = fma_(u, s.x, 0.0416710823774337768554688f);
    u = fma_(u, s.x, 0.166665524244308471679688f);
    u = fma_(u, s.x, 0.499999850988388061523438f);
    DW<float> t = dw_add(s, dw_mul(dw_squ(s), u));
    t = dw_add(1.0f, t);
    u = t.x + t.y;
    u = ldexp2k(u, q);
    return d.x < -104.0f ? 0.0f : u;
}

// ---- double ----
__device__ __forceinline__ DW<double> logk(double d) {
    const bool o = d < 2.2250738585072014e-308;
    d = o ? d * 18446744073709551616.0 : d;
    const double d43 = d * (1.0 / 0.75);
    int e = (int)((__double2hiint(d43) >> 20) & 0x7ff) - 0x3ff;
    const double m = __hiloint2double(__double2hiint(d) - (e << 20), __double2loint(d));
    e = o ? e - 64 : e;
    DW<double> x = dw_div(dw_add2(-1.0, m), dw_add2(1.0, m));
    DW<double> x2 = dw_squ(x);
    const double z = x2.x, z2 = z * z, z4 = z2 * z2, z8 = z4 * z4;
    const double p01 = fma_(z, 0.285714285714249172087875, 0.400000000000000077715612);
    const double p23 = fma_(z, 0.181818180850050775676507, 0.222222222230083560345903);
    const double p45 = fma_(z, 0.13332981086846273921509, 0.153846227114512262845736);
    const double p67 = fma_(z, 0.103239680901072952701192, 0.117754809412463995466069);
    const double lo = fma_(z2, p23, p01), hi = fma_(z2, p67, p45);
    const double t = fma_(z8, 0.116255524079935043668677, fma_(z4, hi, lo));
    const DW<double> c = dw(0.666666666666666629659233, 3.80554962542412056336616e-17);
    DW<double> s = dw_mul(dw(0.693147180559945286226764, 2.319046813846299558417771e-17), (double)e);
    s = dw_add(s, dw_scale(x, 2.0));
    x = dw_mul(x2, x);
    s = dw_add(s, dw_mul(x, c));
    x = dw_mul(x2, x);
    s = dw_add(s, dw_mul(x, t));
    return s;
}

__device__ __forceinline__ double expk(DW<double> d) {
    double u = (d.x + d.y) * 1.442695040888963407359924681001892137426645954152985934135449406931;
    const double dq = __builtin_rint(u);
    const int q = (int)dq;
    DW<double> s = dw_add2(d, dq * -.69314718055966295651160180568695068359375);
    s = dw_add2(s, dq * -.28235290563031577122588448175013436025525412068e-12);
    s = dw_normalize(s);
    const double z = s.x, z2 = z * z, z4 = z2 * z2, z8 = z4 * z4;
    const double p01 = fma_(z, 0.166666666666666740681535, 0.500000000000000999200722);
    const double p23 = fma_(z, 0.00833333333332371417601081, 0.0416666666665409524128449);
    const double p45 = fma_(z, 0.000198412698809069797676111, 0.0013888888939977128960529);
    const double p67 = fma_(z, 2.75572496725023574143864e-06, 2.48014973989819794114153e-05);
    const double p89 = fma_(z, 2.51069683420950419527139e-08, 2.76286166770270649116855e-07);
    const double lo = fma_(z2, p23, p01), hi = fma_(z2, p67, p45);
    u = fma_(z8, p89, fma_(z4, hi, lo));
    DW<double> t = dw_add(1.0, s);
    t = dw_add(t, dw_mul(dw_squ(s), u));
    u = t.x + t.y;
    u = ldexp2k(u, q);
    return d.x < -1000.0 ? 0.0 : u;
}

// exp(lg * y) with the library's "NaN result means overflow" rule; lg = logk(x) of a
// positive finite x.  pow_(x, y) == powk(logk(x), y) on that domain.
template <typename T> __device__ __forceinline__ T powk(DW<T> lg, T y) {
    T r = expk(dw_mul(lg, y));
    return (r != r) ? (T)__builtin_huge_val() : r;
}

// The step factor's powers (step_size_controllers.py:289-294, 598-620) for the kernels that keep
// the history of accepted error ratios as logarithms: safety * ratio^e1 [* prev^e2 [* prev_prev^e3]],
// multiplied in this order.  `ratio` is positive and finite.  NHIST = number of history factors.
template <typename T, int NHIST> struct StepFactor {
    DW<T> lg, lg_prev, lg_pprev;
    __device__ __forceinline__ StepFactor() : lg(dw((T)0, (T)0)), lg_prev(dw((T)0, (T)0)), lg_pprev(dw((T)0, (T)0)) {}
    __device__ __forceinline__ T operator()(T safety, T ratio, T e1, T e2, T e3, bool) {
        lg = logk(ratio);
        T factor = safety * powk<T>(lg, e1);
        if (NHIST >= 1) factor = factor * powk<T>(lg_prev, e2);
        if (NHIST >= 2) factor = factor * powk<T>(lg_pprev, e3);
        return factor;
    }
    // the ratio just used becomes the previous one where `shift` (an accepted step of a running sample)
    __device__ __forceinline__ void shift(bool s) {
        if (NHIST >= 2) {
            lg_pprev.x = s ? lg_prev.x : lg_pprev.x;
            lg_pprev.y = s ? lg_prev.y : lg_pprev.y;
        }
        if (NHIST >= 1) {
            lg_prev.x = s ? lg.x : lg_prev.x;
            lg_prev.y = s ? lg.y : lg_prev.y;
        }
    }
};

// x ** y for x >= 0 or NaN, all special cases included.
template <typename T> __device__ __forceinline__ T pow_(T x, T y) {
    if (y == (T)0 || x == (T)1) return (T)1;
    if (x != x || y != y) return nan_<T>();
    if (x < (T)0) return nan_<T>();
    const T inf = (T)__builtin_huge_val();
    if (x == inf || x == (T)0) return (((x == (T)0) ? -y : y) < (T)0) ? (T)0 : inf;
    if (abs_(y) == inf) {
        T efx = (y < (T)0 ? (T)-1 : (T)1) * (x - (T)1);
        return efx < (T)0 ? (T)0 : (efx == (T)0 ? (T)1 : inf);
    }
    return powk<T>(logk(x), y);
}

// Tensor ** python_float as ATen's CPU kernels compute it: exponents 0 and 1 are a fill and a
// copy (aten/src/ATen/native/Pow.cpp); 0.5, -0.5 and -1 go to the square root, reciprocal square
// root and reciprocal kernels and 2, 3 and -2 are multiplications
// (aten/src/ATen/native/cpu/PowKernel.cpp); every other exponent is rounded to the tensor dtype
// and goes through pow.  The first group compares the exponent as the double it is, the second
// after rounding to the tensor dtype.  The square roots are the correctly rounded ones; an ATen
// build that takes them from a vector math library can differ from that in the last bit
// (exponents 0.5 and -0.5 only).
template <typename T> __host__ __device__ __forceinline__ bool special_exponent(double p) {
    const T e = (T)p;
    return p == 0.0 || p == 1.0 || p == 0.5 || p == -0.5 || p == -1.0 || e == (T)2 || e == (T)3 || e == (T)-2;
}
template <typename T> __device__ __forceinline__ T rpow(T x, double p) {
    if (p == 0.0) return (T)1;
    if (p == 1.0) return x;
    if (p == 0.5) return sqrt_(x);
    if (p == -0.5) return (T)1 / sqrt_(x);
    if (p == -1.0) return (T)1 / x;
    const T e = (T)p;
    if (e == (T)2) return x * x;
    if (e == (T)3) return (x * x) * x;
    if (e == (T)-2) return (T)1 / (x * x);
    return pow_<T>(x, e);
}

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
        {2.9132554618219126, -0.2234, -5.941033872131505, 30.338188630282318, -88.1789048947664, 65.09189467479368,
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
    // an exponent that ATen does not compute through pow (kernels that share one logarithm
    // between the powers do not take such a controller)
    bool shortcut_exponent() const {
        return special_exponent<T>(e1) && e1 != 0.0 || !skip2 && special_exponent<T>(e2) || !skip3 && special_exponent<T>(e3);
    }
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
// With MAGNITUDE_ONLY the first product is taken as it is instead of being added to zero: the
// two differ in the sign of a zero sum at most, which a caller that only uses |out| never sees.
template <typename T, int F, typename Tab, int ROW, bool MAGNITUDE_ONLY = false>
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
            out[f] = (MAGNITUDE_ONLY && s == 0) ? pk : out[f] + pk;
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

// x / sqrt(F) as the reference divides (a true division by the rounded square root), in fewer
// instructions where that is provably the same value: fast() for arguments of at least 2^-100 (or
// zero), exact() for any.  F == 1 and F == 4 are exact scalings.  For
// float32 and F == 2, 3 the quotient by the constant c = float(sqrt(F)) is q = x * (1/c) corrected
// once through the exact remainder: fma(fma(-q, c, x), 1/c, q).  That equals the correctly rounded
// x / c for every float32 mantissa (verified exhaustively for both constants), provided the
// remainder is exact, i.e. nothing underflows: arguments below 2^-100 take the division.
template <typename T, int F> struct DivSqrtFeatures {
    static constexpr bool corrected = false;
    static __device__ __forceinline__ T fast(T x) {
        if (F == 1) return x;
        if (F == 4) return x * (T)0.5;
        return x / (T)__builtin_sqrt((double)F);
    }
    static __device__ __forceinline__ T exact(T x) { return fast(x); }
};
template <int F> struct DivSqrtConstant {};
template <> struct DivSqrtConstant<2> { static constexpr float c = 1.41421354f, rc = 0x1.6a09e6p-1f; };
template <> struct DivSqrtConstant<3> { static constexpr float c = 1.73205078f, rc = 0x1.279a74p-1f; };
template <int F> struct DivSqrtCorrected {
    static constexpr bool corrected = true;
    static __device__ __forceinline__ float fast(float x) {
        const float q = x * DivSqrtConstant<F>::rc;
        return fma_(fma_(-q, DivSqrtConstant<F>::c, x), DivSqrtConstant<F>::rc, q);
    }
    static __device__ __forceinline__ float exact(float x) { return x / DivSqrtConstant<F>::c; }
};
template <> struct DivSqrtFeatures<float, 2> : DivSqrtCorrected<2> {};
template <> struct DivSqrtFeatures<float, 3> : DivSqrtCorrected<3> {};

// Error ratio for the kernels that cover the common case only (and hand every batch with a
// non-finite value to the general kernel): the same operations as error_ratio() with the
// hardware's maximum in place of the NaN-propagating one.  The two differ for a NaN operand alone;
// `unordered` is raised for one (a NaN in y0, y1, err or the sum), and the caller must then leave
// the common case rather than use the returned value.  An infinite operand takes the same path
// through both.
template <typename T, int F>
__device__ __forceinline__ T error_ratio_common(const CtrlParams<T> &cp, const T (&y0)[F], const T (&y1)[F], const T (&err)[F],
                                                bool &unordered) {
    using Div = DivSqrtFeatures<T, F>;
    T q[F], x[F];
    bool nan = false, small = false;
#pragma unroll
    for (int f = 0; f < F; ++f) {
        nan = nan || __builtin_isunordered(y0[f], y1[f]);
        const T m = hwmax(abs_(y0[f]), abs_(y1[f]));
        const T eb = fma_(cp.rtol, m, cp.atol);
        q[f] = abs_(err[f]) / eb;
        x[f] = Div::fast(q[f]);
        if (Div::corrected) small = small || (q[f] < (T)0x1p-100f && q[f] > (T)0);
    }
    if (Div::corrected && __builtin_expect(__any(small), 0)) {  // (one branch for all features, after their divisions)
#pragma unroll
        for (int f = 0; f < F; ++f) x[f] = Div::exact(q[f]);
    }
    T acc = 0;
#pragma unroll
    for (int f = 0; f < F; ++f) {
        if (F <= 3)
            acc = fma_(x[f], x[f], acc);
        else {
            const T sq = x[f] * x[f];
            acc = acc + sq;
        }
    }
    const T r = sqrt_(acc);
    unordered = nan || r != r;
    return hwmax(r, (T)1e-38);
}

// clamp(x, lo, hi) for operands that are known not to be NaN.
template <typename T> __device__ __forceinline__ T clamp_ordered(T x, T lo, T hi) { return hwmin(hwmax(x, lo), hi); }

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

// dt_min / dt_max and the status of a step proposal, limits in the time type
// (step_size_controllers.py:406-422, 751-767).
template <typename TT, typename T>
__device__ __forceinline__ int limit_step(const CtrlParams<T> &cp, TT dt_min, TT dt_max, T ratio, TT &dt_next) {
    int status = finite_(ratio) ? 0 : 4;
    if (cp.has_dt_min || cp.has_dt_max) {
        const TT mag = abs_(dt_next);
        TT c = mag;
        if (cp.has_dt_min) c = tmax(c, dt_min);
        if (cp.has_dt_max) c = tmin(c, dt_max);
        const TT sg = (dt_next > 0) ? (TT)1 : ((dt_next < 0) ? (TT)-1 : dt_next);
        dt_next = sg * c;
        if (cp.has_dt_min && mag < dt_min) status = 2;
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
template <typename T, int F, typename TT = T> __device__ __forceinline__ void quartic_eval(const T (&q)[5][F], TT t0, TT dt, TT t, T (&out)[F]) {
    TT t1 = t0 + dt;
    TT den = t1 - t0;
    if (!(abs_(den) > (TT)0)) den = (TT)1;
    T x = (T)((t - t0) / den);  // (formed in the time type, then taken to the data type: interpolation.py:8-40)
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

// Quartic coefficients for a single feature with run-time choice of ATen's two
// summation forms: products rounded and then added (F <= 57), or one fused chain
// (F >= 58, where the contraction runs as a matrix product).  ks[s] = k_s[b,f].
template <typename T, int METHOD>
__device__ __forceinline__ void quartic_elem(T dt, T y0, T y1, const T (&ks)[7], bool fused, T (&q)[5][1]) {
    if (!fused) {
        T yy0[1] = {y0}, yy1[1] = {y1}, kk[7][1];
#pragma unroll
        for (int s = 0; s < 7; ++s) kk[s][0] = ks[s];
        quartic<T, 1, METHOD>(dt, yy0, yy1, kk, q);
        return;
    }
    using Tab = typename std::conditional<METHOD == 1, Tsit5Tab, Dopri5Tab>::type;
    T w[3] = {0, 0, 0};
#pragma unroll
    for (int r = 0; r < Tab::n_other; ++r)
#pragma unroll
        for (int s = 0; s < 7; ++s) w[r] = fma_(dt * (T)Tab::w[r][s], ks[s], w[r]);
    if (METHOD == 1) {
        q[0][0] = y0;
        q[1][0] = dt * ks[0];
        q[2][0] = w[0];
        q[3][0] = w[1];
        q[4][0] = w[2];
    } else {
        T f0 = dt * ks[0], f1 = dt * ks[6];
        T ym = y0 + w[0];
        T a = (T)2 * (f1 - f0);
        a = fma_((T)-8, y1 + y0, a);
        a = fma_((T)16, ym, a);
        T bq = (T)5 * f0;
        bq = fma_((T)-3, f1, bq);
        bq = fma_((T)18, y0, bq);
        bq = fma_((T)14, y1, bq);
        bq = fma_((T)-32, ym, bq);
        T c = fma_((T)-4, f0, f1);
        c = fma_((T)-11, y0, c);
        c = fma_((T)-5, y1, c);
        c = fma_((T)16, ym, c);
        q[0][0] = y0;
        q[1][0] = f0;
        q[2][0] = c;
        q[3][0] = bq;
        q[4][0] = a;
    }
}

}  // namespace tode
