// Protocol operators: one kernel per protocol method of the reference's plug-in
// interfaces (SingleStepMethod.step, StepSizeController.init / adapt_step_size /
// merge_states, LocalInterpolation.evaluate) plus the bookkeeping of one loop
// iteration.  The package's Python classes call these, so that library parts and
// user-supplied parts can be mixed freely in one solve.
//
// Time (t, dt, evaluation times) and data (y, derivatives, error ratios) may have different
// floating point types, TT and T below; every formula converts where the reference does
// (dt to the data type for the stage sums, the step factor to the time type for the new step).
//
// Elementwise kernels use one thread per value of [B,F].  Per-sample kernels use
// one thread per sample and walk the row in order when F < 64 (the summation
// order of a scalar evaluation), and one wavefront per sample when F >= 64.
#include <limits.h>

#include "tode_solve.h"

namespace tode {

struct Coeffs {
    double v[TODE_MAX_STAGES];
};

// ------------------------------------------------------------------------------------------
// explicit Runge-Kutta step
// ------------------------------------------------------------------------------------------

// y_out = fma(dt, sum_j a_j k_j, y0), t_out = fma(c, dt, t0)   (runge_kutta.py:258-262)
template <typename TT, typename T>
__global__ void __launch_bounds__(256) erk_stage_kernel(long long batch, int F, int n, Coeffs a, double c, const TT *t0, const TT *dt,
                                                        const T *y0, const T *k, T *y_out, TT *t_out) {
    const long long i = (long long)blockIdx.x * 256 + threadIdx.x;
    const long long bf = batch * F;
    if (i >= bf) return;
    const long long b = i / F;
    const T h = (T)dt[b];
    T s = 0;
    for (int j = 0; j < n; ++j) s = fma_((T)a.v[j], k[j * bf + i], s);
    y_out[i] = fma_(h, s, y0[i]);
    if (t_out && i - b * F == 0) t_out[b] = fma_((TT)c, dt[b], t0[b]);
}

// out = sum_s (dt * w_s) * k_s (+ y0)   (runge_kutta.py:264-267).  ATen rounds the products
// before adding them for F <= 57 and runs one fused chain for F >= 58.
template <typename TT, typename T>
__global__ void __launch_bounds__(256) erk_combine_kernel(long long batch, int F, int S, Coeffs w, const TT *dt, const T *k, const T *y0, T *out) {
    const long long i = (long long)blockIdx.x * 256 + threadIdx.x;
    const long long bf = batch * F;
    if (i >= bf) return;
    const T h = (T)dt[i / F];
    const bool fused = F >= 58;
    T acc = 0;
    for (int s = 0; s < S; ++s) {
        const T ps = h * (T)w.v[s];
        const T ks = k[s * bf + i];
        if (fused)
            acc = fma_(ps, ks, acc);
        else {
            const T pk = ps * ks;
            acc = acc + pk;
        }
    }
    out[i] = y0 ? y0[i] + acc : acc;
}

// ------------------------------------------------------------------------------------------
// step size control
// ------------------------------------------------------------------------------------------

template <typename T> __device__ __forceinline__ T scaled_error(T atol, T rtol, T y0, T y1, T err) {
    const T m = tmax(abs_(y0), abs_(y1));
    return abs_(err) / fma_(rtol, m, atol);
}

template <typename T>
__global__ void __launch_bounds__(256) error_scale_kernel(long long n, T atol, T rtol, const T *y0, const T *y1, const T *err, T *out) {
    const long long i = (long long)blockIdx.x * 256 + threadIdx.x;
    if (i < n) out[i] = scaled_error(atol, rtol, y0[i], y1[i], err[i]);
}

// Running norm of a row, fed one value at a time in row order.
template <typename T, int NORM> struct RowNorm {
    T acc = 0, sf;
    int F;
    __device__ __forceinline__ RowNorm(int F_) : sf((T)__builtin_sqrt((double)F_)), F(F_) {}
    __device__ __forceinline__ void add(T v) {
        if (NORM == TODE_NORM_MAX) {
            acc = tmax(acc, abs_(v));
        } else {
            const T x = v / sf;
            if (F <= 3)
                acc = fma_(x, x, acc);
            else {
                const T sq = x * x;
                acc = acc + sq;
            }
        }
    }
    __device__ __forceinline__ T get() const { return NORM == TODE_NORM_MAX ? acc : sqrt_(acc); }
};

template <typename T, int NORM> __global__ void __launch_bounds__(256) row_norm_thread_kernel(long long batch, int F, const T *x, T *out) {
    const long long b = (long long)blockIdx.x * 256 + threadIdx.x;
    if (b >= batch) return;
    RowNorm<T, NORM> r(F);
    for (int f = 0; f < F; ++f) r.add(x[b * F + f]);
    out[b] = r.get();
}

template <typename T, int NORM> __global__ void __launch_bounds__(256) row_norm_wave_kernel(long long batch, int F, const T *x, T *out) {
    const long long b = (long long)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (b >= batch) return;
    const T *row = x + b * F;
    const T r = wave_row_norm<T, NORM>(F, [&](int f) { return row[f]; });
    if ((threadIdx.x & 63) == 0) out[b] = r;
}

struct ControlOut {
    uint8_t *accept;
    void *dt_next, *ratio, *prev_out, *pprev_out;
    int64_t *status;
};

// ratio -> accept, dt_next, status, PID history (step_size_controllers.py:394-429, 640-671, 739-774).
// The factor is formed in the data type and converted; the new step and its limits live in the time type.
template <typename TT> struct StepLimits {
    TT dt_min, dt_max;
};

template <typename TT, typename T, int CTRL>
__device__ __forceinline__ void control_one(const CtrlParams<T> &cp, const StepLimits<TT> &lim, long long b, T norm, TT dt, const T *prev, const T *pprev,
                                            const ControlOut &o) {
    const T ratio = tmax(norm, (T)1e-38);
    const bool accept = ratio < (T)1;
    const T p1 = CTRL == 1 ? prev[b] : (T)1, p2 = CTRL == 1 ? pprev[b] : (T)1;
    const T factor = dt_factor<T, CTRL>(cp, ratio, p1, p2);
    TT dt_next = dt * (TT)factor;
    int status = finite_(ratio) ? 0 : 4;
    if (cp.has_dt_min || cp.has_dt_max) {
        const TT mag = abs_(dt_next);
        TT c = mag;
        if (cp.has_dt_min) c = tmax(c, lim.dt_min);
        if (cp.has_dt_max) c = tmin(c, lim.dt_max);
        const TT sg = (dt_next > 0) ? (TT)1 : ((dt_next < 0) ? (TT)-1 : dt_next);
        dt_next = sg * c;
        if (cp.has_dt_min && mag < lim.dt_min) status = 2;
    }
    o.accept[b] = accept ? 1 : 0;
    ((TT *)o.dt_next)[b] = dt_next;
    if (o.ratio) ((T *)o.ratio)[b] = ratio;
    o.status[b] = status;
    if (CTRL == 1) {
        ((T *)o.prev_out)[b] = accept ? ratio : p1;
        ((T *)o.pprev_out)[b] = accept ? p1 : p2;
    }
}

template <typename TT, typename T, int CTRL>
__global__ void __launch_bounds__(256) control_kernel(CtrlParams<T> cp, StepLimits<TT> lim, long long batch, const T *norm, const TT *dt, const T *prev,
                                                      const T *pprev, ControlOut o) {
    const long long b = (long long)blockIdx.x * 256 + threadIdx.x;
    if (b < batch) control_one<TT, T, CTRL>(cp, lim, b, norm[b], dt[b], prev, pprev, o);
}

template <typename TT, typename T, int CTRL, int NORM>
__global__ void __launch_bounds__(256) adapt_thread_kernel(CtrlParams<T> cp, StepLimits<TT> lim, long long batch, int F, const TT *dt, const T *y0,
                                                           const T *y1, const T *err, const T *prev, const T *pprev, ControlOut o) {
    const long long b = (long long)blockIdx.x * 256 + threadIdx.x;
    if (b >= batch) return;
    RowNorm<T, NORM> r(F);
    for (int f = 0; f < F; ++f) r.add(scaled_error(cp.atol, cp.rtol, y0[b * F + f], y1[b * F + f], err[b * F + f]));
    control_one<TT, T, CTRL>(cp, lim, b, r.get(), dt[b], prev, pprev, o);
}

template <typename TT, typename T, int CTRL, int NORM>
__global__ void __launch_bounds__(256) adapt_wave_kernel(CtrlParams<T> cp, StepLimits<TT> lim, long long batch, int F, const TT *dt, const T *y0,
                                                         const T *y1, const T *err, const T *prev, const T *pprev, ControlOut o) {
    const long long b = (long long)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (b >= batch) return;
    const T *r0 = y0 + b * F, *r1 = y1 + b * F, *re = err + b * F;
    const T norm = wave_row_norm<T, NORM>(F, [&](int f) { return scaled_error(cp.atol, cp.rtol, r0[f], r1[f], re[f]); });
    if ((threadIdx.x & 63) == 0) control_one<TT, T, CTRL>(cp, lim, b, norm, dt[b], prev, pprev, o);
}

// ------------------------------------------------------------------------------------------
// start step (step_size_controllers.py:431-490, 776-835)
// ------------------------------------------------------------------------------------------

template <typename TT, typename T, int NORM>
__global__ void __launch_bounds__(256) initial_a_thread_kernel(long long batch, int F, T atol, T rtol, const TT *t_start, const TT *t_end, const T *y0,
                                                               const T *f0, T *h0_out) {
    const long long b = (long long)blockIdx.x * 256 + threadIdx.x;
    if (b >= batch) return;
    RowNorm<T, NORM> n0(F), n1(F);
    for (int f = 0; f < F; ++f) {
        const T inv = inv_scale(atol, rtol, y0[b * F + f]);
        n0.add(y0[b * F + f] * inv);
        n1.add(f0[b * F + f] * inv);
    }
    const T d0 = n0.get(), d1 = n1.get();
    T h0 = (d0 < (T)1e-5 || d1 < (T)1e-5) ? (T)1e-6 : ((T)0.01 * d0) / d1;
    h0_out[b] = tmin(h0, (T)abs_(t_end[b] - t_start[b]));
}

template <typename TT, typename T, int NORM>
__global__ void __launch_bounds__(256) initial_a_wave_kernel(long long batch, int F, T atol, T rtol, const TT *t_start, const TT *t_end, const T *y0,
                                                             const T *f0, T *h0_out) {
    const long long b = (long long)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (b >= batch) return;
    const T *ry = y0 + b * F, *rf = f0 + b * F;
    const T d0 = wave_row_norm<T, NORM>(F, [&](int f) { return ry[f] * inv_scale(atol, rtol, ry[f]); });
    const T d1 = wave_row_norm<T, NORM>(F, [&](int f) { return rf[f] * inv_scale(atol, rtol, ry[f]); });
    if ((threadIdx.x & 63) == 0) {
        T h0 = (d0 < (T)1e-5 || d1 < (T)1e-5) ? (T)1e-6 : ((T)0.01 * d0) / d1;
        h0_out[b] = tmin(h0, (T)abs_(t_end[b] - t_start[b]));
    }
}

// The same two halves with the norms supplied by the caller (a user-defined norm): scaling for the
// norm's argument, h0 from (d0, d1), the final step from (d1, d2n).
template <typename T>
__global__ void __launch_bounds__(256) tolerance_scale_kernel(long long n, T atol, T rtol, const T *y_ref, const T *v, T *out) {
    const long long i = (long long)blockIdx.x * 256 + threadIdx.x;
    if (i < n) out[i] = v[i] * inv_scale(atol, rtol, y_ref[i]);
}

template <typename TT, typename T>
__global__ void __launch_bounds__(256) initial_h0_kernel(long long batch, const TT *t_start, const TT *t_end, const T *d0, const T *d1, T *h0_out) {
    const long long b = (long long)blockIdx.x * 256 + threadIdx.x;
    if (b >= batch) return;
    T h0 = (d0[b] < (T)1e-5 || d1[b] < (T)1e-5) ? (T)1e-6 : ((T)0.01 * d0[b]) / d1[b];
    h0_out[b] = tmin(h0, (T)abs_(t_end[b] - t_start[b]));
}

template <typename TT, typename T>
__global__ void __launch_bounds__(256) initial_dt_kernel(int kind, double inv_order, long long batch, const TT *t_start, const TT *t_end, const T *h0,
                                                         const T *d1, const T *d2n, TT *dt0) {
    const long long b = (long long)blockIdx.x * 256 + threadIdx.x;
    if (b >= batch) return;
    const T dir = (t_end[b] > t_start[b]) ? (T)1 : (T)-1;
    dt0[b] = (TT)initial_finish<T>(kind, inv_order, dir, h0[b], d1[b], d2n[b]);
}

// y1 = y0 + (direction * h0) * f0, t1 = t_start + direction * h0   (:474-479)
template <typename TT, typename T>
__global__ void __launch_bounds__(256) initial_probe_kernel(long long batch, int F, const TT *t_start, const TT *t_end, const T *y0, const T *f0,
                                                            const T *h0, T *y1, TT *t1) {
    const long long i = (long long)blockIdx.x * 256 + threadIdx.x;
    if (i >= batch * F) return;
    const long long b = i / F;
    const bool fwd = t_end[b] > t_start[b];
    const T h = h0[b];
    y1[i] = fma_((fwd ? (T)1 : (T)-1) * h, f0[i], y0[i]);
    if (i - b * F == 0) t1[b] = fma_(fwd ? (TT)1 : (TT)-1, (TT)h, t_start[b]);
}

template <typename TT, typename T, int NORM>
__global__ void __launch_bounds__(256) initial_b_thread_kernel(int kind, double inv_order, long long batch, int F, T atol, T rtol, const TT *t_start,
                                                               const TT *t_end, const T *y0, const T *f0, const T *f1, const T *h0, TT *dt0) {
    const long long b = (long long)blockIdx.x * 256 + threadIdx.x;
    if (b >= batch) return;
    RowNorm<T, NORM> n1(F), n2(F);
    for (int f = 0; f < F; ++f) {
        const T inv = inv_scale(atol, rtol, y0[b * F + f]);
        n1.add(f0[b * F + f] * inv);
        const T df = f1[b * F + f] - f0[b * F + f];
        n2.add(df * inv);
    }
    const T dir = (t_end[b] > t_start[b]) ? (T)1 : (T)-1;
    dt0[b] = (TT)initial_finish<T>(kind, inv_order, dir, h0[b], n1.get(), n2.get());
}

template <typename TT, typename T, int NORM>
__global__ void __launch_bounds__(256) initial_b_wave_kernel(int kind, double inv_order, long long batch, int F, T atol, T rtol, const TT *t_start,
                                                             const TT *t_end, const T *y0, const T *f0, const T *f1, const T *h0, TT *dt0) {
    const long long b = (long long)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (b >= batch) return;
    const T *ry = y0 + b * F, *r0 = f0 + b * F, *r1 = f1 + b * F;
    const T d1 = wave_row_norm<T, NORM>(F, [&](int f) { return r0[f] * inv_scale(atol, rtol, ry[f]); });
    const T d2n = wave_row_norm<T, NORM>(F, [&](int f) {
        const T df = r1[f] - r0[f];
        return df * inv_scale(atol, rtol, ry[f]);
    });
    if ((threadIdx.x & 63) == 0) {
        const T dir = (t_end[b] > t_start[b]) ? (T)1 : (T)-1;
        dt0[b] = (TT)initial_finish<T>(kind, inv_order, dir, h0[b], d1, d2n);
    }
}

// ------------------------------------------------------------------------------------------
// dense output
// ------------------------------------------------------------------------------------------

template <typename TT, typename T, int METHOD>
__global__ void __launch_bounds__(256) quartic_build_kernel(long long batch, int F, const TT *dt, const T *y0, const T *y1, const T *k, T *coeff) {
    const long long i = (long long)blockIdx.x * 256 + threadIdx.x;
    const long long bf = batch * F;
    if (i >= bf) return;
    T ks[7];
#pragma unroll
    for (int s = 0; s < 7; ++s) ks[s] = k[s * bf + i];
    T q[5][1];
    quartic_elem<T, METHOD>((T)dt[i / F], y0[i], y1[i], ks, F >= 58, q);
#pragma unroll
    for (int p = 0; p < 5; ++p) coeff[p * bf + i] = q[p][0];
}

// Quartic through y0, y1, the end-point slopes and a mid-point value (interpolation.py:138-170).
template <typename TT, typename T>
__global__ void __launch_bounds__(256) quartic_from_mid_kernel(long long batch, int F, const TT *dt, const T *y0, const T *y1, const T *k_first,
                                                               const T *k_last, const T *y_mid, T *coeff) {
    const long long i = (long long)blockIdx.x * 256 + threadIdx.x;
    const long long bf = batch * F;
    if (i >= bf) return;
    const T h = (T)dt[i / F];
    const T f0 = h * k_first[i], f1 = h * k_last[i], ym = y_mid[i], a0 = y0[i], a1 = y1[i];
    T a = (T)2 * (f1 - f0);
    a = fma_((T)-8, a1 + a0, a);
    a = fma_((T)16, ym, a);
    T b = (T)5 * f0;
    b = fma_((T)-3, f1, b);
    b = fma_((T)18, a0, b);
    b = fma_((T)14, a1, b);
    b = fma_((T)-32, ym, b);
    T c = fma_((T)-4, f0, f1);
    c = fma_((T)-11, a0, c);
    c = fma_((T)-5, a1, c);
    c = fma_((T)16, ym, c);
    coeff[i] = a0;
    coeff[bf + i] = f0;
    coeff[2 * bf + i] = c;
    coeff[3 * bf + i] = b;
    coeff[4 * bf + i] = a;
}

// Hermite cubic through y0, y1 and the end-point slopes (interpolation.py:84-106).
template <typename TT, typename T>
__global__ void __launch_bounds__(256) cubic_build_kernel(long long batch, int F, const TT *dt, const T *y0, const T *y1, const T *k_first,
                                                          const T *k_last, T *coeff) {
    const long long i = (long long)blockIdx.x * 256 + threadIdx.x;
    const long long bf = batch * F;
    if (i >= bf) return;
    const T h = (T)dt[i / F];
    const T f0 = k_first[i], f1 = k_last[i];
    const T d01 = y0[i] - y1[i];
    const T a = fma_((T)2, d01, h * (f0 + f1));            // add(dt*(f0+f1), y0-y1, alpha=2)
    const T b = fma_((T)-3, d01, h * fma_((T)-2, f0, -f1));  // add(dt*add(-f1, f0, alpha=-2), y0-y1, alpha=-3)
    coeff[i] = y0[i];
    coeff[bf + i] = h * f0;
    coeff[2 * bf + i] = b;
    coeff[3 * bf + i] = a;
}

template <typename TT, typename T>
__global__ void __launch_bounds__(256) poly_eval_kernel(int degree, int span_is_dt, long long batch, int F, long long count, const T *coeff, const TT *t0, const TT *t1,
                                                        const TT *t, const int64_t *idx, T *out) {
    const long long i = (long long)blockIdx.x * 256 + threadIdx.x;
    if (i >= count * F) return;
    const long long n = i / F;
    const int f = (int)(i - n * F);
    const long long b = idx[n];
    if (b < 0 || b >= batch) return;
    out[i] = horner(coeff, batch * F, b * F + f, degree, (T)unit_time_over(t[n], t0[b], span_is_dt ? t1[b] : t1[b] - t0[b]));
}

// small F: one thread per sample walks its mask row
template <typename TT, typename T>
__global__ void __launch_bounds__(256) poly_eval_masked_thread_kernel(int degree, int span_is_dt, long long batch, int F, int E, const T *coeff, const TT *t0, const TT *t1,
                                                                      const TT *t_eval, const uint8_t *mask, T *ys) {
    const long long b = (long long)blockIdx.x * 256 + threadIdx.x;
    if (b >= batch) return;
    for (int e = 0; e < E; ++e) {
        if (!mask[b * E + e]) continue;
        const T x = (T)unit_time_over(t_eval[b * E + e], t0[b], span_is_dt ? t1[b] : t1[b] - t0[b]);
        for (int f = 0; f < F; ++f) ys[(b * E + e) * F + f] = horner(coeff, batch * F, b * F + f, degree, x);
    }
}

// large F: one workgroup per sample, threads over features
template <typename TT, typename T>
__global__ void __launch_bounds__(256) poly_eval_masked_block_kernel(int degree, int span_is_dt, long long batch, int F, int E, const T *coeff, const TT *t0, const TT *t1,
                                                                     const TT *t_eval, const uint8_t *mask, T *ys) {
    const long long b = blockIdx.x;
    for (int e = 0; e < E; ++e) {
        if (!mask[b * E + e]) continue;  // uniform over the workgroup
        const T x = (T)unit_time_over(t_eval[b * E + e], t0[b], span_is_dt ? t1[b] : t1[b] - t0[b]);
        for (int f = threadIdx.x; f < F; f += 256) ys[(b * E + e) * F + f] = horner(coeff, batch * F, b * F + f, degree, x);
    }
}

template <typename T>
__global__ void __launch_bounds__(256) select_rows_kernel(long long n, int width, const uint8_t *mask, const T *a, const T *b, T *out) {
    const long long i = (long long)blockIdx.x * 256 + threadIdx.x;
    if (i < n) out[i] = mask[i / width] ? a[i] : b[i];
}

// ------------------------------------------------------------------------------------------
// loop bookkeeping (adjoints.py:76-126, 150-255, 284-292)
// ------------------------------------------------------------------------------------------

static __global__ void loop_flags_clear_kernel(int32_t *flags) {
    if (threadIdx.x < TODE_LOOP_FLAG_WORDS) flags[threadIdx.x] = 0;
}

template <typename T> __global__ void __launch_bounds__(256) loop_advance_kernel(tode_loop_args a) {
    const long long b = (long long)blockIdx.x * 256 + threadIdx.x;
    int any_running = 0, any_failure = 0, n_eval_hits = 0;
    if (b < a.batch) {
        const T ts = ((const T *)a.t_start)[b], te = ((const T *)a.t_end)[b];
        const T dir = (te > ts) ? (T)1 : (T)-1;
        const bool running = a.running[b] != 0;
        const bool move = a.accept[b] != 0 && running;
        const T t0 = ((const T *)a.t)[b], dt = ((const T *)a.dt)[b];
        const T t_new = move ? (t0 + dt) : t0;
        ((T *)a.t_out)[b] = t_new;
        a.to_update[b] = move ? 1 : 0;
        const int64_t n_steps = a.n_steps[b] + (running ? 1 : 0);
        a.n_steps[b] = n_steps;
        if (move) a.n_accepted[b] += 1;
        // running = addcmul(-dir * t_end, dir, t) < 0
        const bool running_new = fma_(dir, t_new, -dir * te) < (T)0;
        a.running_out[b] = running_new ? 1 : 0;
        int64_t status = 0;
        if (a.method_status) status = a.method_status[b];
        if (a.controller_status) {
            const int64_t cs = a.controller_status[b];
            status = (a.method_status && status > cs) ? status : cs;
        }
        if (a.max_steps >= 0 && n_steps >= a.max_steps) status = TODE_REACHED_MAX_STEPS;
        a.status[b] = status;
        any_running = running_new ? 1 : 0;
        any_failure = status != 0 ? 1 : 0;
        if (a.n_eval > 0) {
            const int E = a.n_eval;
            const T *tev = (const T *)a.t_eval + b * E;
            for (int e = 0; e < E; ++e) {
                const bool hit = a.pending[b * E + e] != 0 && fma_(dir, t_new, -dir * tev[e]) >= (T)0;
                a.to_evaluate[b * E + e] = hit ? 1 : 0;
                if (hit) {
                    a.pending[b * E + e] = 0;
                    ++n_eval_hits;
                }
            }
        }
        const T dtn = running_new ? ((const T *)a.dt_next)[b] : dt;
        const T tlo = tmin(ts, te), thi = tmax(te, ts);
        ((T *)a.dt_out)[b] = tclamp(dtn, tlo - t_new, thi - t_new);
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        any_running |= __shfl_xor(any_running, off);
        any_failure |= __shfl_xor(any_failure, off);
        n_eval_hits += __shfl_xor(n_eval_hits, off);
    }
    if ((threadIdx.x & 63) == 0) {
        if (any_running) atomicOr(&a.flags[TODE_LOOP_ANY_RUNNING], 1);
        if (any_failure) atomicOr(&a.flags[TODE_LOOP_ANY_FAILURE], 1);
        if (n_eval_hits) atomicAdd(&a.flags[TODE_LOOP_N_TO_EVALUATE], n_eval_hits);
    }
}

template <typename TT, typename T>
__global__ void __launch_bounds__(256) loop_begin_kernel(long long batch, int F, int E, const TT *t_start, const TT *t_end, const TT *t_eval, const T *y0,
                                                         const TT *dt, TT *dt_out, uint8_t *pending, T *ys) {
    const long long b = (long long)blockIdx.x * 256 + threadIdx.x;
    if (b >= batch) return;
    const TT ts = t_start[b], te = t_end[b];
    const TT tlo = tmin(ts, te), thi = tmax(te, ts);
    dt_out[b] = tclamp(dt[b], tlo - ts, thi - ts);
    if (E > 0) {
        const bool at_start = t_eval[b * E] == ts;
        for (int e = 0; e < E; ++e) pending[b * E + e] = (e == 0 && at_start) ? 0 : 1;
        if (at_start)
            for (int f = 0; f < F; ++f) ys[b * E * F + f] = y0[b * F + f];
    }
}

static __global__ void __launch_bounds__(256) count_initialized_kernel(long long batch, int E, const uint8_t *pending, int64_t *out) {
    const long long b = (long long)blockIdx.x * 256 + threadIdx.x;
    if (b >= batch) return;
    out[b] = searchsorted_first_pending(pending + b * E, E);
}

// ------------------------------------------------------------------------------------------
// host side
// ------------------------------------------------------------------------------------------

static unsigned blocks_for(long long n, int per_block) { return (unsigned)((n + per_block - 1) / per_block); }


static int check_common(int32_t dtype, int64_t batch, int32_t F) {
    const int d = data_type(dtype), t = time_type(dtype);
    if ((d != TODE_F32 && d != TODE_F64) || (t != TODE_F32 && t != TODE_F64) || (dtype & ~(TODE_DTYPE_PAIR | 0xFF)))
        return fail(TODE_E_INVALID, "unknown dtype %d", dtype);
    if (batch < 0 || F <= 0) return fail(TODE_E_INVALID, "bad sizes: batch=%lld F=%d", (long long)batch, F);
    if (batch * (long long)F > (long long)INT_MAX * 256) return fail(TODE_E_UNSUPPORTED, "batch * features too large");
    return TODE_OK;
}

static int done(const char *what) { return check_hip(hipGetLastError(), what); }

#define TODE_T(dtype, ...)         \
    do {                           \
        if ((dtype) == TODE_F32) { \
            using T = float;       \
            __VA_ARGS__;           \
        } else {                   \
            using T = double;      \
            __VA_ARGS__;           \
        }                          \
    } while (0)

// TT = time type, T = data type
#define TODE_TT(dtype, ...)                      \
    do {                                         \
        if (time_type(dtype) == TODE_F32) {      \
            using TT = float;                    \
            TODE_T(data_type(dtype), __VA_ARGS__); \
        } else {                                 \
            using TT = double;                   \
            TODE_T(data_type(dtype), __VA_ARGS__); \
        }                                        \
    } while (0)

// dispatch on (controller kind, norm) at compile time
#define TODE_CN(kind, norm, ...)                                         \
    do {                                                                 \
        if ((kind) == TODE_CTRL_PID && (norm) == TODE_NORM_RMS) {        \
            constexpr int CTRL = 1, NORM = TODE_NORM_RMS;                \
            __VA_ARGS__;                                                 \
        } else if ((kind) == TODE_CTRL_PID) {                            \
            constexpr int CTRL = 1, NORM = TODE_NORM_MAX;                \
            __VA_ARGS__;                                                 \
        } else if ((norm) == TODE_NORM_RMS) {                            \
            constexpr int CTRL = 0, NORM = TODE_NORM_RMS;                \
            __VA_ARGS__;                                                 \
        } else {                                                         \
            constexpr int CTRL = 0, NORM = TODE_NORM_MAX;                \
            __VA_ARGS__;                                                 \
        }                                                                \
    } while (0)

static int check_ctrl(const tode_controller *c, int32_t order, const void *prev, const void *pprev, void *prev_out, void *pprev_out) {
    if (!c) return fail(TODE_E_INVALID, "null controller");
    if (c->kind != TODE_CTRL_INTEGRAL && c->kind != TODE_CTRL_PID) return fail(TODE_E_INVALID, "unknown controller kind %d", c->kind);
    if (order <= 0) return fail(TODE_E_INVALID, "method order must be positive, got %d", order);
    if (c->kind == TODE_CTRL_PID && (!prev || !pprev || !prev_out || !pprev_out)) return fail(TODE_E_INVALID, "the PID controller needs its error ratio history");
    return TODE_OK;
}

}  // namespace tode

using namespace tode;

extern "C" {

int tode_tableau(int32_t method, double *c, double *a, double *b_err, double *b_other, int32_t *n_other) {
    if (method != TODE_DOPRI5 && method != TODE_TSIT5) return fail(TODE_E_INVALID, "unknown method %d", method);
    if (!c || !a || !b_err || !b_other || !n_other) return fail(TODE_E_INVALID, "null pointer");
    auto fill = [&](auto tab) {
        using Tab = decltype(tab);
        for (int i = 0; i < 7; ++i) {
            c[i] = Tab::c[i];
            b_err[i] = Tab::b_err[i];
            for (int j = 0; j < 7; ++j) a[i * 7 + j] = Tab::a[i][j];
        }
        *n_other = Tab::n_other;
        for (int r = 0; r < 3; ++r)
            for (int j = 0; j < 7; ++j) b_other[r * 7 + j] = r < Tab::n_other ? Tab::w[r][j] : 0.0;
    };
    if (method == TODE_TSIT5)
        fill(Tsit5Tab{});
    else
        fill(Dopri5Tab{});
    return TODE_OK;
}

int tode_erk_stage(int32_t dtype, int64_t batch, int32_t F, int32_t n_terms, const double *a, double c, const void *t0, const void *dt,
                   const void *y0, const void *k, void *y_out, void *t_out, void *stream) {
    if (int rc = check_common(dtype, batch, F)) return rc;
    if (n_terms < 0 || n_terms > TODE_MAX_STAGES) return fail(TODE_E_UNSUPPORTED, "n_terms=%d outside 0..%d", n_terms, TODE_MAX_STAGES);
    if (batch == 0) return TODE_OK;
    if ((n_terms > 0 && (!a || !k)) || !dt || !y0 || !y_out || (t_out && !t0)) return fail(TODE_E_INVALID, "null pointer");
    Coeffs co{};
    for (int j = 0; j < n_terms; ++j) co.v[j] = a[j];
    TODE_TT(dtype, hipLaunchKernelGGL((erk_stage_kernel<TT, T>), dim3(blocks_for(batch * F, 256)), dim3(256), 0, (hipStream_t)stream, (long long)batch, F,
                                      n_terms, co, c, (const TT *)t0, (const TT *)dt, (const T *)y0, (const T *)k, (T *)y_out, (TT *)t_out));
    return done("tode_erk_stage launch");
}

int tode_erk_combine(int32_t dtype, int64_t batch, int32_t F, int32_t S, const double *w, const void *dt, const void *k, const void *y0, void *out,
                     void *stream) {
    if (int rc = check_common(dtype, batch, F)) return rc;
    if (S <= 0 || S > TODE_MAX_STAGES) return fail(TODE_E_UNSUPPORTED, "n_stages=%d outside 1..%d", S, TODE_MAX_STAGES);
    if (batch == 0) return TODE_OK;
    if (!w || !dt || !k || !out) return fail(TODE_E_INVALID, "null pointer");
    Coeffs co{};
    for (int j = 0; j < S; ++j) co.v[j] = w[j];
    TODE_TT(dtype, hipLaunchKernelGGL((erk_combine_kernel<TT, T>), dim3(blocks_for(batch * F, 256)), dim3(256), 0, (hipStream_t)stream, (long long)batch, F, S,
                                      co, (const TT *)dt, (const T *)k, (const T *)y0, (T *)out));
    return done("tode_erk_combine launch");
}

int tode_error_scale(int32_t dtype, int64_t batch, int32_t F, double atol, double rtol, const void *y0, const void *y1, const void *err, void *out,
                     void *stream) {
    if (int rc = check_common(dtype, batch, F)) return rc;
    if (batch == 0) return TODE_OK;
    if (!y0 || !y1 || !err || !out) return fail(TODE_E_INVALID, "null pointer");
    TODE_T(data_type(dtype), hipLaunchKernelGGL(error_scale_kernel<T>, dim3(blocks_for(batch * F, 256)), dim3(256), 0, (hipStream_t)stream,
                                                (long long)batch * F, (T)(float)atol, (T)(float)rtol, (const T *)y0, (const T *)y1, (const T *)err, (T *)out));
    return done("tode_error_scale launch");
}

int tode_row_norm(int32_t dtype, int32_t norm, int64_t batch, int32_t F, const void *x, void *out, void *stream) {
    if (int rc = check_common(dtype, batch, F)) return rc;
    if (norm != TODE_NORM_RMS && norm != TODE_NORM_MAX) return fail(TODE_E_INVALID, "unknown norm %d", norm);
    if (batch == 0) return TODE_OK;
    if (!x || !out) return fail(TODE_E_INVALID, "null pointer");
    hipStream_t s = (hipStream_t)stream;
    TODE_T(data_type(dtype), TODE_CN(0, norm, {
               (void)CTRL;
               if (F < 64)
                   hipLaunchKernelGGL((row_norm_thread_kernel<T, NORM>), dim3(blocks_for(batch, 256)), dim3(256), 0, s, (long long)batch, F, (const T *)x, (T *)out);
               else
                   hipLaunchKernelGGL((row_norm_wave_kernel<T, NORM>), dim3(blocks_for(batch, 4)), dim3(256), 0, s, (long long)batch, F, (const T *)x, (T *)out);
           }));
    return done("tode_row_norm launch");
}

int tode_control(int32_t dtype, const tode_controller *c, int32_t order, int64_t batch, const void *norm, const void *dt, const void *prev,
                 const void *pprev, uint8_t *accept, void *dt_next, void *ratio, int64_t *status, void *prev_out, void *pprev_out, void *stream) {
    if (int rc = check_common(dtype, batch, 1)) return rc;
    if (int rc = check_ctrl(c, order, prev, pprev, prev_out, pprev_out)) return rc;
    if (batch == 0) return TODE_OK;
    if (!norm || !dt || !accept || !dt_next || !status) return fail(TODE_E_INVALID, "null pointer");
    ControlOut o{accept, dt_next, ratio, prev_out, pprev_out, status};
    TODE_TT(dtype, TODE_CN(c->kind, TODE_NORM_RMS, {
                (void)NORM;
                const StepLimits<TT> lim{(TT)c->dt_min, (TT)c->dt_max};
                hipLaunchKernelGGL((control_kernel<TT, T, CTRL>), dim3(blocks_for(batch, 256)), dim3(256), 0, (hipStream_t)stream,
                                   make_ctrl<T>(*c, (double)order), lim, (long long)batch, (const T *)norm, (const TT *)dt, (const T *)prev, (const T *)pprev, o);
            }));
    return done("tode_control launch");
}

int tode_adapt_step(int32_t dtype, const tode_controller *c, int32_t order, int32_t norm, int64_t batch, int32_t F, const void *dt, const void *y0,
                    const void *y1, const void *err, const void *prev, const void *pprev, uint8_t *accept, void *dt_next, void *ratio, int64_t *status,
                    void *prev_out, void *pprev_out, void *stream) {
    if (int rc = check_common(dtype, batch, F)) return rc;
    if (int rc = check_ctrl(c, order, prev, pprev, prev_out, pprev_out)) return rc;
    if (norm != TODE_NORM_RMS && norm != TODE_NORM_MAX) return fail(TODE_E_INVALID, "unknown norm %d", norm);
    if (batch == 0) return TODE_OK;
    if (!dt || !y0 || !y1 || !err || !accept || !dt_next || !status) return fail(TODE_E_INVALID, "null pointer");
    ControlOut o{accept, dt_next, ratio, prev_out, pprev_out, status};
    hipStream_t s = (hipStream_t)stream;
    TODE_TT(dtype, TODE_CN(c->kind, norm, {
                const CtrlParams<T> cp = make_ctrl<T>(*c, (double)order);
                const StepLimits<TT> lim{(TT)c->dt_min, (TT)c->dt_max};
                if (F < 64)
                    hipLaunchKernelGGL((adapt_thread_kernel<TT, T, CTRL, NORM>), dim3(blocks_for(batch, 256)), dim3(256), 0, s, cp, lim, (long long)batch, F,
                                       (const TT *)dt, (const T *)y0, (const T *)y1, (const T *)err, (const T *)prev, (const T *)pprev, o);
                else
                    hipLaunchKernelGGL((adapt_wave_kernel<TT, T, CTRL, NORM>), dim3(blocks_for(batch, 4)), dim3(256), 0, s, cp, lim, (long long)batch, F,
                                       (const TT *)dt, (const T *)y0, (const T *)y1, (const T *)err, (const T *)prev, (const T *)pprev, o);
            }));
    return done("tode_adapt_step launch");
}

int tode_initial_step_a(int32_t dtype, int32_t norm, int64_t batch, int32_t F, double atol, double rtol, const void *t_start, const void *t_end,
                        const void *y0, const void *f0, void *h0, void *y1, void *t1, void *stream) {
    if (int rc = check_common(dtype, batch, F)) return rc;
    if (norm != TODE_NORM_RMS && norm != TODE_NORM_MAX) return fail(TODE_E_INVALID, "unknown norm %d", norm);
    if (batch == 0) return TODE_OK;
    if (!t_start || !t_end || !y0 || !f0 || !h0 || !y1 || !t1) return fail(TODE_E_INVALID, "null pointer");
    hipStream_t s = (hipStream_t)stream;
    TODE_TT(dtype, TODE_CN(0, norm, {
                (void)CTRL;
                const T at = (T)(float)atol, rt = (T)(float)rtol;
                if (F < 64)
                    hipLaunchKernelGGL((initial_a_thread_kernel<TT, T, NORM>), dim3(blocks_for(batch, 256)), dim3(256), 0, s, (long long)batch, F, at, rt,
                                       (const TT *)t_start, (const TT *)t_end, (const T *)y0, (const T *)f0, (T *)h0);
                else
                    hipLaunchKernelGGL((initial_a_wave_kernel<TT, T, NORM>), dim3(blocks_for(batch, 4)), dim3(256), 0, s, (long long)batch, F, at, rt,
                                       (const TT *)t_start, (const TT *)t_end, (const T *)y0, (const T *)f0, (T *)h0);
                hipLaunchKernelGGL((initial_probe_kernel<TT, T>), dim3(blocks_for(batch * F, 256)), dim3(256), 0, s, (long long)batch, F, (const TT *)t_start,
                                   (const TT *)t_end, (const T *)y0, (const T *)f0, (const T *)h0, (T *)y1, (TT *)t1);
            }));
    return done("tode_initial_step_a launch");
}

int tode_tolerance_scale(int32_t dtype, int64_t batch, int32_t F, double atol, double rtol, const void *y_ref, const void *v, void *out, void *stream) {
    if (int rc = check_common(dtype, batch, F)) return rc;
    if (batch == 0) return TODE_OK;
    if (!y_ref || !v || !out) return fail(TODE_E_INVALID, "null pointer");
    TODE_T(data_type(dtype), hipLaunchKernelGGL(tolerance_scale_kernel<T>, dim3(blocks_for(batch * F, 256)), dim3(256), 0, (hipStream_t)stream,
                                                (long long)batch * F, (T)(float)atol, (T)(float)rtol, (const T *)y_ref, (const T *)v, (T *)out));
    return done("tode_tolerance_scale launch");
}

int tode_initial_step_a_norms(int32_t dtype, int64_t batch, int32_t F, const void *t_start, const void *t_end, const void *y0, const void *f0,
                              const void *d0, const void *d1, void *h0, void *y1, void *t1, void *stream) {
    if (int rc = check_common(dtype, batch, F)) return rc;
    if (batch == 0) return TODE_OK;
    if (!t_start || !t_end || !y0 || !f0 || !d0 || !d1 || !h0 || !y1 || !t1) return fail(TODE_E_INVALID, "null pointer");
    hipStream_t s = (hipStream_t)stream;
    TODE_TT(dtype, {
        hipLaunchKernelGGL((initial_h0_kernel<TT, T>), dim3(blocks_for(batch, 256)), dim3(256), 0, s, (long long)batch, (const TT *)t_start, (const TT *)t_end,
                           (const T *)d0, (const T *)d1, (T *)h0);
        hipLaunchKernelGGL((initial_probe_kernel<TT, T>), dim3(blocks_for(batch * F, 256)), dim3(256), 0, s, (long long)batch, F, (const TT *)t_start,
                           (const TT *)t_end, (const T *)y0, (const T *)f0, (const T *)h0, (T *)y1, (TT *)t1);
    });
    return done("tode_initial_step_a_norms launch");
}

int tode_initial_step_b_norms(int32_t dtype, int32_t kind, int32_t order, int64_t batch, const void *t_start, const void *t_end, const void *h0,
                              const void *d1, const void *d2n, void *dt0, void *stream) {
    if (int rc = check_common(dtype, batch, 1)) return rc;
    if (kind != TODE_CTRL_INTEGRAL && kind != TODE_CTRL_PID) return fail(TODE_E_INVALID, "unknown controller kind %d", kind);
    if (order <= 0) return fail(TODE_E_INVALID, "method order must be positive, got %d", order);
    if (batch == 0) return TODE_OK;
    if (!t_start || !t_end || !h0 || !d1 || !d2n || !dt0) return fail(TODE_E_INVALID, "null pointer");
    TODE_TT(dtype, hipLaunchKernelGGL((initial_dt_kernel<TT, T>), dim3(blocks_for(batch, 256)), dim3(256), 0, (hipStream_t)stream, kind, 1.0 / (double)order,
                                      (long long)batch, (const TT *)t_start, (const TT *)t_end, (const T *)h0, (const T *)d1, (const T *)d2n, (TT *)dt0));
    return done("tode_initial_step_b_norms launch");
}

int tode_initial_step_b(int32_t dtype, int32_t kind, int32_t norm, int32_t order, int64_t batch, int32_t F, double atol, double rtol,
                        const void *t_start, const void *t_end, const void *y0, const void *f0, const void *f1, const void *h0, void *dt0, void *stream) {
    if (int rc = check_common(dtype, batch, F)) return rc;
    if (kind != TODE_CTRL_INTEGRAL && kind != TODE_CTRL_PID) return fail(TODE_E_INVALID, "unknown controller kind %d", kind);
    if (norm != TODE_NORM_RMS && norm != TODE_NORM_MAX) return fail(TODE_E_INVALID, "unknown norm %d", norm);
    if (order <= 0) return fail(TODE_E_INVALID, "method order must be positive, got %d", order);
    if (batch == 0) return TODE_OK;
    if (!t_start || !t_end || !y0 || !f0 || !f1 || !h0 || !dt0) return fail(TODE_E_INVALID, "null pointer");
    hipStream_t s = (hipStream_t)stream;
    const double inv_order = 1.0 / (double)order;
    TODE_TT(dtype, TODE_CN(0, norm, {
                (void)CTRL;
                const T at = (T)(float)atol, rt = (T)(float)rtol;
                if (F < 64)
                    hipLaunchKernelGGL((initial_b_thread_kernel<TT, T, NORM>), dim3(blocks_for(batch, 256)), dim3(256), 0, s, kind, inv_order, (long long)batch, F,
                                       at, rt, (const TT *)t_start, (const TT *)t_end, (const T *)y0, (const T *)f0, (const T *)f1, (const T *)h0, (TT *)dt0);
                else
                    hipLaunchKernelGGL((initial_b_wave_kernel<TT, T, NORM>), dim3(blocks_for(batch, 4)), dim3(256), 0, s, kind, inv_order, (long long)batch, F,
                                       at, rt, (const TT *)t_start, (const TT *)t_end, (const T *)y0, (const T *)f0, (const T *)f1, (const T *)h0, (TT *)dt0);
            }));
    return done("tode_initial_step_b launch");
}

int tode_quartic_build(int32_t dtype, int32_t method, int64_t batch, int32_t F, const void *dt, const void *y0, const void *y1, const void *k,
                       void *coeff, void *stream) {
    if (int rc = check_common(dtype, batch, F)) return rc;
    if (method != TODE_DOPRI5 && method != TODE_TSIT5) return fail(TODE_E_INVALID, "unknown method %d", method);
    if (batch == 0) return TODE_OK;
    if (!dt || !y0 || !y1 || !k || !coeff) return fail(TODE_E_INVALID, "null pointer");
    const dim3 grid(blocks_for(batch * F, 256));
    hipStream_t s = (hipStream_t)stream;
    TODE_TT(dtype, {
        if (method == TODE_TSIT5)
            hipLaunchKernelGGL((quartic_build_kernel<TT, T, 1>), grid, dim3(256), 0, s, (long long)batch, F, (const TT *)dt, (const T *)y0, (const T *)y1,
                               (const T *)k, (T *)coeff);
        else
            hipLaunchKernelGGL((quartic_build_kernel<TT, T, 0>), grid, dim3(256), 0, s, (long long)batch, F, (const TT *)dt, (const T *)y0, (const T *)y1,
                               (const T *)k, (T *)coeff);
    });
    return done("tode_quartic_build launch");
}

int tode_quartic_from_mid(int32_t dtype, int64_t batch, int32_t F, const void *dt, const void *y0, const void *y1, const void *k_first,
                          const void *k_last, const void *y_mid, void *coeff, void *stream) {
    if (int rc = check_common(dtype, batch, F)) return rc;
    if (batch == 0) return TODE_OK;
    if (!dt || !y0 || !y1 || !k_first || !k_last || !y_mid || !coeff) return fail(TODE_E_INVALID, "null pointer");
    TODE_TT(dtype, hipLaunchKernelGGL((quartic_from_mid_kernel<TT, T>), dim3(blocks_for(batch * F, 256)), dim3(256), 0, (hipStream_t)stream, (long long)batch,
                                      F, (const TT *)dt, (const T *)y0, (const T *)y1, (const T *)k_first, (const T *)k_last, (const T *)y_mid, (T *)coeff));
    return done("tode_quartic_from_mid launch");
}

int tode_cubic_build(int32_t dtype, int64_t batch, int32_t F, const void *dt, const void *y0, const void *y1, const void *k_first,
                     const void *k_last, void *coeff, void *stream) {
    if (int rc = check_common(dtype, batch, F)) return rc;
    if (batch == 0) return TODE_OK;
    if (!dt || !y0 || !y1 || !k_first || !k_last || !coeff) return fail(TODE_E_INVALID, "null pointer");
    TODE_TT(dtype, hipLaunchKernelGGL((cubic_build_kernel<TT, T>), dim3(blocks_for(batch * F, 256)), dim3(256), 0, (hipStream_t)stream, (long long)batch, F,
                                      (const TT *)dt, (const T *)y0, (const T *)y1, (const T *)k_first, (const T *)k_last, (T *)coeff));
    return done("tode_cubic_build launch");
}

int tode_poly_eval(int32_t dtype, int32_t degree, int32_t span_is_dt, int64_t batch, int32_t F, int64_t count, const void *coeff, const void *t0,
                   const void *t1, const void *t, const int64_t *idx, void *out, void *stream) {
    if (int rc = check_common(dtype, batch, F)) return rc;
    if (degree < 1 || degree > 4) return fail(TODE_E_INVALID, "degree %d outside 1..4", degree);
    if (count < 0) return fail(TODE_E_INVALID, "negative count");
    if (count == 0) return TODE_OK;
    if (batch == 0) return fail(TODE_E_INVALID, "evaluation points but an empty batch");
    if (!coeff || !t0 || !t1 || !t || !idx || !out) return fail(TODE_E_INVALID, "null pointer");
    TODE_TT(dtype, hipLaunchKernelGGL((poly_eval_kernel<TT, T>), dim3(blocks_for(count * F, 256)), dim3(256), 0, (hipStream_t)stream, degree, span_is_dt != 0,
                                      (long long)batch, F, (long long)count, (const T *)coeff, (const TT *)t0, (const TT *)t1, (const TT *)t, idx, (T *)out));
    return done("tode_poly_eval launch");
}

int tode_poly_eval_masked(int32_t dtype, int32_t degree, int32_t span_is_dt, int64_t batch, int32_t F, int32_t E, const void *coeff, const void *t0,
                          const void *t1, const void *t_eval, const uint8_t *mask, void *ys, void *stream) {
    if (int rc = check_common(dtype, batch, F)) return rc;
    if (degree < 1 || degree > 4) return fail(TODE_E_INVALID, "degree %d outside 1..4", degree);
    if (E < 0) return fail(TODE_E_INVALID, "negative n_eval");
    if (batch == 0 || E == 0) return TODE_OK;
    if (!coeff || !t0 || !t1 || !t_eval || !mask || !ys) return fail(TODE_E_INVALID, "null pointer");
    hipStream_t s = (hipStream_t)stream;
    TODE_TT(dtype, {
        if (F < 64)
            hipLaunchKernelGGL((poly_eval_masked_thread_kernel<TT, T>), dim3(blocks_for(batch, 256)), dim3(256), 0, s, degree, span_is_dt != 0, (long long)batch, F, E,
                               (const T *)coeff, (const TT *)t0, (const TT *)t1, (const TT *)t_eval, mask, (T *)ys);
        else
            hipLaunchKernelGGL((poly_eval_masked_block_kernel<TT, T>), dim3((unsigned)batch), dim3(256), 0, s, degree, span_is_dt != 0, (long long)batch, F, E, (const T *)coeff,
                               (const TT *)t0, (const TT *)t1, (const TT *)t_eval, mask, (T *)ys);
    });
    return done("tode_poly_eval_masked launch");
}

int tode_select_rows(int32_t dtype, int64_t batch, int32_t width, const uint8_t *mask, const void *a, const void *b, void *out, void *stream) {
    if (int rc = check_common(dtype, batch, width)) return rc;
    if (batch == 0) return TODE_OK;
    if (!mask || !a || !b || !out) return fail(TODE_E_INVALID, "null pointer");
    TODE_T(data_type(dtype), hipLaunchKernelGGL(select_rows_kernel<T>, dim3(blocks_for(batch * width, 256)), dim3(256), 0, (hipStream_t)stream,
                                                (long long)batch * width, width, mask, (const T *)a, (const T *)b, (T *)out));
    return done("tode_select_rows launch");
}

int tode_loop_advance(const tode_loop_args *a, void *stream) {
    if (!a) return fail(TODE_E_INVALID, "null argument struct");
    if (int rc = check_common(a->dtype, a->batch, a->n_features)) return rc;
    if (a->n_eval < 0) return fail(TODE_E_INVALID, "negative n_eval");
    if (!a->flags) return fail(TODE_E_INVALID, "null flags pointer");
    hipStream_t s = (hipStream_t)stream;
    hipLaunchKernelGGL(loop_flags_clear_kernel, dim3(1), dim3(64), 0, s, a->flags);
    if (a->batch == 0) return done("tode_loop_advance launch");
    if (!a->t_start || !a->t_end || !a->t || !a->dt || !a->y || !a->running || !a->y_new || !a->accept || !a->dt_next || !a->t_out || !a->dt_out ||
        !a->y_out || !a->running_out || !a->to_update || !a->status || !a->n_steps || !a->n_accepted)
        return fail(TODE_E_INVALID, "null pointer");
    if (a->n_eval > 0 && (!a->t_eval || !a->pending || !a->to_evaluate)) return fail(TODE_E_INVALID, "n_eval > 0 needs t_eval, pending and to_evaluate");
    if (a->t_out == a->t || a->dt_out == a->dt || a->y_out == a->y || a->y_out == a->y_new)
        return fail(TODE_E_INVALID, "outputs must not alias inputs");
    const long long n = a->batch * a->n_features;
    // the time side of the bookkeeping, then y where to_update (written by the first kernel, same stream)
    TODE_T(time_type(a->dtype), hipLaunchKernelGGL(loop_advance_kernel<T>, dim3(blocks_for(a->batch, 256)), dim3(256), 0, s, *a));
    TODE_T(data_type(a->dtype), hipLaunchKernelGGL(select_rows_kernel<T>, dim3(blocks_for(n, 256)), dim3(256), 0, s, n, a->n_features,
                                                   (const uint8_t *)a->to_update, (const T *)a->y_new, (const T *)a->y, (T *)a->y_out));
    return done("tode_loop_advance launch");
}

int tode_loop_begin(int32_t dtype, int64_t batch, int32_t F, int32_t E, const void *t_start, const void *t_end, const void *t_eval, const void *y0,
                    const void *dt, void *dt_out, uint8_t *pending, void *ys, void *stream) {
    if (int rc = check_common(dtype, batch, F)) return rc;
    if (E < 0) return fail(TODE_E_INVALID, "negative n_eval");
    if (batch == 0) return TODE_OK;
    if (!t_start || !t_end || !y0 || !dt || !dt_out) return fail(TODE_E_INVALID, "null pointer");
    if (E > 0 && (!t_eval || !pending || !ys)) return fail(TODE_E_INVALID, "n_eval > 0 needs t_eval, pending and ys");
    TODE_TT(dtype, hipLaunchKernelGGL((loop_begin_kernel<TT, T>), dim3(blocks_for(batch, 256)), dim3(256), 0, (hipStream_t)stream, (long long)batch, F, E,
                                      (const TT *)t_start, (const TT *)t_end, (const TT *)t_eval, (const T *)y0, (const TT *)dt, (TT *)dt_out, pending,
                                      (T *)ys));
    return done("tode_loop_begin launch");
}

int tode_count_initialized(int64_t batch, int32_t E, const uint8_t *pending, int64_t *n_initialized, void *stream) {
    if (batch < 0 || E < 0) return fail(TODE_E_INVALID, "bad sizes");
    if (batch == 0) return TODE_OK;
    if ((E > 0 && !pending) || !n_initialized) return fail(TODE_E_INVALID, "null pointer");
    hipLaunchKernelGGL(count_initialized_kernel, dim3(blocks_for(batch, 256)), dim3(256), 0, (hipStream_t)stream, (long long)batch, E, pending, n_initialized);
    return done("tode_count_initialized launch");
}

}  // extern "C"
