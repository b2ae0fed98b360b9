// Per-step kernels for right-hand sides that live outside the library (any Python
// f): the loop state stays on the device, the host enqueues
//     6 x (stage kernel, user f)  ->  finish kernel  ->  loop-control kernel
// per iteration and never waits for a step; it polls the flag block every few
// iterations.  Once the loop has ended on the device, kernels of iterations
// that were enqueued speculatively return immediately.
//
// Rows of fewer than 64 features: one thread per sample, features walked with run-time
// loops in the same order as a scalar evaluation.  Longer rows: one wavefront per sample,
// lanes strided over the features, norms in the fixed order of wave_row_norm (the stage
// kernel is per element either way).  The stage arrays necessarily go through HBM because
// f is external.
//
// Time and data may have different types (problems.py:44-56): every kernel is a template of the
// time type TT and the data type T.  Times, steps and their limits are TT; the state, the
// derivatives, the tolerances, the error ratio and the step factor are T; the step is converted
// to T where it multiplies derivatives and the factor to TT where it multiplies the step, as in
// the reference (runge_kutta.py:247, step_size_controllers.py:419, interpolation.py:32).
#include "tode_solve.h"
#include "tode_adjoint.h"

namespace tode {

template <typename TT, typename T> struct StepParams {
    // problem
    const T *y0;
    const TT *t_start, *t_end, *t_eval;
    long long batch;
    int F, E;
    int max_steps;
    // loop state (device, owned by the caller for the duration of a solve)
    TT *t, *dt;                   // [B], [B]
    T *y, *k0;                    // [B,F], [B,F] (FSAL derivative)
    T *ratio_prev, *ratio_pprev;  // [B] the last two accepted error ratios (PID history)
    int32_t *running, *cursor, *n_steps, *n_accepted, *status, *monotone;
    uint8_t *pending;  // [B,E]
    T *ys;             // [B,max(E,1),F]
    int32_t *flags;    // TODE_STEP_FLAG_*
    // per-iteration buffers
    T *ystage[7];    // [B,F] stage inputs; ystage[6] is y1
    const T *k[7];   // [B,F] stage derivatives; k[0] aliases k0
    TT *tnode;       // [B]
    CtrlParams<T> cp;
    TT dt_min, dt_max;  // limits of the step (step_size_controllers.py:406-422), in the time type
    const TT *fixed_dt;  // [B] CTRL == 2: the fixed step (step_size_controllers.py:116-167)
    double inv_order;    // 1 / convergence order of the step method, the exponent of the start step rule
    bool carry;          // the method keeps the last stage's derivative as the next step's first (Dopri5, Tsit5)
};

// Heun 2(1) (heun.py:10-13): c = (0, 1), a_10 = 1, b = (1/2, 1/2), low-order weights (1, 0), b_err = b - b_low in
// float64 (runge_kutta.py:84-88).  Neither first-same-as-last nor solution-same-as-last-stage: the first stage is
// evaluated anew in every step and y1 = y0 + sum_s (dt b_s) k_s.  Euler (euler.py:29-56) has one stage and no tableau.
struct HeunTab {
    static constexpr double c[7] = {0.0, 1.0};
    static constexpr double a[7][7] = {{0}, {1.0}};
    static constexpr double b[2] = {0.5, 0.5};
    static constexpr double b_err[2] = {0.5 - 1.0, 0.5 - 0.0};
};
template <int METHOD> struct TabOf { using type = Dopri5Tab; };
template <> struct TabOf<1> { using type = Tsit5Tab; };
template <> struct TabOf<2> { using type = HeunTab; };
// stages per step, and the convergence order the controllers divide by (dopri5.py:49-51, tsit5.py:119-121, heun.py,
// euler.py)
__host__ __device__ constexpr int stages_of(int method) { return method <= TODE_TSIT5 ? 7 : (method == TODE_HEUN ? 2 : 1); }
__host__ __device__ constexpr double order_of(int method) { return method <= TODE_TSIT5 ? 5.0 : (method == TODE_HEUN ? 2.0 : 1.0); }

// ystage[s] = fma(dt, sum_j a_sj k_j, y); tnode = fma(c_s, dt, t)   (runge_kutta.py:259-262)
template <typename TT, typename T, int METHOD, int S> __global__ void __launch_bounds__(256) stage_kernel(const StepParams<TT, T> p) {
    using Tab = typename TabOf<METHOD>::type;
    if (p.flags[TODE_STEP_FLAG_STOPPED]) return;
    const long long i = (long long)blockIdx.x * 256 + threadIdx.x;
    const long long n = p.batch * p.F;
    if (i >= n) return;
    const long long b = i / p.F;
    const T dt = (T)p.dt[b];
    T s = 0;
#pragma unroll
    for (int j = 0; j < S; ++j) s = fma_((T)Tab::a[S][j], p.k[j][i], s);
    p.ystage[S][i] = fma_(dt, s, p.y[i]);
    if (i - b * p.F == 0) p.tnode[b] = fma_((TT)Tab::c[S], p.dt[b], p.t[b]);
}

// Start step, first half (step_size_controllers.py:459-479): from f0 = f(t0, y0) compute h0,
// y1 = y0 + dir*h0*f0 -> ystage[1], t1 -> tnode; h0 (data type) is parked in ratio_prev.
template <typename TT, typename T> __global__ void __launch_bounds__(256) init_a_kernel(const StepParams<TT, T> p) {
    const long long b = (long long)blockIdx.x * 256 + threadIdx.x;
    if (b >= p.batch) return;
    const int F = p.F;
    const CtrlParams<T> &cp = p.cp;
    const T *y0 = p.y0 + b * F, *f0 = p.k[0] + b * F;
    const T sf = (T)__builtin_sqrt((double)F);
    T a0 = 0, a1 = 0;
    for (int f = 0; f < F; ++f) {
        T inv = (T)1 / fma_(cp.rtol, abs_(y0[f]), cp.atol);
        T x0 = (y0[f] * inv) / sf, x1 = (f0[f] * inv) / sf;
        if (F <= 3) {
            a0 = fma_(x0, x0, a0);
            a1 = fma_(x1, x1, a1);
        } else {
            T s0 = x0 * x0, s1 = x1 * x1;
            a0 = a0 + s0;
            a1 = a1 + s1;
        }
    }
    const T d0 = sqrt_(a0), d1 = sqrt_(a1);
    const TT ts = p.t_start[b], te = p.t_end[b];
    const bool fwd = te > ts;
    T h0 = (d0 < (T)1e-5 || d1 < (T)1e-5) ? (T)1e-6 : ((T)0.01 * d0) / d1;
    h0 = tmin(h0, (T)abs_(te - ts));
    const T dh = (fwd ? (T)1 : (T)-1) * h0;
    T *y1 = p.ystage[1] + b * F;
    for (int f = 0; f < F; ++f) y1[f] = fma_(dh, f0[f], y0[f]);
    p.tnode[b] = fma_(fwd ? (TT)1 : (TT)-1, (TT)h0, ts);
    p.ratio_prev[b] = h0;
}

// Loop state at t_start; with FROM_F1 also the second half of the start step
// (step_size_controllers.py:481-490 integral, 826-835 PID) from f1 = k[1].
template <typename TT, typename T, int CTRL, bool FROM_F1>
__global__ void __launch_bounds__(256) init_b_kernel(const StepParams<TT, T> p, const TT *dt0) {
    const long long b = (long long)blockIdx.x * 256 + threadIdx.x;
    if (b >= p.batch) return;
    const int F = p.F, E = p.E;
    const CtrlParams<T> &cp = p.cp;
    const T *y0 = p.y0 + b * F, *f0 = p.k[0] + b * F;
    const TT ts = p.t_start[b], te = p.t_end[b];
    const bool fwd = te > ts;
    const T dir = fwd ? (T)1 : (T)-1;
    TT dt;
    if (FROM_F1) {
        const T *f1 = p.k[1] + b * F;
        const T sf = (T)__builtin_sqrt((double)F);
        const T h0 = p.ratio_prev[b];
        T a1 = 0, a2 = 0;
        for (int f = 0; f < F; ++f) {
            T inv = (T)1 / fma_(cp.rtol, abs_(y0[f]), cp.atol);
            T x1 = (f0[f] * inv) / sf;
            T df = f1[f] - f0[f];
            T x2 = (df * inv) / sf;
            if (F <= 3) {
                a1 = fma_(x1, x1, a1);
                a2 = fma_(x2, x2, a2);
            } else {
                T s1 = x1 * x1, s2 = x2 * x2;
                a1 = a1 + s1;
                a2 = a2 + s2;
            }
        }
        const T d1 = sqrt_(a1);
        T d2 = sqrt_(a2) / h0;
        if (CTRL == 0 && h0 == (T)0) d2 = (T)__builtin_huge_val();
        const T m = tmax(d1, d2);
        T h1;
        if (m <= (T)1e-15) {
            h1 = tmax((T)1e-6, h0 * (T)1e-3);
        } else {
            T rm = (T)1 / m;
            h1 = rpow<T>(rm * (T)0.01, p.inv_order);
        }
        dt = (TT)(dir * tmin((T)100 * h0, h1));
    } else {
        dt = dt0[b];
    }
    const TT tlo = tmin(ts, te), thi = tmax(te, ts);
    p.t[b] = ts;
    p.dt[b] = tclamp(dt, tlo - ts, thi - ts);
    for (int f = 0; f < F; ++f) {
        p.y[b * F + f] = y0[f];
        if (p.carry) p.k0[b * F + f] = f0[f];
    }
    p.ratio_prev[b] = (T)1;
    p.ratio_pprev[b] = (T)1;
    p.running[b] = 1;
    p.n_steps[b] = 0;
    p.n_accepted[b] = 0;
    p.status[b] = 0;
    int cursor = 0, mono = 1;
    if (E > 0) {
        const TT *tev = p.t_eval + b * E;
        TT prev_te = tev[0];
        for (int e = 0; e < E; ++e) {
            TT cur = tev[e];
            if (e > 0 && !(fwd ? cur >= prev_te : cur <= prev_te)) mono = 0;
            prev_te = cur;
            p.pending[b * E + e] = 1;
        }
        if (tev[0] == ts) {
            for (int f = 0; f < F; ++f) p.ys[(b * E) * F + f] = y0[f];
            p.pending[b * E] = 0;
            cursor = 1;
        }
    }
    p.cursor[b] = cursor;
    p.monotone[b] = mono;
}

// Quartic of the attempted step for one feature, evaluated at time te (tsit5.py:123-139,
// dopri5.py:53-60, interpolation.py:25-40, 138-175).  ks[s] = k_s[b,f].
// The value that lane `src` of the wavefront holds; `src` is the same for all lanes.
__device__ __forceinline__ float wave_read(float v, int src) { return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), src)); }
__device__ __forceinline__ double wave_read(double v, int src) {
    const int lo = __builtin_amdgcn_readlane(__double2loint(v), src), hi = __builtin_amdgcn_readlane(__double2hiint(v), src);
    return __hiloint2double(hi, lo);
}

template <typename T> __device__ __forceinline__ T quartic_at(const T (&q)[5][1], T x) {
    T y = q[4][0];
    y = fma_(y, x, q[3][0]);
    y = fma_(y, x, q[2][0]);
    y = fma_(y, x, q[1][0]);
    return fma_(y, x, q[0][0]);
}

template <typename TT, typename T, int METHOD>
__device__ __forceinline__ T dense_value(TT t0, TT dt, T y0, T y1, const T (&ks)[7], bool fused, TT te) {
    if (METHOD == TODE_EULER) {
        // linear (interpolation.py:48-62): the step itself divides, not (t0 + dt) - t0
        return fma_(y1 - y0, (T)unit_time_over<TT>(te, t0, dt), y0);
    }
    if (METHOD == TODE_HEUN) {
        // Hermite cubic from the first and the last slope (interpolation.py:84-106), ks[1] = f at the step's end
        const T h = (T)dt, f0 = ks[0], f1 = ks[1], d01 = y0 - y1;
        const T a = fma_((T)2, d01, h * (f0 + f1));
        const T b = fma_((T)-3, d01, h * fma_((T)-2, f0, -f1));
        const T x = (T)unit_time<TT>(te, t0, t0 + dt);
        T v = a;
        v = fma_(v, x, b);
        v = fma_(v, x, h * f0);
        return fma_(v, x, y0);
    }
    T q[5][1];
    quartic_elem<T, (METHOD == 1 ? 1 : 0)>((T)dt, y0, y1, ks, fused, q);
    return quartic_at<T>(q, (T)unit_time<TT>(te, t0, t0 + dt));
}

// Everything after the last stage of one loop iteration, for one sample per thread:
// error estimate, error ratio, accept/reject, PI/PID proposal, dt_min/dt_max, status,
// counters, dense output at the evaluation points the step passed, state update, running
// flag, dt clamp (runge_kutta.py:265-272, step_size_controllers.py:370-429 / 715-774,
// adjoints.py:150-255).
// FC: the row length where the launch knows it at compile time (0: p.F).  With it, and with Dopri5 / Tsit5, the
// thread loads its sample's rows once, into registers, and everything below works from there.
template <typename TT, typename T, int METHOD, int CTRL, int FC = 0> __global__ void __launch_bounds__(256) finish_kernel(const StepParams<TT, T> p) {
    using Tab = typename TabOf<METHOD>::type;
    constexpr int NS = stages_of(METHOD);
    constexpr bool ESTIMATE = METHOD != TODE_EULER;  // Euler has no error estimate: every step is accepted, the step kept
    if (p.flags[TODE_STEP_FLAG_STOPPED]) return;
    const long long b = (long long)blockIdx.x * 256 + threadIdx.x;
    if (b >= p.batch) return;
    const int F = FC > 0 ? FC : p.F, E = p.E;
    const CtrlParams<T> &cp = p.cp;
    const bool fused = F >= 58;
    const T sf = (T)__builtin_sqrt((double)F);
    const TT t0 = p.t[b], dt = p.dt[b];
    const T h = (T)dt;
    const TT ts = p.t_start[b], te = p.t_end[b];
    const bool fwd = te > ts;
    const T *y = p.y + b * F;
    T *y1 = p.ystage[6] + b * F;
    constexpr bool REG = FC > 0 && NS == 7;
    constexpr int FR = REG ? FC : 1;
    T k_reg[NS][FR], y_reg[FR], y1_reg[FR];
    if (REG) {
#pragma unroll
        for (int f = 0; f < FR; ++f) {
            y_reg[f] = y[f], y1_reg[f] = y1[f];
#pragma unroll
            for (int s = 0; s < NS; ++s) k_reg[s][f] = p.k[s][b * F + f];
        }
    }
    auto K = [&](int s, int f) -> T { return REG ? k_reg[s][REG ? f : 0] : p.k[s][b * F + f]; };
    auto Y = [&](int f) -> T { return REG ? y_reg[REG ? f : 0] : y[f]; };
    auto Y1 = [&](int f) -> T { return REG ? y1_reg[REG ? f : 0] : y1[f]; };

    // ---- the step's result where it is not the input of the last stage (heun.py, euler.py; runge_kutta.py:265-269) ----
    if (METHOD == TODE_HEUN) {
        for (int f = 0; f < F; ++f) {
            T sum = 0;
#pragma unroll
            for (int s = 0; s < NS; ++s) {
                const T ps = h * (T)HeunTab::b[s], ks = p.k[s][b * F + f];
                if (fused)
                    sum = fma_(ps, ks, sum);
                else {
                    const T pk = ps * ks;
                    sum = sum + pk;
                }
            }
            y1[f] = y[f] + sum;
        }
    } else if (METHOD == TODE_EULER) {
        for (int f = 0; f < F; ++f) y1[f] = fma_(h, p.k[0][b * F + f], y[f]);
    }

    // ---- error estimate and error ratio (not looked at by the fixed-step controller) ----
    T acc = 0;
#pragma unroll
    for (int f = 0; ESTIMATE && CTRL != 2 && f < F; ++f) {
        T err = 0;
#pragma unroll
        for (int s = 0; s < NS; ++s) {
            T ps = h * (T)Tab::b_err[s];
            T ks = K(s, f);
            if (fused)
                err = fma_(ps, ks, err);
            else {
                T pk = ps * ks;
                err = err + pk;
            }
        }
        T m = tmax(abs_(Y(f)), abs_(Y1(f)));
        T eb = fma_(cp.rtol, m, cp.atol);
        T x = (abs_(err) / eb) / sf;
        if (F <= 3)
            acc = fma_(x, x, acc);
        else {
            T sq = x * x;
            acc = acc + sq;
        }
    }
    const T ratio = tmax(sqrt_(acc), (T)1e-38);
    const bool accept = CTRL == 2 || !ESTIMATE || ratio < (T)1;

    // ---- step size proposal ----
    const T prev = p.ratio_prev[b], pprev = p.ratio_pprev[b];
    TT dt_next;
    int status = 0;
    if (CTRL == 2) {
        dt_next = p.fixed_dt[b];
    } else if (!ESTIMATE) {
        dt_next = dt;  // (step_size_controllers.py:382-391, 727-736: accepted, step size unchanged, no status)
    } else {
        dt_next = dt * (TT)dt_factor<T, (CTRL == 2 ? 0 : CTRL)>(cp, ratio, prev, pprev);
        status = limit_step<TT, T>(cp, p.dt_min, p.dt_max, ratio, dt_next);
    }

    const bool running = p.running[b] != 0;
    const bool move = accept && running;
    const TT t_new = move ? (t0 + dt) : t0;
    const bool running_new = fwd ? (t_new < te) : (t_new > te);
    const int n_steps = p.n_steps[b] + (running ? 1 : 0);
    p.n_steps[b] = n_steps;
    if (move) p.n_accepted[b] += 1;
    if (p.max_steps != INT_MAX && n_steps >= p.max_steps) status = TODE_REACHED_MAX_STEPS;
    if (status == 0 && n_steps >= TODE_HARD_STEP_LIMIT) status = TODE_GENERAL_ERROR;
    p.status[b] = status;

    // ---- dense output with the interpolant of the attempted step ----
    if (E > 0) {
        const TT *tev = p.t_eval + b * E;
        T *ys = p.ys + b * (long long)E * F;
        uint8_t *pend = p.pending + b * (long long)E;
        const bool mono = p.monotone[b] != 0;
        int cursor = p.cursor[b];
        int e = mono ? cursor : 0;
        T q_reg[FR][5][1];  // (REG: every feature's interpolant, built when the first point turns out to have been passed)
        bool built = false;
        for (; e < E; ++e) {
            if (!pend[e]) continue;
            const TT te_e = tev[e];
            const bool passed = fwd ? t_new >= te_e : t_new <= te_e;
            if (!passed) {
                if (mono) break;
                continue;
            }
            if (REG) {
                if (!built) {
#pragma unroll
                    for (int f = 0; f < FR; ++f) {
                        T ks[7];
#pragma unroll
                        for (int s = 0; s < 7; ++s) ks[s] = K(s, f);
                        quartic_elem<T, (METHOD == 1 ? 1 : 0)>(h, Y(f), Y1(f), ks, fused, q_reg[f]);
                    }
                    built = true;
                }
                const T x = (T)unit_time<TT>(te_e, t0, t0 + dt);
#pragma unroll
                for (int f = 0; f < FR; ++f) ys[(long long)e * F + f] = quartic_at<T>(q_reg[f], x);
            } else {
                for (int f = 0; f < F; ++f) {
                    T ks[7] = {};
#pragma unroll
                    for (int s = 0; s < NS; ++s) ks[s] = p.k[s][b * F + f];
                    ys[(long long)e * F + f] = dense_value<TT, T, METHOD>(t0, dt, y[f], y1[f], ks, fused, te_e);
                }
            }
            pend[e] = 0;
        }
        while (cursor < E && !pend[cursor]) ++cursor;  // first still-pending point
        p.cursor[b] = cursor;
    } else {
        // no evaluation points: the end-point value of the loop's last interpolant
        // (adjoints.py:295-309); rewritten every iteration, the last one stays
#pragma unroll
        for (int f = 0; f < F; ++f) {
            T ks[7] = {};
#pragma unroll
            for (int s = 0; s < NS; ++s) ks[s] = K(s, f);
            p.ys[b * F + f] = dense_value<TT, T, METHOD>(t0, dt, Y(f), Y1(f), ks, fused, te);
        }
    }

    // ---- state update ----
    if (move) {
#pragma unroll
        for (int f = 0; f < F; ++f) {
            p.y[b * F + f] = Y1(f);
            if (NS == 7) p.k0[b * F + f] = K(6, f);  // (first same as last: Dopri5 and Tsit5 only)
        }
    }
    p.t[b] = t_new;
    const TT tlo = tmin(ts, te), thi = tmax(te, ts);
    const TT dtn = running_new ? dt_next : dt;
    p.dt[b] = tclamp(dtn, tlo - t_new, thi - t_new);
    if (CTRL == 1 && ESTIMATE && running_new && accept) {
        p.ratio_pprev[b] = prev;
        p.ratio_prev[b] = ratio;
    }
    p.running[b] = running_new ? 1 : 0;
    if (running_new) p.flags[TODE_STEP_FLAG_ANY_RUNNING] = 1;
    if (status != 0) p.flags[TODE_STEP_FLAG_ANY_FAILURE] = 1;
}

// ------------------------------------------------------------------------------------------
// The same three kernels for long rows: one wavefront per sample, four samples per workgroup.
// Per-sample scalars are computed by every lane; lane 0 stores them.
// ------------------------------------------------------------------------------------------

template <typename TT, typename T> __global__ void __launch_bounds__(256) init_a_wave_kernel(const StepParams<TT, T> p) {
    const long long b = (long long)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (b >= p.batch) return;
    const int F = p.F, lane = threadIdx.x & 63;
    const CtrlParams<T> &cp = p.cp;
    const T *y0 = p.y0 + b * F, *f0 = p.k[0] + b * F;
    const T d0 = wave_row_norm<T, TODE_NORM_RMS>(F, [&](int f) { return y0[f] * inv_scale(cp.atol, cp.rtol, y0[f]); });
    const T d1 = wave_row_norm<T, TODE_NORM_RMS>(F, [&](int f) { return f0[f] * inv_scale(cp.atol, cp.rtol, y0[f]); });
    const TT ts = p.t_start[b], te = p.t_end[b];
    const bool fwd = te > ts;
    T h0 = (d0 < (T)1e-5 || d1 < (T)1e-5) ? (T)1e-6 : ((T)0.01 * d0) / d1;
    h0 = tmin(h0, (T)abs_(te - ts));
    const T dh = (fwd ? (T)1 : (T)-1) * h0;
    T *y1 = p.ystage[1] + b * F;
    for (int f = lane; f < F; f += 64) y1[f] = fma_(dh, f0[f], y0[f]);
    if (lane == 0) {
        p.tnode[b] = fma_(fwd ? (TT)1 : (TT)-1, (TT)h0, ts);
        p.ratio_prev[b] = h0;
    }
}

template <typename TT, typename T, int CTRL, bool FROM_F1>
__global__ void __launch_bounds__(256) init_b_wave_kernel(const StepParams<TT, T> p, const TT *dt0) {
    const long long b = (long long)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (b >= p.batch) return;
    const int F = p.F, E = p.E, lane = threadIdx.x & 63;
    const CtrlParams<T> &cp = p.cp;
    const T *y0 = p.y0 + b * F, *f0 = p.k[0] + b * F;
    const TT ts = p.t_start[b], te = p.t_end[b];
    const bool fwd = te > ts;
    const T dir = fwd ? (T)1 : (T)-1;
    TT dt;
    if (FROM_F1) {
        const T *f1 = p.k[1] + b * F;
        const T d1 = wave_row_norm<T, TODE_NORM_RMS>(F, [&](int f) { return f0[f] * inv_scale(cp.atol, cp.rtol, y0[f]); });
        const T d2n = wave_row_norm<T, TODE_NORM_RMS>(F, [&](int f) {
            const T df = f1[f] - f0[f];
            return df * inv_scale(cp.atol, cp.rtol, y0[f]);
        });
        dt = (TT)initial_finish<T>(CTRL == 1 ? TODE_CTRL_PID : TODE_CTRL_INTEGRAL, p.inv_order, dir, p.ratio_prev[b], d1, d2n);
    } else {
        dt = dt0[b];
    }
    for (int f = lane; f < F; f += 64) {
        p.y[b * F + f] = y0[f];
        if (p.carry) p.k0[b * F + f] = f0[f];
    }
    bool ordered = true;
    int cursor = 0;
    if (E > 0) {
        const TT *tev = p.t_eval + b * E;
        for (int e = lane; e < E; e += 64) {
            if (e > 0 && !(fwd ? tev[e] >= tev[e - 1] : tev[e] <= tev[e - 1])) ordered = false;
            p.pending[b * E + e] = (e == 0 && tev[0] == ts) ? 0 : 1;
        }
        if (tev[0] == ts) {
            for (int f = lane; f < F; f += 64) p.ys[(b * E) * F + f] = y0[f];
            cursor = 1;
        }
    }
    ordered = !__any(!ordered);
    if (lane == 0) {
        const TT tlo = tmin(ts, te), thi = tmax(te, ts);
        p.t[b] = ts;
        p.dt[b] = tclamp(dt, tlo - ts, thi - ts);
        p.ratio_prev[b] = (T)1;
        p.ratio_pprev[b] = (T)1;
        p.running[b] = 1;
        p.n_steps[b] = 0;
        p.n_accepted[b] = 0;
        p.status[b] = 0;
        p.cursor[b] = cursor;
        p.monotone[b] = ordered ? 1 : 0;
    }
}

// The row norm of wave_row_norm with the four wavefronts of a workgroup sharing one row: wavefront w takes the chunks
// w, w + 4, ..., the chunk sums meet in LDS and every thread adds them in the order of the chunks -- the same sums in
// the same order, so the same bits as one wavefront walking the whole row.
constexpr int TODE_BLOCK_ROW_CHUNKS = 1024;  // rows of up to 262144 values
template <typename T, typename Load> __device__ __forceinline__ T block_row_rms(int F, T *chunk_sums, Load load) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const T sf = (T)__builtin_sqrt((double)F);
    const int chunks = (F + 255) / 256;
    for (int c = wave; c < chunks; c += 4) {
        T part = 0;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int f = c * 256 + 4 * lane + j;
            if (f < F) {
                const T x = load(f) / sf;
                part = fma_(x, x, part);
            }
        }
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) part = part + __shfl_xor(part, off);
        if (lane == 0) chunk_sums[c] = part;
    }
    __syncthreads();
    T total = 0;
    for (int c = 0; c < chunks; ++c) total = total + chunk_sums[c];
    return sqrt_(total);
}

// BLOCK false: one wavefront per sample, four samples per workgroup.  BLOCK true (long rows): the workgroup's four
// wavefronts share one sample -- each walks every fourth group of 256 features, all four take the same decisions from
// the same norm, thread 0 stores the sample's scalars.
template <typename TT, typename T, int METHOD, int CTRL, bool BLOCK = false> __global__ void __launch_bounds__(256) finish_wave_kernel(const StepParams<TT, T> p) {
    using Tab = typename TabOf<METHOD>::type;
    constexpr int NS = stages_of(METHOD);
    constexpr bool ESTIMATE = METHOD != TODE_EULER;
    __shared__ T chunk_sums[BLOCK ? TODE_BLOCK_ROW_CHUNKS : 1];
    if (p.flags[TODE_STEP_FLAG_STOPPED]) return;
    const long long b = BLOCK ? (long long)blockIdx.x : (long long)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (b >= p.batch) return;
    const int F = p.F, E = p.E, lane = threadIdx.x & 63;
    // a thread's features: `first`, `first + stride`, ...; the dense output walks groups of 256 features, `group_first`
    // and every `group_stride`-th after it; `scalar_thread` stores what the sample has one of
    const int first = BLOCK ? (int)threadIdx.x : lane, stride = BLOCK ? 256 : 64;
    const int group_first = BLOCK ? 256 * (int)(threadIdx.x >> 6) : 0, group_stride = BLOCK ? 1024 : 256;
    const bool scalar_thread = BLOCK ? threadIdx.x == 0 : lane == 0;
    const CtrlParams<T> &cp = p.cp;
    const bool fused = F >= 58;
    const TT t0 = p.t[b], dt = p.dt[b];
    const T h = (T)dt;
    const TT ts = p.t_start[b], te = p.t_end[b];
    const bool fwd = te > ts;
    const T *y = p.y + b * F;
    // The step's result: Dopri5 and Tsit5 hand it over as the input of their last stage; for Heun and Euler it is
    // formed here (heun.py, euler.py; runge_kutta.py:265-269), by whichever lane needs it and as often as it does,
    // so that no lane reads what another lane of the wavefront has just written.
    auto y1 = [&](int f) -> T {
        if (METHOD == TODE_EULER) return fma_(h, p.k[0][b * F + f], y[f]);
        if (METHOD == TODE_HEUN) {
            T sum = 0;
#pragma unroll
            for (int s = 0; s < NS; ++s) {
                const T ps = h * (T)HeunTab::b[s], ks = p.k[s][b * F + f];
                if (fused)
                    sum = fma_(ps, ks, sum);
                else {
                    const T pk = ps * ks;
                    sum = sum + pk;
                }
            }
            return y[f] + sum;
        }
        return p.ystage[6][b * F + f];
    };

    // ---- error estimate and error ratio (not looked at by the fixed-step controller) ----
    auto scaled_error = [&](int f) {
        T err = 0;
#pragma unroll
        for (int s = 0; s < NS; ++s) {
            const T ps = h * (T)Tab::b_err[s], ks = p.k[s][b * F + f];
            if (fused)
                err = fma_(ps, ks, err);
            else {
                const T pk = ps * ks;
                err = err + pk;
            }
        }
        const T m = tmax(abs_(y[f]), abs_(y1(f)));
        return abs_(err) / fma_(cp.rtol, m, cp.atol);
    };
    const T norm = (CTRL == 2 || !ESTIMATE) ? (T)0
                   : BLOCK                  ? block_row_rms<T>(F, chunk_sums, scaled_error)
                                            : wave_row_norm<T, TODE_NORM_RMS>(F, scaled_error);
    const T ratio = tmax(norm, (T)1e-38);
    const bool accept = CTRL == 2 || !ESTIMATE || ratio < (T)1;

    // ---- step size proposal ----
    const T prev = p.ratio_prev[b], pprev = p.ratio_pprev[b];
    TT dt_next;
    int status = 0;
    if (CTRL == 2) {
        dt_next = p.fixed_dt[b];
    } else if (!ESTIMATE) {
        dt_next = dt;  // (step_size_controllers.py:382-391, 727-736: accepted, step size unchanged, no status)
    } else {
        dt_next = dt * (TT)dt_factor<T, (CTRL == 2 ? 0 : CTRL)>(cp, ratio, prev, pprev);
        status = limit_step<TT, T>(cp, p.dt_min, p.dt_max, ratio, dt_next);
    }

    const bool running = p.running[b] != 0;
    const bool move = accept && running;
    const TT t_new = move ? (t0 + dt) : t0;
    const bool running_new = fwd ? (t_new < te) : (t_new > te);
    const int n_steps = p.n_steps[b] + (running ? 1 : 0);
    if (p.max_steps != INT_MAX && n_steps >= p.max_steps) status = TODE_REACHED_MAX_STEPS;
    if (status == 0 && n_steps >= TODE_HARD_STEP_LIMIT) status = TODE_GENERAL_ERROR;

    // ---- dense output with the interpolant of the attempted step: the quartic of a feature is
    // built once, when the first evaluation point turns out to have been passed ----
    if (E > 0) {
        const TT *tev = p.t_eval + b * E;
        T *ys = p.ys + b * (long long)E * F;
        uint8_t *pend = p.pending + b * (long long)E;
        const bool mono = p.monotone[b] != 0;
        const int cursor = p.cursor[b];
        // The pending points are looked at 64 at a time, one per lane: which of them the step has passed (for a
        // monotone row: those in front of the first one it has not) comes out as a mask that is the same for the whole
        // wavefront, and each lane keeps its point's position in the step.  Then the row is walked once per such group
        // of points -- 256 features at a time, so that the loads of four features are in flight together -- and every
        // feature's interpolant is evaluated at the points of the mask, their positions read from the lanes that hold
        // them.  Nothing in the inner loops waits for memory but the row itself.
        for (int e0 = mono ? cursor : 0; e0 < E; e0 += 64) {
            const int e = e0 + lane;
            const bool valid = e < E;
            const bool pending = valid && pend[e] != 0;
            const TT te_e = valid ? tev[e] : t0;
            const bool passed = fwd ? t_new >= te_e : t_new <= te_e;
            unsigned long long take = __ballot(pending && passed);
            const unsigned long long blocked = mono ? __ballot(pending && !passed) : 0ull;
            if (blocked) take &= (blocked & (~blocked + 1ull)) - 1ull;  // (only the points in front of the first one not passed)
            if (take) {
                const T x = (T)unit_time<TT>(te_e, t0, t0 + dt);
                for (int f0 = group_first; f0 < F; f0 += group_stride) {
                    T q[4][5][1], ks[4][7] = {}, y0f[4] = {}, y1f[4] = {};
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        const int f = f0 + 64 * j + lane;
                        if (f < F) {
#pragma unroll
                            for (int s = 0; s < NS; ++s) ks[j][s] = p.k[s][b * F + f];
                            y0f[j] = y[f], y1f[j] = y1(f);
                        }
                    }
                    if (NS == 7) {
#pragma unroll
                        for (int j = 0; j < 4; ++j) quartic_elem<T, (METHOD == 1 ? 1 : 0)>(h, y0f[j], y1f[j], ks[j], fused, q[j]);
                    }
                    for (unsigned long long m = take; m; m &= m - 1ull) {
                        const int i = __builtin_ctzll(m);
                        T *row = ys + (long long)(e0 + i) * F + f0 + lane;
                        const T xi = wave_read(x, i);
                        const TT ti = wave_read(te_e, i);
#pragma unroll
                        for (int j = 0; j < 4; ++j) {
                            if (f0 + 64 * j + lane < F) {
                                if (NS == 7)
                                    row[64 * j] = quartic_at<T>(q[j], xi);
                                else  // (Hermite cubic / linear interpolant: cheap enough to form per point)
                                    row[64 * j] = dense_value<TT, T, METHOD>(t0, dt, y0f[j], y1f[j], ks[j], fused, ti);
                            }
                        }
                    }
                }
            }
            if (blocked) break;
        }
        // (every lane has finished reading the pending marks: a wavefront runs in lock step, a workgroup waits here;
        // the marks are then brought up to date by one wavefront)
        if (BLOCK) __syncthreads();
        if (!BLOCK || threadIdx.x < 64) {
            int first_pending = E;
            for (int e = lane; e < E; e += 64) {
                if (!pend[e]) continue;
                const TT te_e = tev[e];
                const bool passed = fwd ? t_new >= te_e : t_new <= te_e;
                const bool taken = passed && (!mono || e >= cursor);
                if (taken) pend[e] = 0;
                else first_pending = min(first_pending, e);
            }
#pragma unroll
            for (int off = 32; off > 0; off >>= 1) first_pending = min(first_pending, __shfl_xor(first_pending, off));
            if (lane == 0) p.cursor[b] = first_pending;
        }
    } else {
        for (int f = first; f < F; f += stride) {
            T ks[7] = {};
#pragma unroll
            for (int s = 0; s < NS; ++s) ks[s] = p.k[s][b * F + f];
            p.ys[b * F + f] = dense_value<TT, T, METHOD>(t0, dt, y[f], y1(f), ks, fused, te);
        }
    }

    // ---- state update ----
    if (BLOCK) __syncthreads();  // (no thread of the workgroup still reads what is overwritten now)
    if (move) {
        for (int f = first; f < F; f += stride) {
            const T moved = y1(f);  // (read before the write: for Heun and Euler y1 is formed from y)
            p.y[b * F + f] = moved;
            if (NS == 7) p.k0[b * F + f] = p.k[6][b * F + f];  // (first same as last: Dopri5 and Tsit5 only)
        }
    }
    if (scalar_thread) {
        p.n_steps[b] = n_steps;
        if (move) p.n_accepted[b] += 1;
        p.status[b] = status;
        p.t[b] = t_new;
        const TT tlo = tmin(ts, te), thi = tmax(te, ts);
        const TT dtn = running_new ? dt_next : dt;
        p.dt[b] = tclamp(dtn, tlo - t_new, thi - t_new);
        if (CTRL == 1 && ESTIMATE && running_new && accept) {
            p.ratio_pprev[b] = prev;
            p.ratio_prev[b] = ratio;
        }
        p.running[b] = running_new ? 1 : 0;
        if (running_new) p.flags[TODE_STEP_FLAG_ANY_RUNNING] = 1;
        if (status != 0) p.flags[TODE_STEP_FLAG_ANY_FAILURE] = 1;
    }
}

// One thread: closes the iteration.  The loop goes on iff some sample is still running and
// every status is SUCCESS (adjoints.py:186-190).
static __global__ void loop_control_kernel(int32_t *flags, int32_t *host_flags) {
    if (threadIdx.x != 0 || flags[TODE_STEP_FLAG_STOPPED]) return;
    const int iterations = flags[TODE_STEP_FLAG_ITERATIONS] + 1;
    const int stopped = (!flags[TODE_STEP_FLAG_ANY_RUNNING] || flags[TODE_STEP_FLAG_ANY_FAILURE]) ? 1 : 0;
    flags[TODE_STEP_FLAG_ITERATIONS] = iterations;
    flags[TODE_STEP_FLAG_STOPPED] = stopped;
    flags[TODE_STEP_FLAG_ANY_RUNNING] = 0;
    if (host_flags) {  // the count first: a host that sees "stopped" also sees the final count
        __hip_atomic_store(&host_flags[1], iterations, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
        __hip_atomic_store(&host_flags[0], stopped, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_SYSTEM);
    }
}

static __global__ void step_flags_init_kernel(int32_t *flags, int32_t *host_flags) {
    if (threadIdx.x < TODE_STEP_FLAG_WORDS) flags[threadIdx.x] = 0;
    if (host_flags && threadIdx.x < 2) __hip_atomic_store(&host_flags[threadIdx.x], 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
}

// int32 device state -> the reference's int64 stats (adjoints.py:267-292)
static __global__ void step_stats_kernel(long long batch, const int32_t *n_steps, const int32_t *n_accepted, const int32_t *cursor,
                                         const int32_t *status, const int32_t *monotone, const uint8_t *pending, int n_eval,
                                         int64_t *o_steps, int64_t *o_acc, int64_t *o_init, int64_t *o_status) {
    const long long b = (long long)blockIdx.x * 256 + threadIdx.x;
    if (b >= batch) return;
    o_steps[b] = n_steps[b];
    o_acc[b] = n_accepted[b];
    // (a monotone row's marks are sorted: the search of the reference finds the cursor)
    o_init[b] = n_eval <= 0 ? 1 : (monotone[b] ? cursor[b] : searchsorted_first_pending(pending + b * n_eval, n_eval));
    o_status[b] = status[b];
}

template <typename TT, typename T> static StepParams<TT, T> make_step_params(const tode_step_state &s, const tode_controller &c) {
    StepParams<TT, T> p;
    p.y0 = (const T *)s.y0;
    p.t_start = (const TT *)s.t_start;
    p.t_end = (const TT *)s.t_end;
    p.t_eval = (const TT *)s.t_eval;
    p.batch = s.batch;
    p.F = s.n_features;
    p.E = s.n_eval;
    p.max_steps = (s.max_steps < 0 || s.max_steps >= INT_MAX) ? INT_MAX : (int)s.max_steps;
    p.t = (TT *)s.t;
    p.dt = (TT *)s.dt;
    p.y = (T *)s.y;
    p.k0 = (T *)s.k0;
    p.ratio_prev = (T *)s.ratio_prev;
    p.ratio_pprev = (T *)s.ratio_pprev;
    p.running = s.running;
    p.cursor = s.cursor;
    p.n_steps = s.n_steps;
    p.n_accepted = s.n_accepted;
    p.status = s.status;
    p.monotone = s.monotone;
    p.pending = s.pending;
    p.ys = (T *)s.ys;
    p.flags = s.flags;
    for (int i = 0; i < 7; ++i) {
        p.ystage[i] = (T *)s.ystage[i];
        p.k[i] = (const T *)s.k[i];
    }
    p.tnode = (TT *)s.tnode;
    p.cp = make_ctrl<T>(c, order_of(s.method));
    p.dt_min = (TT)c.dt_min;
    p.dt_max = (TT)c.dt_max;
    p.fixed_dt = (const TT *)s.fixed_dt;
    p.inv_order = 1.0 / order_of(s.method);
    p.carry = s.method <= TODE_TSIT5;
    return p;
}

static int check_state(const tode_step_state *s, const tode_controller *c) {
    if (!s || !c) return fail(TODE_E_INVALID, "null argument struct");
    if (s->batch < 0 || s->n_features <= 0 || s->n_eval < 0) return fail(TODE_E_INVALID, "bad sizes");
    if (s->dtype != TODE_F32 && s->dtype != TODE_F64) return fail(TODE_E_INVALID, "unknown dtype %d", s->dtype);
    if (s->time_dtype != TODE_F32 && s->time_dtype != TODE_F64) return fail(TODE_E_INVALID, "unknown time dtype %d", s->time_dtype);
    if (s->method < TODE_DOPRI5 || s->method > TODE_EULER) return fail(TODE_E_INVALID, "unknown method %d", s->method);
    if (c->kind != TODE_CTRL_INTEGRAL && c->kind != TODE_CTRL_PID && c->kind != TODE_CTRL_FIXED)
        return fail(TODE_E_INVALID, "unknown controller kind %d", c->kind);
    if (c->kind == TODE_CTRL_FIXED && s->batch > 0 && !s->fixed_dt) return fail(TODE_E_INVALID, "the fixed-step controller needs fixed_dt");
    if (!s->flags) return fail(TODE_E_INVALID, "null flags pointer");
    if (s->batch > 0 && (!s->y0 || !s->t_start || !s->t_end || !s->t || !s->dt || !s->y || !s->k0 || !s->ratio_prev || !s->ratio_pprev ||
                         !s->running || !s->cursor || !s->n_steps || !s->n_accepted || !s->status || !s->monotone || !s->ys || !s->tnode))
        return fail(TODE_E_INVALID, "null state pointer");
    if (s->batch > 0 && s->n_eval > 0 && (!s->t_eval || !s->pending)) return fail(TODE_E_INVALID, "n_eval > 0 needs t_eval and pending");
    return TODE_OK;
}

// The statements given, with TT = the state's time type and T = its data type
#define TODE_DISPATCH_T(state, ...)                                        \
    do {                                                                   \
        if ((state)->time_dtype == TODE_F32 && (state)->dtype == TODE_F32) {  \
            using TT = float;                                              \
            using T = float;                                               \
            __VA_ARGS__;                                                   \
        } else if ((state)->time_dtype == TODE_F64 && (state)->dtype == TODE_F64) { \
            using TT = double;                                             \
            using T = double;                                              \
            __VA_ARGS__;                                                   \
        } else if ((state)->time_dtype == TODE_F64) {                      \
            using TT = double;                                             \
            using T = float;                                               \
            __VA_ARGS__;                                                   \
        } else {                                                           \
            using TT = float;                                              \
            using T = double;                                              \
            __VA_ARGS__;                                                   \
        }                                                                  \
    } while (0)

}  // namespace tode

extern "C" {

int tode_step_begin(const tode_step_state *s, const tode_controller *c, const void *dt0, int phase, void *stream) {
    using namespace tode;
    int rc = check_state(s, c);
    if (rc) return rc;
    hipStream_t st = (hipStream_t)stream;
    const bool wide = s->n_features >= 64;  // one wavefront per sample
    const unsigned blocks = wide ? (unsigned)((s->batch + 3) / 4) : (unsigned)((s->batch + 255) / 256);
    if (phase == 0) {
        hipLaunchKernelGGL(step_flags_init_kernel, dim3(1), dim3(64), 0, st, s->flags, s->host_flags);
        if (blocks == 0) return check_hip(hipGetLastError(), "tode_step_begin");
        if (dt0) {
            if (!s->k[0] && s->method <= TODE_TSIT5) return fail(TODE_E_INVALID, "k[0] (f at t_start) is null");
            TODE_DISPATCH_T(s, {
                auto p = make_step_params<TT, T>(*s, *c);
                if (wide)
                    hipLaunchKernelGGL((init_b_wave_kernel<TT, T, 0, false>), dim3(blocks), dim3(256), 0, st, p, (const TT *)dt0);  // (CTRL is unused here)
                else if (c->kind != TODE_CTRL_PID)  // (CTRL is unused here as well)
                    hipLaunchKernelGGL((init_b_kernel<TT, T, 0, false>), dim3(blocks), dim3(256), 0, st, p, (const TT *)dt0);
                else
                    hipLaunchKernelGGL((init_b_kernel<TT, T, 1, false>), dim3(blocks), dim3(256), 0, st, p, (const TT *)dt0);
            });
        } else {
            if (c->kind == TODE_CTRL_FIXED) return fail(TODE_E_INVALID, "the fixed-step controller needs dt0");
            if (!s->k[0] || !s->ystage[1]) return fail(TODE_E_INVALID, "k[0] or ystage[1] is null");
            TODE_DISPATCH_T(s, {
                auto p = make_step_params<TT, T>(*s, *c);
                if (wide)
                    hipLaunchKernelGGL((init_a_wave_kernel<TT, T>), dim3(blocks), dim3(256), 0, st, p);
                else
                    hipLaunchKernelGGL((init_a_kernel<TT, T>), dim3(blocks), dim3(256), 0, st, p);
            });
        }
    } else {
        if (c->kind == TODE_CTRL_FIXED) return fail(TODE_E_INVALID, "the fixed-step controller has no second phase");
        if (blocks == 0) return TODE_OK;
        if (!s->k[0] || !s->k[1]) return fail(TODE_E_INVALID, "k[0] or k[1] is null");
        TODE_DISPATCH_T(s, {
            auto p = make_step_params<TT, T>(*s, *c);
            if (wide && c->kind == TODE_CTRL_INTEGRAL)
                hipLaunchKernelGGL((init_b_wave_kernel<TT, T, 0, true>), dim3(blocks), dim3(256), 0, st, p, (const TT *)nullptr);
            else if (wide)
                hipLaunchKernelGGL((init_b_wave_kernel<TT, T, 1, true>), dim3(blocks), dim3(256), 0, st, p, (const TT *)nullptr);
            else if (c->kind == TODE_CTRL_INTEGRAL)
                hipLaunchKernelGGL((init_b_kernel<TT, T, 0, true>), dim3(blocks), dim3(256), 0, st, p, (const TT *)nullptr);
            else
                hipLaunchKernelGGL((init_b_kernel<TT, T, 1, true>), dim3(blocks), dim3(256), 0, st, p, (const TT *)nullptr);
        });
    }
    return check_hip(hipGetLastError(), "tode_step_begin");
}

int tode_step_stage(const tode_step_state *s, const tode_controller *c, int stage, void *stream) {
    using namespace tode;
    int rc = check_state(s, c);
    if (rc) return rc;
    const int last_stage = stages_of(s->method) - 1;
    if (stage < 1 || stage > last_stage) return fail(TODE_E_INVALID, "stage must be 1..%d for this method, got %d", last_stage, stage);
    for (int j = 0; j < stage; ++j)
        if (s->batch > 0 && !s->k[j]) return fail(TODE_E_INVALID, "k[%d] is null", j);
    if (s->batch > 0 && !s->ystage[stage]) return fail(TODE_E_INVALID, "ystage[%d] is null", stage);
    const long long n = s->batch * s->n_features;
    if (n == 0) return TODE_OK;
    hipStream_t st = (hipStream_t)stream;
    const unsigned blocks = (unsigned)((n + 255) / 256);
#define TODE_STAGE_CASE(M, S) \
    case S: hipLaunchKernelGGL((stage_kernel<TT, T, M, S>), dim3(blocks), dim3(256), 0, st, p); break;
#define TODE_STAGE_SWITCH(M)                                                                  \
    switch (stage) {                                                                          \
        TODE_STAGE_CASE(M, 1) TODE_STAGE_CASE(M, 2) TODE_STAGE_CASE(M, 3) TODE_STAGE_CASE(M, 4) \
        TODE_STAGE_CASE(M, 5) TODE_STAGE_CASE(M, 6)                                           \
    }
    TODE_DISPATCH_T(s, {
        auto p = make_step_params<TT, T>(*s, *c);
        if (s->method == TODE_HEUN) {
            hipLaunchKernelGGL((stage_kernel<TT, T, 2, 1>), dim3(blocks), dim3(256), 0, st, p);
        } else if (s->method == TODE_TSIT5) {
            TODE_STAGE_SWITCH(1)
        } else {
            TODE_STAGE_SWITCH(0)
        }
    });
#undef TODE_STAGE_SWITCH
#undef TODE_STAGE_CASE
    return check_hip(hipGetLastError(), "tode_step_stage");
}

#define TODE_FINISH(KERNEL, M, C) hipLaunchKernelGGL((KERNEL<TT, T, M, C>), dim3(blocks), dim3(256), 0, st, p)
// (rows of 2, 3 or 4 values with Dopri5 / Tsit5: the thread-per-sample kernel with the row length a template argument)
#define TODE_FINISH_SHORT(M, FCV)                                                                                          \
    do {                                                                                                                   \
        if (c->kind == TODE_CTRL_PID) hipLaunchKernelGGL((finish_kernel<TT, T, M, 1, FCV>), dim3(blocks), dim3(256), 0, st, p);        \
        else if (c->kind == TODE_CTRL_FIXED) hipLaunchKernelGGL((finish_kernel<TT, T, M, 2, FCV>), dim3(blocks), dim3(256), 0, st, p); \
        else hipLaunchKernelGGL((finish_kernel<TT, T, M, 0, FCV>), dim3(blocks), dim3(256), 0, st, p);                                 \
    } while (0)
// (long rows: the workgroup-per-sample form of the wavefront kernel)
#define TODE_FINISH_ROWS(M)                                                                                                        \
    do {                                                                                                                           \
        if (c->kind == TODE_CTRL_PID) hipLaunchKernelGGL((finish_wave_kernel<TT, T, M, 1, true>), dim3(blocks), dim3(256), 0, st, p);        \
        else if (c->kind == TODE_CTRL_FIXED) hipLaunchKernelGGL((finish_wave_kernel<TT, T, M, 2, true>), dim3(blocks), dim3(256), 0, st, p); \
        else hipLaunchKernelGGL((finish_wave_kernel<TT, T, M, 0, true>), dim3(blocks), dim3(256), 0, st, p);                                 \
    } while (0)
#define TODE_FINISH_CTRL(KERNEL, M)                                     \
    do {                                                                \
        if (c->kind == TODE_CTRL_PID) TODE_FINISH(KERNEL, M, 1);        \
        else if (c->kind == TODE_CTRL_FIXED) TODE_FINISH(KERNEL, M, 2); \
        else TODE_FINISH(KERNEL, M, 0);                                 \
    } while (0)

int tode_step_finish(const tode_step_state *s, const tode_controller *c, void *stream) {
    using namespace tode;
    int rc = check_state(s, c);
    if (rc) return rc;
    hipStream_t st = (hipStream_t)stream;
    const bool wide = s->n_features >= 64;
    // rows of 1024 values and more: a workgroup per sample instead of a wavefront (more loads and stores in flight per
    // sample; the same sums in the same order)
    const bool rows = s->n_features >= 1024 && (s->n_features + 255) / 256 <= TODE_BLOCK_ROW_CHUNKS && s->batch <= 0x7fffffff;
    const unsigned blocks = rows ? (unsigned)s->batch : wide ? (unsigned)((s->batch + 3) / 4) : (unsigned)((s->batch + 255) / 256);
    if (blocks > 0) {
        for (int j = 0; j < stages_of(s->method); ++j)
            if (!s->k[j]) return fail(TODE_E_INVALID, "k[%d] is null", j);
        if (!s->ystage[6] && !(wide && s->method > TODE_TSIT5)) return fail(TODE_E_INVALID, "ystage[6] is null");
        TODE_DISPATCH_T(s, {
            auto p = make_step_params<TT, T>(*s, *c);
            const bool tsit5 = s->method == TODE_TSIT5;
            if (rows) {
                if (s->method == TODE_HEUN) TODE_FINISH_ROWS(2);
                else if (s->method == TODE_EULER) TODE_FINISH_ROWS(3);
                else if (tsit5) TODE_FINISH_ROWS(1);
                else TODE_FINISH_ROWS(0);
            } else if (s->method == TODE_HEUN) {
                if (wide) TODE_FINISH_CTRL(finish_wave_kernel, 2);
                else TODE_FINISH_CTRL(finish_kernel, 2);
            } else if (s->method == TODE_EULER) {
                if (wide) TODE_FINISH_CTRL(finish_wave_kernel, 3);
                else TODE_FINISH_CTRL(finish_kernel, 3);
            } else if (wide) {
                if (tsit5) TODE_FINISH_CTRL(finish_wave_kernel, 1);
                else TODE_FINISH_CTRL(finish_wave_kernel, 0);
            } else if (s->n_features == 2) {
                if (tsit5) TODE_FINISH_SHORT(1, 2);
                else TODE_FINISH_SHORT(0, 2);
            } else if (s->n_features == 3) {
                if (tsit5) TODE_FINISH_SHORT(1, 3);
                else TODE_FINISH_SHORT(0, 3);
            } else if (s->n_features == 4) {
                if (tsit5) TODE_FINISH_SHORT(1, 4);
                else TODE_FINISH_SHORT(0, 4);
            } else {
                if (tsit5) TODE_FINISH_CTRL(finish_kernel, 1);
                else TODE_FINISH_CTRL(finish_kernel, 0);
            }
        });
    }
    hipLaunchKernelGGL(loop_control_kernel, dim3(1), dim3(64), 0, st, s->flags, s->host_flags);
    return check_hip(hipGetLastError(), "tode_step_finish");
}
#undef TODE_FINISH_CTRL
#undef TODE_FINISH

int tode_step_stats(const tode_step_state *s, int64_t *n_steps, int64_t *n_accepted, int64_t *n_initialized, int64_t *status, void *stream) {
    using namespace tode;
    if (!s) return fail(TODE_E_INVALID, "null state");
    if (s->batch == 0) return TODE_OK;
    if (!n_steps || !n_accepted || !n_initialized || !status || !s->n_steps || !s->n_accepted || !s->cursor || !s->status || !s->monotone ||
        (s->n_eval > 0 && !s->pending))
        return fail(TODE_E_INVALID, "null pointer");
    const unsigned blocks = (unsigned)((s->batch + 255) / 256);
    hipLaunchKernelGGL(step_stats_kernel, dim3(blocks), dim3(256), 0, (hipStream_t)stream, (long long)s->batch, s->n_steps, s->n_accepted,
                       s->cursor, s->status, s->monotone, s->pending, s->n_eval, n_steps, n_accepted, n_initialized, status);
    return check_hip(hipGetLastError(), "tode_step_stats");
}

}  // extern "C"

namespace tode {

template <typename TT, typename T> static AdjointParams<TT, T> make_adjoint_params(const tode_step_adjoint &a, const tode_controller &c) {
    AdjointParams<TT, T> p;
    p.batch = a.batch;
    p.F = a.n_features;
    p.E = a.n_eval;
    p.iteration = a.iteration;
    p.through_control = a.through_control;
    p.end_point = a.end_point;
    p.t_start = (const TT *)a.t_start, p.t_end = (const TT *)a.t_end, p.t_eval = (const TT *)a.t_eval;
    p.t = (const TT *)a.t, p.dt = (const TT *)a.dt, p.fixed_dt = (const TT *)a.fixed_dt;
    p.y = (const T *)a.y, p.y1 = (const T *)a.y1, p.prev = (const T *)a.ratio_prev, p.pprev = (const T *)a.ratio_pprev;
    p.grad_ys = (const T *)a.grad_ys;
    for (int s = 0; s < 7; ++s) p.k[s] = (const T *)a.k[s], p.g_k[s] = (T *)a.g_k[s];
    p.running = a.running, p.moved = a.moved, p.running_next = a.running_next, p.hit_iteration = a.hit_iteration;
    p.a_t = (const TT *)a.a_t, p.a_dt = (const TT *)a.a_dt;
    p.a_y = (const T *)a.a_y, p.a_k0 = (const T *)a.a_k0, p.a_prev = (const T *)a.a_prev, p.a_pprev = (const T *)a.a_pprev;
    p.g_y = (T *)a.g_y, p.g_y1 = (T *)a.g_y1, p.g_prev = (T *)a.g_prev, p.g_pprev = (T *)a.g_pprev;
    p.g_t = (TT *)a.g_t, p.g_dt = (TT *)a.g_dt;
    p.g_t_start = (TT *)a.g_t_start, p.g_t_end = (TT *)a.g_t_end, p.g_t_eval = (TT *)a.g_t_eval, p.g_fixed_dt = (TT *)a.g_fixed_dt;
    p.cp = make_ctrl<T>(c);
    p.dt_min = (TT)c.dt_min;
    p.dt_max = (TT)c.dt_max;
    return p;
}

static int check_adjoint(const tode_step_adjoint *a, const tode_controller *c) {
    if (!a || !c) return fail(TODE_E_INVALID, "null argument struct");
    if (a->batch < 0 || a->n_features <= 0 || a->n_eval < 0) return fail(TODE_E_INVALID, "bad sizes");
    if (a->dtype != TODE_F32 && a->dtype != TODE_F64) return fail(TODE_E_INVALID, "unknown dtype %d", a->dtype);
    if (a->time_dtype != TODE_F32 && a->time_dtype != TODE_F64) return fail(TODE_E_INVALID, "unknown time dtype %d", a->time_dtype);
    if (a->method != TODE_DOPRI5 && a->method != TODE_TSIT5) return fail(TODE_E_INVALID, "unknown method %d", a->method);
    if (c->kind != TODE_CTRL_INTEGRAL && c->kind != TODE_CTRL_PID && c->kind != TODE_CTRL_FIXED)
        return fail(TODE_E_INVALID, "unknown controller kind %d", c->kind);
    if (a->batch == 0) return TODE_OK;
    if (!a->t_start || !a->t_end || !a->t || !a->dt || !a->y || !a->y1 || !a->ratio_prev || !a->ratio_pprev || !a->moved || !a->running_next ||
        !a->grad_ys || !a->g_y || !a->g_y1 || !a->g_t || !a->g_dt || !a->g_prev || !a->g_pprev)
        return fail(TODE_E_INVALID, "null pointer");
    for (int s = 0; s < 7; ++s)
        if (!a->k[s] || !a->g_k[s]) return fail(TODE_E_INVALID, "k[%d] or g_k[%d] is null", s, s);
    if (a->n_eval > 0 && (!a->t_eval || !a->hit_iteration)) return fail(TODE_E_INVALID, "n_eval > 0 needs t_eval and hit_iteration");
    if (c->kind == TODE_CTRL_FIXED && !a->fixed_dt) return fail(TODE_E_INVALID, "the fixed-step controller needs fixed_dt");
    return TODE_OK;
}

}  // namespace tode

extern "C" {

#define TODE_FINISH_BWD(M, C)                                                                                         \
    do {                                                                                                              \
        if (wide) hipLaunchKernelGGL((finish_backward_kernel<TT, T, M, C, true>), dim3(blocks), dim3(256), 0, st, p);  \
        else hipLaunchKernelGGL((finish_backward_kernel<TT, T, M, C, false>), dim3(blocks), dim3(256), 0, st, p);     \
    } while (0)
int tode_step_finish_backward(const tode_step_adjoint *a, const tode_controller *c, void *stream) {
    using namespace tode;
    int rc = check_adjoint(a, c);
    if (rc || a->batch == 0) return rc;
    hipStream_t st = (hipStream_t)stream;
    const bool wide = a->n_features >= 64;  // one wavefront per sample
    const unsigned blocks = wide ? (unsigned)((a->batch + 3) / 4) : (unsigned)((a->batch + 255) / 256);
    TODE_DISPATCH_T(a, {
        auto p = make_adjoint_params<TT, T>(*a, *c);
        if (a->method == TODE_TSIT5) {
            if (c->kind == TODE_CTRL_PID) TODE_FINISH_BWD(1, 1);
            else if (c->kind == TODE_CTRL_FIXED) TODE_FINISH_BWD(1, 2);
            else TODE_FINISH_BWD(1, 0);
        } else {
            if (c->kind == TODE_CTRL_PID) TODE_FINISH_BWD(0, 1);
            else if (c->kind == TODE_CTRL_FIXED) TODE_FINISH_BWD(0, 2);
            else TODE_FINISH_BWD(0, 0);
        }
    });
    return check_hip(hipGetLastError(), "tode_step_finish_backward");
}
#undef TODE_FINISH_BWD

int tode_step_stage_backward(const tode_step_adjoint *a, const tode_controller *c, int stage, const void *g_ystage, const void *g_tnode, void *stream) {
    using namespace tode;
    int rc = check_adjoint(a, c);
    if (rc || a->batch == 0) return rc;
    if (stage < 1 || stage > 6) return fail(TODE_E_INVALID, "stage must be 1..6, got %d", stage);
    if (!g_ystage) return fail(TODE_E_INVALID, "null g_ystage");
    hipStream_t st = (hipStream_t)stream;
    const bool wide = a->n_features >= 64;
    const unsigned blocks = wide ? (unsigned)((a->batch + 3) / 4) : (unsigned)((a->batch + 255) / 256);
#define TODE_STAGE_BWD(M, W) hipLaunchKernelGGL((stage_backward_kernel<TT, T, M, W>), dim3(blocks), dim3(256), 0, st, p, stage, (const T *)g_ystage, (const TT *)g_tnode)
    TODE_DISPATCH_T(a, {
        auto p = make_adjoint_params<TT, T>(*a, *c);
        if (a->method == TODE_TSIT5) {
            if (wide) TODE_STAGE_BWD(1, true);
            else TODE_STAGE_BWD(1, false);
        } else {
            if (wide) TODE_STAGE_BWD(0, true);
            else TODE_STAGE_BWD(0, false);
        }
    });
#undef TODE_STAGE_BWD
    return check_hip(hipGetLastError(), "tode_step_stage_backward");
}

}  // extern "C"
