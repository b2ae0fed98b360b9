// Reverse of one loop iteration, shared by the per-iteration kernels (tode_stepwise.hip) and the whole-sweep kernel
// (tode_backward.hip).
#pragma once
#include "tode_solve.h"

namespace tode {

// ==========================================================================================
// Reverse of one loop iteration: vector-Jacobian products of the stage and finish kernels
// ==========================================================================================
// The reference differentiates its loop by recording every torch operation (adjoints.py:33-40,
// 111-113, 145-147).  Here a solve that needs gradients keeps the loop state of every iteration,
// and the backward pass walks the iterations in reverse.  For one iteration it is handed the
// state before it, the stage values k_0..k_6 and y1 (recomputed by the forward kernels), the
// decisions taken (accepted, still running), and the cotangents of the state after it and of the
// evaluation points it wrote.  finish_backward_kernel pulls those through everything after the
// sixth stage -- dense output (tsit5.py:123-139, dopri5.py:53-60, interpolation.py:25-40,
// 138-175), state update and clamp of the step to the time range (adjoints.py:150-155, 247-251),
// controller history, step proposal, error ratio and error estimate (step_size_controllers.py:
// 598-620, 738-767, runge_kutta.py:265-272) -- to cotangents of k_0..k_6, y, y1, t, dt and the
// history.  stage_backward_kernel, once per stage from the last to the first, takes the cotangent
// of a stage input (which the caller gets from f's own vector-Jacobian product of the cotangent of
// k_s) through  ystage_s = y + dt sum_j a_sj k_j,  tnode_s = t + c_s dt  (runge_kutta.py:259-262).
// Selections follow torch's rules: maximum / minimum give half to each operand on a tie, clamp
// passes the cotangent on where the value lies within the bounds (inclusive), a bound receives it
// where the value lies outside; abs has slope sign(x).

template <typename TT, typename T> struct AdjointParams {
    long long batch;
    int F, E, iteration, through_control, end_point;
    const TT *t_start, *t_end, *t_eval, *t, *dt, *fixed_dt;
    const T *y, *y1, *prev, *pprev, *k[7], *grad_ys;
    const int32_t *running, *moved, *running_next, *hit_iteration;
    const TT *a_t, *a_dt;
    const T *a_y, *a_k0, *a_prev, *a_pprev;
    T *g_k[7], *g_y, *g_y1, *g_prev, *g_pprev;
    TT *g_t, *g_dt, *g_t_start, *g_t_end, *g_t_eval, *g_fixed_dt;
    CtrlParams<T> cp;
    TT dt_min, dt_max;
};

template <typename T> __device__ __forceinline__ T sign_(T x) { return x > (T)0 ? (T)1 : (x < (T)0 ? (T)-1 : (T)0); }

// cotangents of the operands of maximum(a, b) given the cotangent g of the result
template <typename T> __device__ __forceinline__ void max_backward(T a, T b, T g, T &ga, T &gb) {
    ga = a > b ? g : (a == b ? g / (T)2 : (T)0);
    gb = b > a ? g : (a == b ? g / (T)2 : (T)0);
}

// Both reverse kernels come in two shapes, like the forward ones: one thread per sample walking its row (WAVE false,
// rows of fewer than 64 features), and one wavefront per sample with its lanes strided over the row (WAVE true); sums
// over a row are then completed across the wavefront and per-sample results are stored by lane 0.
template <bool WAVE, typename T> __device__ __forceinline__ T row_sum(T v) {
    if (WAVE) {
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off);
    }
    return v;
}

// (the body of finish_backward_kernel for sample b; f_first / f_step: the features this thread walks)
// points / n_listed: the evaluation points this iteration wrote, where the caller knows them (n_listed >= 0); else
// every point of the row is looked at and those with hit_iteration == iteration are taken.
// FC: the row length where the caller knows it at compile time (0: p.F).  With FC set, b == 0 and every per-sample
// array a thread-private one, all indices are constants and the arrays can live in registers.
template <typename TT, typename T, int METHOD, int CTRL, bool WAVE, int FC = 0>
__device__ __forceinline__ void finish_backward_sample(const AdjointParams<TT, T> &p, const long long b, const int f_first, const int f_step,
                                                       const int32_t *points = nullptr, const int n_listed = -1) {
    using Tab = typename std::conditional<METHOD == 1, Tsit5Tab, Dopri5Tab>::type;
    const bool scalar_lane = f_first == 0;
    const int F = FC > 0 ? FC : p.F, E = p.E;
    const CtrlParams<T> &cp = p.cp;
    const TT t0 = p.t[b], dt = p.dt[b];
    const T h = (T)dt;
    const TT ts = p.t_start[b], te = p.t_end[b];
    const bool move = p.moved[b] != 0, running_new = p.running_next[b] != 0;
    const T *y = p.y + b * F, *y1 = p.y1 + b * F;
    const T sf = (T)__builtin_sqrt((double)F);

    // ---- forward values of the controller ----
    T acc = 0;
#pragma unroll
    for (int f = f_first; CTRL != 2 && f < F; f += f_step) {
        T err = 0;
#pragma unroll
        for (int s = 0; s < 7; ++s) err = fma_(h * (T)Tab::b_err[s], p.k[s][b * F + f], err);
        const T m = tmax(abs_(y[f]), abs_(y1[f]));
        const T x = (abs_(err) / fma_(cp.rtol, m, cp.atol)) / sf;
        acc = fma_(x, x, acc);
    }
    acc = row_sum<WAVE>(acc);
    const T r = sqrt_(acc), ratio = tmax(r, (T)1e-38);
    const T prev = p.prev[b], pprev = p.pprev[b];
    T F0 = 1, factor = 1;
    TT raw = 0, dt_next = 0;
    if (CTRL == 2) {
        dt_next = p.fixed_dt[b];
    } else {
        F0 = cp.safety * rpow<T>(ratio, cp.e1);
        if (CTRL == 1) {
            F0 = F0 * (cp.skip2 ? (T)1 : rpow<T>(prev, cp.e2));
            F0 = F0 * (cp.skip3 ? (T)1 : rpow<T>(pprev, cp.e3));
        }
        factor = tclamp(F0, cp.fmin, cp.fmax);
        raw = dt * (TT)factor;
        dt_next = raw;
        (void)limit_step<TT, T>(cp, p.dt_min, p.dt_max, ratio, dt_next);
    }
    const TT t_new = move ? (t0 + dt) : t0;
    const TT tlo = tmin(ts, te), thi = tmax(te, ts);
    const TT lo = tlo - t_new, hi = thi - t_new;
    const TT dtn = running_new ? dt_next : dt;

    // ---- clamp of the step to the time range, and the new time ----
    const TT a_dt = p.a_dt ? p.a_dt[b] : (TT)0;
    TT g_tnew = p.a_t ? p.a_t[b] : (TT)0;
    TT g_dt = 0, g_dt_next = 0;
    {
        const TT g_self = (dtn >= lo && dtn <= hi) ? a_dt : (TT)0;
        const TT g_lo = (dtn < lo && lo < hi) ? a_dt : (TT)0;
        const TT g_hi = (dtn > hi || hi < lo) ? a_dt : (TT)0;
        g_tnew -= g_lo + g_hi;
        TT g_ts_lo, g_te_lo, g_ts_hi, g_te_hi;
        // tlo = minimum(t_start, t_end), thi = maximum(t_start, t_end) (problems.py:58-64)
        max_backward<TT>(-ts, -te, g_lo, g_ts_lo, g_te_lo);  // minimum(a, b) = -maximum(-a, -b): same split
        max_backward<TT>(ts, te, g_hi, g_ts_hi, g_te_hi);
        if (p.g_t_start && scalar_lane) p.g_t_start[b] += g_ts_lo + g_ts_hi;
        if (p.g_t_end && scalar_lane) p.g_t_end[b] += g_te_lo + g_te_hi;
        if (running_new) g_dt_next = g_self;
        else g_dt = g_self;
    }
    TT g_t = g_tnew;
    if (move) g_dt += g_tnew;

    // ---- controller history and step proposal ----
    T g_ratio = 0, g_prev = 0, g_pprev = 0;
    if (CTRL == 1) {
        const bool keep = running_new && move;
        const T a_prev = p.a_prev ? p.a_prev[b] : (T)0, a_pprev = p.a_pprev ? p.a_pprev[b] : (T)0;
        g_ratio = keep ? a_prev : (T)0;
        g_prev = keep ? a_pprev : a_prev;
        g_pprev = keep ? (T)0 : a_pprev;
    }
    if (CTRL == 2) {
        if (p.through_control && p.g_fixed_dt && scalar_lane) p.g_fixed_dt[b] += g_dt_next;
    } else if (p.through_control) {
        TT g_raw = g_dt_next;
        if (cp.has_dt_min || cp.has_dt_max) {
            const TT mag = abs_(raw);
            const bool inside = (!cp.has_dt_min || mag >= p.dt_min) && (!cp.has_dt_max || mag <= p.dt_max);
            g_raw = (inside && raw != (TT)0) ? g_dt_next : (TT)0;
        }
        g_dt += g_raw * (TT)factor;
        const T g_factor = (T)(g_raw * dt);
        const T g_F0 = (F0 >= cp.fmin && F0 <= cp.fmax) ? g_factor : (T)0;
        g_ratio += g_F0 * F0 * (T)cp.e1 / ratio;
        if (CTRL == 1) {
            if (!cp.skip2) g_prev += g_F0 * F0 * (T)cp.e2 / prev;
            if (!cp.skip3) g_pprev += g_F0 * F0 * (T)cp.e3 / pprev;
        }
    }

    // ---- error ratio and error estimate; state update ----
    const T tiny = (T)1e-38;
    const T g_r = r > tiny ? g_ratio : (r == tiny ? g_ratio / (T)2 : (T)0);
    T g_h = 0;  // (this lane's share; summed over the row at the end)
#pragma unroll
    for (int f = f_first; f < F; f += f_step) {
        const long long i = b * F + f;
        const T a_y = p.a_y ? p.a_y[i] : (T)0, a_k0 = p.a_k0 ? p.a_k0[i] : (T)0;
        T gy = move ? (T)0 : a_y, gy1 = move ? a_y : (T)0;
        T gk[7] = {move ? (T)0 : a_k0, 0, 0, 0, 0, 0, move ? a_k0 : (T)0};
        if (CTRL != 2 && g_r != (T)0 && r > (T)0) {
            T err = 0, bk = 0;
#pragma unroll
            for (int s = 0; s < 7; ++s) {
                err = fma_(h * (T)Tab::b_err[s], p.k[s][i], err);
                bk = fma_((T)Tab::b_err[s], p.k[s][i], bk);
            }
            const T ay = abs_(y[f]), ay1 = abs_(y1[f]);
            const T eb = fma_(cp.rtol, tmax(ay, ay1), cp.atol);
            const T q = abs_(err) / eb;
            const T g_q = g_r * (q / sf) / r / sf;
            const T g_err = g_q / eb * sign_(err);
            const T g_m = -g_q * q / eb * cp.rtol;
            T ga, gb;
            max_backward<T>(ay, ay1, g_m, ga, gb);
            gy += ga * sign_(y[f]);
            gy1 += gb * sign_(y1[f]);
#pragma unroll
            for (int s = 0; s < 7; ++s) gk[s] += g_err * (h * (T)Tab::b_err[s]);
            g_h += g_err * bk;
        }
        p.g_y[i] = gy;
        p.g_y1[i] = gy1;
#pragma unroll
        for (int s = 0; s < 7; ++s) p.g_k[s][i] = gk[s];
    }

    // ---- dense output: the evaluation points this iteration wrote ----
    const TT t1 = t0 + dt;
    TT den = t1 - t0;
    const bool flat = !(abs_(den) > (TT)0);
    if (flat) den = (TT)1;
    const int n_points = E > 0 ? (n_listed >= 0 ? n_listed : E) : (p.end_point ? 1 : 0);
    for (int idx = 0; idx < n_points; ++idx) {
        const int e = (E > 0 && n_listed >= 0) ? points[idx] : idx;
        if (E > 0 && n_listed < 0 && p.hit_iteration[b * E + e] != p.iteration) continue;
        const TT at = E > 0 ? p.t_eval[b * E + e] : te;
        const T x = (T)((at - t0) / den);
        T g_x = 0;
#pragma unroll
        for (int f = f_first; f < F; f += f_step) {
            const long long i = b * F + f;
            const T g = p.grad_ys[(b * (long long)(E > 0 ? E : 1) + e) * F + f];
            if (g == (T)0) continue;
            T ks[7];
#pragma unroll
            for (int s = 0; s < 7; ++s) ks[s] = p.k[s][i];
            // coefficients (lowest power first) and their cotangents g x^p
            T q[5][1];
            quartic_elem<T, METHOD>(h, y[f], y1[f], ks, true, q);
            g_x += g * (q[1][0] + x * ((T)2 * q[2][0] + x * ((T)3 * q[3][0] + x * (T)4 * q[4][0])));
            const T g0 = g, g1 = g * x, g2 = g1 * x, g3 = g2 * x, g4 = g3 * x;
            if (METHOD == 1) {
                p.g_y[i] += g0;
                p.g_k[0][i] += g1 * h;
                g_h += g1 * ks[0];
#pragma unroll
                for (int s = 0; s < 7; ++s) {
                    const T w = g2 * (T)Tsit5Tab::w[0][s] + g3 * (T)Tsit5Tab::w[1][s] + g4 * (T)Tsit5Tab::w[2][s];
                    p.g_k[s][i] += w * h;
                    g_h += w * ks[s];
                }
            } else {
                const T g_f0 = (T)-2 * g4 + (T)5 * g3 - (T)4 * g2 + g1, g_f1 = (T)2 * g4 - (T)3 * g3 + g2;
                const T g_mid = (T)16 * g4 - (T)32 * g3 + (T)16 * g2;
                p.g_y[i] += (T)-8 * g4 + (T)18 * g3 - (T)11 * g2 + g0 + g_mid;
                p.g_y1[i] += (T)-8 * g4 + (T)14 * g3 - (T)5 * g2;
                p.g_k[0][i] += g_f0 * h;
                p.g_k[6][i] += g_f1 * h;
                g_h += g_f0 * ks[0] + g_f1 * ks[6];
#pragma unroll
                for (int s = 0; s < 7; ++s) {
                    p.g_k[s][i] += g_mid * (h * (T)Dopri5Tab::w[0][s]);
                    g_h += g_mid * (T)Dopri5Tab::w[0][s] * ks[s];
                }
            }
        }
        // x = (at - t0) / ((t0 + dt) - t0)
        const TT gx = (TT)row_sum<WAVE>(g_x);
        if (E > 0) {
            if (p.g_t_eval && scalar_lane) p.g_t_eval[b * E + e] += gx / den;
        } else if (p.g_t_end && scalar_lane) {
            p.g_t_end[b] += gx / den;
        }
        g_t -= gx / den;
        if (!flat) g_dt -= gx * (TT)x / den;
    }

    g_h = row_sum<WAVE>(g_h);
    if (scalar_lane) {
        p.g_t[b] = g_t;
        p.g_dt[b] = g_dt + (TT)g_h;
        p.g_prev[b] = g_prev;
        p.g_pprev[b] = g_pprev;
    }
}

template <typename TT, typename T, int METHOD, int CTRL, bool WAVE> __global__ void __launch_bounds__(256) finish_backward_kernel(const AdjointParams<TT, T> p) {
    const long long b = WAVE ? (long long)blockIdx.x * 4 + (threadIdx.x >> 6) : (long long)blockIdx.x * 256 + threadIdx.x;
    if (b >= p.batch) return;
    finish_backward_sample<TT, T, METHOD, CTRL, WAVE>(p, b, WAVE ? (int)(threadIdx.x & 63) : 0, WAVE ? 64 : 1);
}

// Stage S reversed.  g_ystage [B,F]: cotangent of the stage input; g_tnode [B] (may be null): of its time.
template <typename TT, typename T, int METHOD, bool WAVE, int FC = 0>
__device__ __forceinline__ void stage_backward_sample(const AdjointParams<TT, T> &p, const long long b, const int S, const T *g_ystage, const TT *g_tnode,
                                                      const int f_first, const int f_step) {
    using Tab = typename std::conditional<METHOD == 1, Tsit5Tab, Dopri5Tab>::type;
    const int F = FC > 0 ? FC : p.F;
    const T h = (T)p.dt[b];
    T a[7];
#pragma unroll
    for (int j = 0; j < 7; ++j) a[j] = j < S ? (T)Tab::a[S][j] : (T)0;
    T g_h = 0;
#pragma unroll
    for (int f = f_first; f < F; f += f_step) {
        const long long i = b * F + f;
        const T g = g_ystage[i];
        p.g_y[i] += g;
        T s = 0;
#pragma unroll
        for (int j = 0; j < S; ++j) {
            s = fma_(a[j], p.k[j][i], s);
            p.g_k[j][i] += a[j] * h * g;
        }
        g_h += g * s;
    }
    g_h = row_sum<WAVE>(g_h);
    if (f_first != 0) return;
    const TT g_tau = g_tnode ? g_tnode[b] : (TT)0;
    p.g_t[b] += g_tau;
    p.g_dt[b] += (TT)g_h + (TT)Tab::c[S] * g_tau;
}

template <typename TT, typename T, int METHOD, bool WAVE> __global__ void __launch_bounds__(256)
stage_backward_kernel(const AdjointParams<TT, T> p, int S, const T *g_ystage, const TT *g_tnode) {
    const long long b = WAVE ? (long long)blockIdx.x * 4 + (threadIdx.x >> 6) : (long long)blockIdx.x * 256 + threadIdx.x;
    if (b >= p.batch) return;
    stage_backward_sample<TT, T, METHOD, WAVE>(p, b, S, g_ystage, g_tnode, WAVE ? (int)(threadIdx.x & 63) : 0, WAVE ? 64 : 1);
}

}  // namespace tode
