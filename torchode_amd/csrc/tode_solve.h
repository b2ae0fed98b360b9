// Pieces shared by the whole-solve kernels: built-in right-hand sides, kernel
// parameter block and the start-step selection.
#pragma once
#include <hip/hip_runtime.h>
#include <limits.h>

#include <type_traits>

#include "../../include/torchode_amd.h"
#include "tode_internal.h"
#include "tode_math.h"

namespace tode {


// ---------------------------------------------------------------------------
// Built-in right-hand sides.  Op order is part of the contract: each line is one
// rounding, matching an eager evaluation of the torch expression in the comment.
// ---------------------------------------------------------------------------
template <typename T, int F_> struct LinearDecayTerm {  // (-k) * y
    static constexpr int F = F_;
    static constexpr int P = F_;
    T nk[F_];
    __device__ __forceinline__ void load(const T *par, const double *) {
#pragma unroll
        for (int f = 0; f < F; ++f) nk[f] = -par[f];
    }
    __device__ __forceinline__ void operator()(T, const T (&y)[F_], T (&dy)[F_]) const {
#pragma unroll
        for (int f = 0; f < F; ++f) dy[f] = nk[f] * y[f];
    }
    // vector-Jacobian product: g is the cotangent of dy; gy receives that of y, gpar is added to that of k
    __device__ __forceinline__ void vjp(T, const T (&y)[F_], const T (&g)[F_], T (&gy)[F_], T (&gpar)[F_]) const {
#pragma unroll
        for (int f = 0; f < F; ++f) {
            gy[f] = nk[f] * g[f];
            gpar[f] -= y[f] * g[f];
        }
    }
};

template <typename T> struct VanDerPolTerm {  // dx = v ; dv = ((mu*(1-(x*x)))*v)-x
    static constexpr int F = 2;
    static constexpr int P = 1;
    T mu;
    __device__ __forceinline__ void load(const T *par, const double *) { mu = par[0]; }
    __device__ __forceinline__ void operator()(T, const T (&y)[2], T (&dy)[2]) const {
        T x = y[0], v = y[1];
        T xx = x * x;
        T om = (T)1 - xx;
        T m1 = mu * om;
        T m2 = m1 * v;
        dy[0] = v;
        dy[1] = m2 - x;
    }
    __device__ __forceinline__ void vjp(T, const T (&y)[2], const T (&g)[2], T (&gy)[2], T (&gpar)[1]) const {
        const T x = y[0], v = y[1], om = (T)1 - x * x;
        gy[0] = g[1] * (mu * ((T)-2 * x) * v - (T)1);
        gy[1] = g[0] + g[1] * (mu * om);
        gpar[0] += g[1] * (om * v);
    }
};

template <typename T> struct Lorenz63Term {  // dx=sigma*(y-x); dy=(x*(rho-z))-y; dz=(x*y)-(beta*z)
    static constexpr int F = 3;
    static constexpr int P = 1;
    T rho, sigma, beta;
    __device__ __forceinline__ void load(const T *par, const double *sc) {
        rho = par[0];
        sigma = (T)sc[0];
        beta = (T)sc[1];
    }
    __device__ __forceinline__ void operator()(T, const T (&y)[3], T (&dy)[3]) const {
        T x = y[0], yy = y[1], z = y[2];
        T d1 = yy - x;
        T r1 = rho - z;
        T xr = x * r1;
        T xy = x * yy;
        T bz = beta * z;
        dy[0] = sigma * d1;
        dy[1] = xr - yy;
        dy[2] = xy - bz;
    }
    __device__ __forceinline__ void vjp(T, const T (&y)[3], const T (&g)[3], T (&gy)[3], T (&gpar)[1]) const {
        const T x = y[0], yy = y[1], z = y[2];
        gy[0] = (rho - z) * g[1] + yy * g[2] - sigma * g[0];
        gy[1] = sigma * g[0] - g[1] + x * g[2];
        gy[2] = -(x * g[1]) - beta * g[2];
        gpar[0] += x * g[1];
    }
};

// T: data type (state, parameters, tolerances, error ratio, step factor, output).  TT: time type (times, steps and
// their limits; problems.py:44-56 lets the two differ).  Only the general kernel is built for TT != T.
template <typename T, typename TT = T> struct SolveParams {
    const T *y0, *params;
    const TT *t_start, *t_end, *t_eval, *dt0;
    TT dt_min, dt_max;  // the controller's step limits in the time type
    T *ys, *y_idle;
    uint8_t *pending;
    int32_t *n_steps, *n_accepted, *n_initialized, *status_last, *status_idle, *flags;
    int32_t *host_flags;  // pinned host words the last workgroup publishes the flags to, or null
    int32_t sequence;     // written behind them, so that the host sees when they have arrived
    long long batch, ts_stride, te_stride;
    int n_eval;
    int max_steps;  // INT_MAX: unlimited
    int cap;        // INT_MAX: unlimited
    double scalars[4];
    CtrlParams<T> cp;
    // record of the loop state per iteration (tode_solve_record), null pointers when none is kept
    long long rec_capacity;
    TT *rec_t, *rec_dt;
    T *rec_y, *rec_k0, *rec_prev, *rec_pprev;
    int32_t *rec_running, *rec_n_accepted;
};

// Entry `at` of the record of the loop state (tode_solve_record) for sample b: what the reference's loop variables hold
// before that iteration (adjoints.py:135-260).  The caller has checked at < p.rec_capacity.
template <typename T, typename TT, int F>
__device__ __forceinline__ void record_entry(const SolveParams<T, TT> &p, long long at, long long b, TT t, TT dt, const T (&y)[F], const T (&k0)[F], T prev,
                                             T prev_prev, bool running, int n_accepted) {
    const long long i = at * p.batch + b;
    p.rec_t[i] = t, p.rec_dt[i] = dt;
#pragma unroll
    for (int f = 0; f < F; ++f) p.rec_y[i * F + f] = y[f], p.rec_k0[i * F + f] = k0[f];
    p.rec_prev[i] = prev, p.rec_pprev[i] = prev_prev;
    p.rec_running[i] = running ? 1 : 0, p.rec_n_accepted[i] = n_accepted;
}

// Start step (step_size_controllers.py:431-490 integral, 776-835 PID; the integral
// copy maps h0 == 0 to d2 = inf, the PID copy does not).
template <typename T, int CTRL, typename Term>
__device__ __forceinline__ T initial_step(const CtrlParams<T> &cp, const Term &rhs, T t0, const T (&y0)[Term::F], T dir, T span,
                                          T (&f0)[Term::F]) {
    constexpr int F = Term::F;
    rhs(t0, y0, f0);
    T inv[F], w[F];
#pragma unroll
    for (int f = 0; f < F; ++f) inv[f] = (T)1 / fma_(cp.rtol, abs_(y0[f]), cp.atol);
#pragma unroll
    for (int f = 0; f < F; ++f) w[f] = y0[f] * inv[f];
    T d0 = rms<T, F>(w);
#pragma unroll
    for (int f = 0; f < F; ++f) w[f] = f0[f] * inv[f];
    T d1 = rms<T, F>(w);
    const T tiny = (T)1e-6;
    T h0 = (d0 < (T)1e-5 || d1 < (T)1e-5) ? tiny : ((T)0.01 * d0) / d1;
    h0 = tmin(h0, span);
    T dh = dir * h0;
    T y1[F], f1[F];
#pragma unroll
    for (int f = 0; f < F; ++f) y1[f] = fma_(dh, f0[f], y0[f]);
    T t1 = fma_(dir, h0, t0);
    rhs(t1, y1, f1);
#pragma unroll
    for (int f = 0; f < F; ++f) {
        T df = f1[f] - f0[f];
        w[f] = df * inv[f];
    }
    T d2 = rms<T, F>(w) / h0;
    if (CTRL == 0 && h0 == (T)0) d2 = (T)__builtin_huge_val();
    T m = tmax(d1, d2);
    T h1;
    if (m <= (T)1e-15) {
        h1 = tmax(tiny, h0 * (T)1e-3);
    } else {
        // python_float / tensor is evaluated by torch as reciprocal(tensor) * python_float
        T rm = (T)1 / m;
        h1 = rpow<T>(rm * (T)0.01, 1.0 / 5.0);
    }
    return dir * tmin((T)100 * h0, h1);
}


// Pieces of the start step and of the dense output shared by the per-call operators and the
// whole-solve kernels for long rows.
template <typename T> __device__ __forceinline__ T inv_scale(T atol, T rtol, T y0) { return (T)1 / fma_(rtol, abs_(y0), atol); }

template <typename T> __device__ __forceinline__ T initial_finish(int kind, double inv_order, T dir, T h0, T d1, T d2n) {
    T d2 = d2n / h0;
    if (kind == TODE_CTRL_INTEGRAL && h0 == (T)0) d2 = (T)__builtin_huge_val();
    const T m = tmax(d1, d2);
    T h1;
    if (m <= (T)1e-15) {
        h1 = tmax((T)1e-6, h0 * (T)1e-3);
    } else {
        const T rm = (T)1 / m;  // python_float / tensor runs as reciprocal(tensor) * python_float
        h1 = rpow<T>(rm * (T)0.01, inv_order);
    }
    return dir * tmin((T)100 * h0, h1);
}

// n_initialized as the reference forms it (adjoints.py:289-292): torch.searchsorted(pending, 1), ATen's
// lower-bound binary search.  On a sorted row of marks (evaluation times monotone in the sample's direction) this
// is the index of the first pending point; on any other row it is whatever the search lands on, mirrored here.
__device__ __forceinline__ int searchsorted_first_pending(const uint8_t *pending, int E) {
    int lo = 0, hi = E;
    while (lo < hi) {
        const int mid = lo + ((hi - lo) >> 1);
        if (!pending[mid]) lo = mid + 1; else hi = mid;
    }
    return lo;
}

// x = (t - t0) / (t1 - t0) with a zero interval mapped to 1 (interpolation.py:8-40)
template <typename T> __device__ __forceinline__ T unit_time_over(T t, T t0, T den) {
    if (!(abs_(den) > (T)0)) den = (T)1;
    return (t - t0) / den;
}
template <typename T> __device__ __forceinline__ T unit_time(T t, T t0, T t1) { return unit_time_over(t, t0, t1 - t0); }

template <typename T> __device__ __forceinline__ T horner(const T *coeff, long long bf, long long at, int degree, T x) {
    T y = coeff[degree * bf + at];
    for (int p = degree - 1; p >= 0; --p) y = fma_(y, x, coeff[p * bf + at]);
    return y;
}

// Controller parameters in the working type from the ABI struct.
template <typename T> static CtrlParams<T> make_ctrl(const tode_controller &c, double order = 5.0) {
    CtrlParams<T> cp;
    cp.atol = (T)(float)c.atol;
    cp.rtol = (T)(float)c.rtol;
    cp.safety = (T)c.safety;
    cp.fmin = (T)c.factor_min;
    cp.fmax = (T)c.factor_max;
    cp.dt_min = (T)c.dt_min;
    cp.dt_max = (T)c.dt_max;
    cp.has_dt_min = c.has_dt_min;
    cp.has_dt_max = c.has_dt_max;
    // order: convergence order of the step method; 5 for both pairs (dopri5.py:49-51, tsit5.py:119-121)
    if (c.kind == TODE_CTRL_INTEGRAL) {
        cp.e1 = -(1.0 / order);
        cp.e2 = cp.e3 = 0.0;
    } else {
        double k_i = c.icoeff / order, k_p = c.pcoeff / order, k_d = c.dcoeff / order;
        cp.e1 = -(k_i + k_p + k_d);
        cp.e2 = k_p + 2 * k_d;
        cp.e3 = -k_d;
    }
    cp.skip2 = ((double)(T)cp.e2 == 0.0);
    cp.skip3 = ((double)(T)cp.e3 == 0.0);
    return cp;
}

template <typename T, typename TT = T> static SolveParams<T, TT> make_params(const tode_solve_args &a, const tode_controller &c) {
    SolveParams<T, TT> p;
    p.y0 = (const T *)a.y0;
    p.t_start = (const TT *)a.t_start;
    p.t_end = (const TT *)a.t_end;
    p.t_eval = a.n_eval > 0 ? (const TT *)a.t_eval : nullptr;
    p.dt0 = (const TT *)a.dt0;
    p.dt_min = (TT)c.dt_min;
    p.dt_max = (TT)c.dt_max;
    p.params = (const T *)a.params;
    p.ys = (T *)a.ys;
    p.y_idle = (T *)a.y_idle;
    p.pending = a.pending;
    p.n_steps = a.n_steps;
    p.n_accepted = a.n_accepted;
    p.n_initialized = a.n_initialized;
    p.status_last = a.status_last;
    p.status_idle = a.status_idle;
    const FlagTarget *target = flag_target();
    p.flags = target ? target->dev : a.flags;
    p.host_flags = target ? target->host : nullptr;
    p.sequence = target ? target->sequence : 0;
    p.batch = a.batch;
    p.ts_stride = a.t_start_stride;
    p.te_stride = a.t_end_stride;
    p.n_eval = a.n_eval;
    p.max_steps = (a.max_steps < 0 || a.max_steps >= INT_MAX) ? INT_MAX : (int)a.max_steps;
    p.cap = (a.iteration_cap < 0 || a.iteration_cap >= INT_MAX) ? INT_MAX : (int)a.iteration_cap;
    for (int i = 0; i < 4; ++i) p.scalars[i] = a.term_scalars[i];
    p.cp = make_ctrl<T>(c);
    const tode_solve_record *r = a.record;
    p.rec_capacity = r ? r->capacity : 0;
    p.rec_t = r ? (TT *)r->t : nullptr, p.rec_dt = r ? (TT *)r->dt : nullptr;
    p.rec_y = r ? (T *)r->y : nullptr, p.rec_k0 = r ? (T *)r->k0 : nullptr;
    p.rec_prev = r ? (T *)r->prev : nullptr, p.rec_pprev = r ? (T *)r->pprev : nullptr;
    p.rec_running = r ? r->running : nullptr, p.rec_n_accepted = r ? r->n_accepted : nullptr;
    return p;
}

// One wavefront reduces one row (F >= 64).  The order of summation is fixed, so that every kernel
// that forms such a norm gets the same bits: the row is cut into chunks of 256 values; within a
// chunk lane l accumulates values 4l..4l+3 in order (fused multiply-add from zero), the 64 partial
// sums are combined by a butterfly (xor 32, 16, .., 1), and the chunk sums are added in order.
template <typename T, int NORM, typename Load> __device__ __forceinline__ T wave_row_norm(int F, Load load) {
    const int lane = threadIdx.x & 63;
    const T sf = (T)__builtin_sqrt((double)F);
    T total = 0;
    for (int base = 0; base < F; base += 256) {
        T p = 0;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int f = base + 4 * lane + j;
            if (f < F) {
                const T v = load(f);
                if (NORM == TODE_NORM_MAX)
                    p = tmax(p, abs_(v));
                else {
                    const T x = v / sf;
                    p = fma_(x, x, p);
                }
            }
        }
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) {
            const T o = __shfl_xor(p, off);
            p = NORM == TODE_NORM_MAX ? tmax(p, o) : p + o;
        }
        total = NORM == TODE_NORM_MAX ? tmax(total, p) : total + p;
    }
    return NORM == TODE_NORM_MAX ? total : sqrt_(total);
}

// Workgroup barrier that orders LDS accesses only.  __syncthreads() also waits for the wavefront's
// global stores to be acknowledged -- in the whole-solve kernels the dense output, which no thread
// of the kernel ever reads -- and that wait (a round trip to memory) would sit on the critical path
// of the next stage.
__device__ __forceinline__ void lds_barrier() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

// End of a whole-solve kernel, reached by every thread of every workgroup after the workgroup's
// updates of the flag words.  With a host target, word TODE_FLAG_WORDS counts finished workgroups;
// the last one takes the flag words, puts them back to their start values for the next solve that
// uses them, and stores them to the host, the sequence number last.
//
// Only the flag words themselves need ordering, and they are touched by device-scope atomics alone,
// which act on the one coherent copy of each word: no release of the workgroup's other writes (it
// would write back the L2 once per workgroup).  The barrier makes every wavefront wait for its own
// atomics to complete; the count is incremented after it, so whoever sees the final count issues
// its exchanges after every update has been performed.
template <typename T, typename TT> __device__ __forceinline__ void publish_flags(const SolveParams<T, TT> &p) {
    if (p.host_flags == nullptr) return;
    __syncthreads();
    if (threadIdx.x != 0 || threadIdx.y != 0) return;
    const int finished = __hip_atomic_fetch_add(&p.flags[TODE_FLAG_WORDS], 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (finished != (int)(gridDim.x * gridDim.y) - 1) return;
    const int32_t start[TODE_FLAG_WORDS] = {0, INT_MAX, 0, 0};
    int32_t v[TODE_FLAG_WORDS];
#pragma unroll
    for (int i = 0; i < TODE_FLAG_WORDS; ++i) v[i] = __hip_atomic_exchange(&p.flags[i], start[i], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    (void)__hip_atomic_exchange(&p.flags[TODE_FLAG_WORDS], 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
    for (int i = 0; i < TODE_FLAG_WORDS; ++i) __hip_atomic_store(&p.host_flags[i], v[i], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
    // (the release also covers the exchanges above: a later kernel finds the words reset)
    // (a target without a sequence number is read in stream order, after the kernel: nothing to announce)
    if (p.sequence != 0) __hip_atomic_store(&p.host_flags[TODE_FLAG_WORDS], p.sequence, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_SYSTEM);
}

// Resets the flag block; launched in front of every solve kernel.
static __global__ void init_flags_kernel(int32_t *flags) {
    if (threadIdx.x == 0) {
        flags[TODE_FLAG_MAX_ITERATIONS] = 0;
        flags[TODE_FLAG_FIRST_FAILURE] = INT_MAX;
        flags[TODE_FLAG_NON_MONOTONE] = 0;
        flags[TODE_FLAG_NEEDS_GENERAL] = 0;
    }
}

// In front of a fast solve kernel: resets the caller's flag block, unless the kernel works on the
// library's self-resetting words.
static inline void reset_flags(int32_t *flags, hipStream_t stream) {
    if (flag_target() == nullptr) hipLaunchKernelGGL(init_flags_kernel, dim3(1), dim3(64), 0, stream, flags);
}

}  // namespace tode
