// Persistent whole-solve kernel: one sample per lane, the complete adaptive
// Runge-Kutta loop (start step, stages, error estimate, step size control,
// accept/reject, dense output, counters and status) runs in registers, and the
// only HBM traffic is the problem in and the solution out.
//
// The reference steps the whole batch in lock step (torchode adjoints.py:135-260).
// Samples are independent except for two batch-wide effects -- the loop runs
// until the slowest sample has finished, and the first non-success status stops
// everybody -- so each lane runs its own loop and reports, through the flag
// block, what the caller needs to restore those two effects.
#include "tode_solve.h"

namespace tode {

// T: data type, TT: time type (the same in the common case; where they differ the conversions stand where the
// reference's loop of torch operations has them: the step in the data type for stage sums and interpolants, the step
// factor in the time type for the next step, the position of an evaluation point in its step formed in the time type).
// RECORD: the loop state before every iteration goes to p.rec_* (tode_solve_record), for a reverse sweep.
template <typename T, int METHOD, int CTRL, typename Term, typename TT = T, bool RECORD = false>
__global__ void __launch_bounds__(TODE_BLOCK) solve_kernel(const SolveParams<T, TT> p) {
    using Tab = typename std::conditional<METHOD == 1, Tsit5Tab, Dopri5Tab>::type;
    constexpr int F = Term::F;
    constexpr int P = Term::P;
    const long long b = (long long)blockIdx.x * TODE_BLOCK + threadIdx.x;
    const bool live = b < p.batch;
    const CtrlParams<T> &cp = p.cp;
    const int E = p.n_eval;

    int my_fail = INT_MAX, my_steps = 0, my_nonmono = 0, my_overflow = 0;

    if (live) {
        Term rhs;
        rhs.load(p.params + b * P, p.scalars);
        T y[F], k[7][F];
#pragma unroll
        for (int f = 0; f < F; ++f) y[f] = p.y0[b * F + f];
        const TT ts = p.t_start[b * p.ts_stride], te = p.t_end[b * p.te_stride];
        const T dir = (te > ts) ? (T)1 : (T)-1;
        const TT tlo = tmin(ts, te), thi = tmax(te, ts);
        const TT *tev = p.t_eval ? p.t_eval + b * E : nullptr;
        T *ys = p.ys + b * (long long)(E > 0 ? E : 1) * F;

        // evaluation points: a cursor is equivalent to the reference's pending mask when
        // the row is monotone in the direction of time; otherwise fall back to the mask
        bool use_mask = false;
        if (tev) {
            TT prev_te = tev[0];
            for (int e = 1; e < E; ++e) {
                TT cur = tev[e];
                if (!(dir > 0 ? cur >= prev_te : cur <= prev_te)) use_mask = true;
                prev_te = cur;
            }
        }
        uint8_t *pend = nullptr;
        bool bail = false;
        if (use_mask) {
            if (p.pending) {
                pend = p.pending + b * (long long)E;
                for (int e = 0; e < E; ++e) pend[e] = 1;
            } else {
                my_nonmono = 1;
                bail = true;
            }
        }

        TT t = ts, dt;
        if (p.dt0) {
            dt = p.dt0[b];
            rhs((T)ts, y, k[0]);
        } else {
            // (the terms built for this kernel do not look at the time they are given)
            dt = (TT)initial_step<T, CTRL, Term>(cp, rhs, (T)ts, y, dir, (T)abs_(te - ts), k[0]);
        }
        dt = tclamp(dt, tlo - t, thi - t);
        T prev = (T)1, prev_prev = (T)1;
        int cursor = 0;
        if (tev && E > 0 && tev[0] == ts) {
#pragma unroll
            for (int f = 0; f < F; ++f) ys[f] = y[f];
            if (pend)
                pend[0] = 0;
            else
                cursor = 1;
        }

        // next pending evaluation time, kept in a register between iterations
        TT te_next = (tev && cursor < E) ? tev[cursor] : (TT)0;

        int n_steps = 0, n_acc = 0, status_last = 0, status_idle = 0;
        bool idle_pass = false;
        bool go = !bail && p.cap > 0;
        bool still_running = true;  // (RECORD) the sample's `running` after its last own iteration
        // (RECORD) entry `at` of the record: the state as it is now
        auto keep = [&](long long at, bool running) {
            if (at >= p.rec_capacity) {
                my_overflow = 1;
                return;
            }
            record_entry<T, TT, F>(p, at, b, t, dt, y, k[0], prev, prev_prev, running, n_acc);
        };
        while (go) {
            if (RECORD && !idle_pass) keep(n_steps, true);
            // ---- stages (runge_kutta.py:255-263) ----
            const TT t0 = t;
            const T h = (T)dt;  // (the step in the data type: runge_kutta.py:246)
            T y1[F], err[F];
#pragma unroll
            for (int i = 1; i < 7; ++i) {
                TT tn = fma_((TT)Tab::c[i], dt, t0);
                T yi[F];
#pragma unroll
                for (int f = 0; f < F; ++f) {
                    T s = 0;
#pragma unroll
                    for (int j = 0; j < i; ++j) s = fma_((T)Tab::a[i][j], k[j][f], s);
                    yi[f] = fma_(h, s, y[f]);
                }
                rhs((T)tn, yi, k[i]);
                if (i == 6) {
#pragma unroll
                    for (int f = 0; f < F; ++f) y1[f] = yi[f];
                }
            }
            weighted_k<T, F, Tab, -1>(h, k, err);

            // ---- step size control (step_size_controllers.py:370-429, 715-774) ----
            const T ratio = error_ratio<T, F>(cp, y, y1, err);
            const bool accept = ratio < (T)1;
            TT dt_next = dt * (TT)dt_factor<T, CTRL>(cp, ratio, prev, prev_prev);
            int status = limit_step<TT, T>(cp, p.dt_min, p.dt_max, ratio, dt_next);

            const bool running = !idle_pass;
            const bool move = accept && running;
            const TT t_new = move ? (t0 + dt) : t0;
            const bool running_new = dir > 0 ? (t_new < te) : (t_new > te);
            if (RECORD && running) still_running = running_new;
            if (running) {
                n_steps += 1;
                n_acc += move ? 1 : 0;
            }
            if (p.max_steps != INT_MAX && n_steps >= p.max_steps) status = TODE_REACHED_MAX_STEPS;
            if (status == 0 && n_steps >= TODE_HARD_STEP_LIMIT) status = TODE_GENERAL_ERROR;
            const bool last_own = running && (status != 0 || !running_new || n_steps >= p.cap);

            // ---- dense output (adjoints.py:215-234): points passed by the new t ----
            bool have_q = false;
            T q[5][F];
            if (tev) {
                if (pend) {
                    for (int e = 0; e < E; ++e) {
                        if (!pend[e]) continue;
                        TT te_e = tev[e];
                        if (dir > 0 ? t_new >= te_e : t_new <= te_e) {
                            if (!have_q) {
                                quartic<T, F, METHOD>(h, y, y1, k, q);
                                have_q = true;
                            }
                            T out[F];
                            quartic_eval<T, F, TT>(q, t0, dt, te_e, out);
#pragma unroll
                            for (int f = 0; f < F; ++f) ys[(long long)e * F + f] = out[f];
                            pend[e] = 0;
                        }
                    }
                } else {
                    while (cursor < E) {
                        const TT te_e = te_next;
                        if (!(dir > 0 ? t_new >= te_e : t_new <= te_e)) break;
                        if (!have_q) {
                            quartic<T, F, METHOD>(h, y, y1, k, q);
                            have_q = true;
                        }
                        T out[F];
                        quartic_eval<T, F, TT>(q, t0, dt, te_e, out);
#pragma unroll
                        for (int f = 0; f < F; ++f) ys[(long long)cursor * F + f] = out[f];
                        ++cursor;
                        if (cursor < E) te_next = tev[cursor];
                    }
                }
            } else if (last_own || idle_pass) {
                // no evaluation points (adjoints.py:295-309): the interpolant of the loop's
                // last iteration evaluated at t_end
                quartic<T, F, METHOD>(h, y, y1, k, q);
                T out[F];
                quartic_eval<T, F, TT>(q, t0, dt, te, out);
                T *dst = idle_pass ? (p.y_idle + b * F) : ys;
#pragma unroll
                for (int f = 0; f < F; ++f) dst[f] = out[f];
            }

            // ---- state update (adjoints.py:150-155, 247-255) ----
            if (move) {
#pragma unroll
                for (int f = 0; f < F; ++f) {
                    y[f] = y1[f];
                    k[0][f] = k[6][f];
                }
            }
            t = t_new;
            const TT dtn = running_new ? dt_next : dt;
            dt = tclamp(dtn, tlo - t, thi - t);
            if (CTRL == 1 && running_new && accept) {
                prev_prev = prev;
                prev = ratio;
            }

            if (idle_pass) {
                status_idle = status;
                if (status != 0 && n_steps + 1 < my_fail) my_fail = n_steps + 1;
                break;
            }
            status_last = status;
            if (status != 0) {
                my_fail = n_steps;
                break;
            }
            if (!running_new) {
                // Finished.  Later iterations of the reference loop keep stepping this sample
                // with the clamped dt; that is observable only through its status and, without
                // evaluation points, through the end-point interpolant.  Both are trivial
                // (status 0, value y) unless one of the following holds.
                bool nontrivial = cp.has_dt_min || !(t == te);
#pragma unroll
                for (int f = 0; f < F; ++f) nontrivial = nontrivial || !settles_(y[f], k[0][f]);
                if (nontrivial) {
                    idle_pass = true;
                    continue;
                }
                if (!tev) {
#pragma unroll
                    for (int f = 0; f < F; ++f) p.y_idle[b * F + f] = y[f];
                }
                break;
            }
            if (n_steps >= p.cap) break;
        }

        if (RECORD) {
            // the state the sample is left in, and the same for every later iteration of the batch (a sample that never
            // started -- rows that need the pending mask and have none -- records nothing: the solve is repeated)
            if (!bail) {
                keep(n_steps, still_running);
                for (long long at = n_steps + 1; at < p.rec_capacity; ++at) keep(at, false);
            }
        }
        int n_init = 1;
        if (tev) {
            if (pend) {
                n_init = searchsorted_first_pending(pend, E);
            } else {
                n_init = cursor;
            }
        }
        p.n_steps[b] = n_steps;
        p.n_accepted[b] = n_acc;
        p.n_initialized[b] = n_init;
        p.status_last[b] = status_last;
        p.status_idle[b] = status_idle;
        my_steps = n_steps;
    }

    // one atomic per wave for the batch-wide facts
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        my_fail = min(my_fail, __shfl_xor(my_fail, off));
        my_steps = max(my_steps, __shfl_xor(my_steps, off));
        my_nonmono = max(my_nonmono, __shfl_xor(my_nonmono, off));
        my_overflow = max(my_overflow, __shfl_xor(my_overflow, off));
    }
    if ((threadIdx.x & 63) == 0) {
        if (my_steps > 0) atomicMax(&p.flags[TODE_FLAG_MAX_ITERATIONS], my_steps);
        if (my_fail != INT_MAX) atomicMin(&p.flags[TODE_FLAG_FIRST_FAILURE], my_fail);
        if (my_nonmono) atomicMax(&p.flags[TODE_FLAG_NON_MONOTONE], 1);
        if (my_overflow) atomicMax(&p.flags[TODE_FLAG_NEEDS_GENERAL], 1);  // (the record was too short)
    }
}

template <typename T, int METHOD, int CTRL, typename Term, typename TT>
static int launch(const tode_solve_args &a, const tode_controller &c, hipStream_t stream) {
    SolveParams<T, TT> p = make_params<T, TT>(a, c);
    if ((TODE_INSTANTIATE_RECORD != 0) != (a.record != nullptr)) return fail(TODE_E_INVALID, "internal: record variant mismatch");
    if (a.record) {
        const tode_solve_record &r = *a.record;
        if (r.capacity < 1 || (a.batch > 0 && (!r.t || !r.dt || !r.y || !r.k0 || !r.prev || !r.pprev || !r.running || !r.n_accepted)))
            return fail(TODE_E_INVALID, "tode_solve_record: capacity %lld, or a null array", (long long)r.capacity);
    }
    const long long blocks = (a.batch + TODE_BLOCK - 1) / TODE_BLOCK;
    hipLaunchKernelGGL(init_flags_kernel, dim3(1), dim3(64), 0, stream, a.flags);
    if (blocks > 0) {
        timing_before(stream, "tode::solve_kernel");
        hipLaunchKernelGGL((solve_kernel<T, METHOD, CTRL, Term, TT, TODE_INSTANTIATE_RECORD != 0>), dim3((unsigned)blocks), dim3(TODE_BLOCK), 0, stream, p);
        timing_after(stream);
    }
    return check_hip(hipGetLastError(), "tode_solve_builtin launch");
}

template <typename T, typename TT, typename Term> static int dispatch_mc(const tode_solve_args &a, const tode_controller &c, hipStream_t s) {
    if (a.method == TODE_DOPRI5 && c.kind == TODE_CTRL_INTEGRAL) return launch<T, 0, 0, Term, TT>(a, c, s);
    if (a.method == TODE_DOPRI5 && c.kind == TODE_CTRL_PID) return launch<T, 0, 1, Term, TT>(a, c, s);
    if (a.method == TODE_TSIT5 && c.kind == TODE_CTRL_INTEGRAL) return launch<T, 1, 0, Term, TT>(a, c, s);
    if (a.method == TODE_TSIT5 && c.kind == TODE_CTRL_PID) return launch<T, 1, 1, Term, TT>(a, c, s);
    return fail(TODE_E_INVALID, "unknown method %d or controller kind %d", a.method, c.kind);
}

template <typename T, typename TT = T> static int dispatch_term(const tode_solve_args &a, const tode_controller &c, hipStream_t s) {
    switch (a.term) {
    case TODE_TERM_VAN_DER_POL:
        if (a.n_features != 2 || a.n_params != 1) return fail(TODE_E_INVALID, "Van der Pol needs F=2, P=1");
        return dispatch_mc<T, TT, VanDerPolTerm<T>>(a, c, s);
    case TODE_TERM_LORENZ63:
        if (a.n_features != 3 || a.n_params != 1) return fail(TODE_E_INVALID, "Lorenz-63 needs F=3, P=1");
        return dispatch_mc<T, TT, Lorenz63Term<T>>(a, c, s);
    case TODE_TERM_LINEAR_DECAY:
        if (a.n_params != a.n_features) return fail(TODE_E_INVALID, "linear decay needs P == F");
        switch (a.n_features) {
        case 1: return dispatch_mc<T, TT, LinearDecayTerm<T, 1>>(a, c, s);
        case 2: return dispatch_mc<T, TT, LinearDecayTerm<T, 2>>(a, c, s);
        case 3: return dispatch_mc<T, TT, LinearDecayTerm<T, 3>>(a, c, s);
        case 4: return dispatch_mc<T, TT, LinearDecayTerm<T, 4>>(a, c, s);
        case 8: return dispatch_mc<T, TT, LinearDecayTerm<T, 8>>(a, c, s);
        default: return fail(TODE_E_UNSUPPORTED, "linear decay is built for F in {1,2,3,4,8}, got %d", a.n_features);
        }
    default:
        return fail(TODE_E_INVALID, "unknown built-in term %d", a.term);
    }
}

int solve_builtin_f32(const tode_solve_args &a, const tode_controller &c, hipStream_t s);
int solve_builtin_f64(const tode_solve_args &a, const tode_controller &c, hipStream_t s);
int solve_builtin_t64_y32(const tode_solve_args &a, const tode_controller &c, hipStream_t s);  // float64 times, float32 data
int solve_builtin_t32_y64(const tode_solve_args &a, const tode_controller &c, hipStream_t s);
int solve_builtin_f32_record(const tode_solve_args &a, const tode_controller &c, hipStream_t s);
int solve_builtin_f64_record(const tode_solve_args &a, const tode_controller &c, hipStream_t s);
int solve_builtin_t64_y32_record(const tode_solve_args &a, const tode_controller &c, hipStream_t s);
int solve_builtin_t32_y64_record(const tode_solve_args &a, const tode_controller &c, hipStream_t s);

// (each translation unit instantiates one pair of types, with or without the record: TODE_INSTANTIATE_RECORD)
#if TODE_INSTANTIATE_RECORD
#define TODE_SOLVE_ENTRY(name) name##_record
#else
#define TODE_SOLVE_ENTRY(name) name
#endif
#if TODE_INSTANTIATE_F32
int TODE_SOLVE_ENTRY(solve_builtin_f32)(const tode_solve_args &a, const tode_controller &c, hipStream_t s) { return dispatch_term<float>(a, c, s); }
#endif
#if TODE_INSTANTIATE_F64
int TODE_SOLVE_ENTRY(solve_builtin_f64)(const tode_solve_args &a, const tode_controller &c, hipStream_t s) { return dispatch_term<double>(a, c, s); }
#endif
#if TODE_INSTANTIATE_T64_Y32
int TODE_SOLVE_ENTRY(solve_builtin_t64_y32)(const tode_solve_args &a, const tode_controller &c, hipStream_t s) { return dispatch_term<float, double>(a, c, s); }
#endif
#if TODE_INSTANTIATE_T32_Y64
int TODE_SOLVE_ENTRY(solve_builtin_t32_y64)(const tode_solve_args &a, const tode_controller &c, hipStream_t s) { return dispatch_term<double, float>(a, c, s); }
#endif

}  // namespace tode
