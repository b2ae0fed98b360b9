// Two-wavefront variant of the fast whole-solve kernel, for batches that would
// otherwise leave the SIMDs with a single wavefront each (B <= 2 * 65536 on an
// MI355X: 256 CUs x 4 SIMDs x 64 lanes).
//
// A single in-order wavefront cannot keep a SIMD busy: every instruction costs an
// issue slot and every dependent result is waited for (measured: one dependent fp32
// FMA every 7.7 cycles with one wave per SIMD, one every 5.3 per SIMD with two).  The solve
// loop has exactly one piece of work that the next step does not depend on -- the
// dense output -- so each group of 64 samples gets two wavefronts:
//   * the STEPPER runs the adaptive loop (stages, error ratio, step size control,
//     state update) and, after every attempted step, leaves the step's
//     (t0, dt, y0, y1, k_0..k_6, new time, active flag) in LDS;
//   * the EVALUATOR picks that record up one barrier later, builds the quartic
//     interpolant and writes the evaluation points the step passed, while the
//     stepper is already computing the next step.
// Records are double-buffered; one s_barrier per loop iteration orders the
// hand-over.  Stepper and evaluator roles alternate between neighbouring
// workgroups so that every SIMD hosts one of each.
//
// Same arithmetic, bit for bit, and same contract as tode_fast.hip
// (TODE_FLAG_NEEDS_GENERAL when the batch leaves the common case).
//
// RECORD: the stepper also writes the loop state before every iteration to p.rec_* (tode_solve_record), as
// tode_fast.hip's recording variant does, for the reverse sweep of a differentiable solve.
#include "tode_solve.h"

namespace tode {

template <typename T> struct PairOut {
    int64_t *n_steps, *n_accepted, *n_initialized, *status;
};

template <typename T, int METHOD, int CTRL, int NHIST, typename Term, bool STAGE_TE, bool RECORD = false>
__global__ void __launch_bounds__(128) solve_pair_kernel(const SolveParams<T> p, const PairOut<T> o) {
    using Tab = typename std::conditional<METHOD == 1, Tsit5Tab, Dopri5Tab>::type;
    constexpr int F = Term::F;
    constexpr int P = Term::P;
    constexpr int NF = 4 + 9 * F;  // record: t0, dt, dir*t_new, active, y[F], y1[F], k[7][F]
    extern __shared__ __align__(16) unsigned char smem_raw[];
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const bool stepper = ((wave + (blockIdx.x >> 1)) & 1) == 0;
    const long long b0 = (long long)blockIdx.x * 64;
    const long long b = b0 + lane;
    const int rows = (int)min((long long)64, p.batch - b0);
    const bool live = lane < rows;
    const long long bs = live ? b : b0;
    const CtrlParams<T> &cp = p.cp;
    // Without evaluation points the reference reports the end point alone (adjoints.py:296-311): the
    // interpolant of the batch's last iteration at t_end.  Here: t_end as the one evaluation point of
    // every sample, and the final state next to it in y_idle; which of the two a sample gets depends on
    // whether its last step was the batch's last iteration, known only when all samples are done
    // (tode_select_end_point).
    const bool end_only = p.n_eval == 0;
    const int E = end_only ? 1 : p.n_eval;

    T *rec = reinterpret_cast<T *>(smem_raw);                // [2][NF][64]
    int *ctl = reinterpret_cast<int *>(rec + 2 * NF * 64);   // [2] "stepper is done" per phase
    T *te_s = reinterpret_cast<T *>(ctl + 4);                // [E][64] when STAGE_TE

    const T ts = p.t_start[bs * p.ts_stride], te = p.t_end[bs * p.te_stride];
    const bool fwd = te > ts;
    const T dir = fwd ? (T)1 : (T)-1;

    if (stepper) {
        // =============================== stepper ===============================
        Term rhs;
        rhs.load(p.params + bs * P, p.scalars);
        T y[F], k[7][F];
#pragma unroll
        for (int f = 0; f < F; ++f) y[f] = p.y0[bs * F + f];
        const T tlo = tmin(ts, te), thi = tmax(te, ts);
        T t = ts, dt;
        if (p.dt0) {
            dt = p.dt0[bs];
            rhs(ts, y, k[0]);
        } else {
            dt = initial_step<T, CTRL, Term>(cp, rhs, ts, y, dir, abs_(te - ts), k[0]);
        }
        dt = tclamp(dt, tlo - t, thi - t);
        StepFactor<T, NHIST> step_factor;  // with the logarithms of the previous two accepted error ratios (both start at 1)
        const T dte_end = dir * te;
        int n_steps = 0, n_acc = 0;
        // The loop below uses the hardware's minimum and maximum, which is the reference's arithmetic as long as no
        // operand is NaN: a sample that starts with a NaN or infinite time, step or state goes to the general kernel,
        // and so does one that produces a non-finite error ratio, step factor or step later.
        bool odd_start = !finite_(dt) || !finite_(ts) || !finite_(te);
#pragma unroll
        for (int f = 0; f < F; ++f) odd_start = odd_start || !finite_(y[f]) || !finite_(k[0][f]);
        bool bail = live && odd_start;
        bool active = live && !odd_start;
        const int step_limit = p.max_steps < TODE_HARD_STEP_LIMIT ? p.max_steps : TODE_HARD_STEP_LIMIT;
        const T e1 = (T)cp.e1, e2 = (T)cp.e2, e3 = (T)cp.e3;

        // (RECORD) the last two accepted error ratios as values (the step factor keeps their logarithms)
        T ratio_prev = 1, ratio_prev_prev = 1;
        bool record_full = false;
        auto keep = [&](long long at, bool running) {
            if (at >= p.rec_capacity) {
                record_full = true;
                return;
            }
            if (!live) return;
            record_entry<T, T, F>(p, at, b, t, dt, y, k[0], ratio_prev, ratio_prev_prev, running, n_acc);
        };

        // A sample that has landed past t_end (t + (t_end - t) rounded upwards) keeps stepping in the reference's
        // later iterations with the clamped step t_end - t: with evaluation points that is seen only in the status of
        // that step, a success unless its error ratio is not finite.  The sample sits through one more iteration here,
        // as an inactive lane whose error ratio is looked at.
        bool idle = false;
        int phase = 0;
        for (;; ++phase) {
            const bool any = __any(active || idle);
            if (any) {
                if (RECORD) keep(phase, active);
                // ---- stages (runge_kutta.py:255-263) ----
                const T t0 = t;
                T y1[F], err[F];
#pragma unroll
                for (int i = 1; i < 7; ++i) {
                    T tn = fma_((T)Tab::c[i], dt, t0);
                    T yi[F];
#pragma unroll
                    for (int f = 0; f < F; ++f) {
                        T s = 0;
#pragma unroll
                        for (int j = 0; j < i; ++j) s = fma_((T)Tab::a[i][j], k[j][f], s);
                        yi[f] = fma_(dt, s, y[f]);
                    }
                    rhs(tn, yi, k[i]);
                    if (i == 6) {
#pragma unroll
                        for (int f = 0; f < F; ++f) y1[f] = yi[f];
                    }
                }
                // hand the attempted step to the evaluator (everything it needs is known now)
                const bool pre_active = active;
                T *r = rec + (phase & 1) * NF * 64 + lane;
                r[0 * 64] = t0;
                r[1 * 64] = dt;
#pragma unroll
                for (int f = 0; f < F; ++f) {
                    r[(4 + f) * 64] = y[f];
                    if (METHOD != 1) r[(4 + F + f) * 64] = y1[f];  // (Tsit5's interpolant does not look at the step's result)
                }
#pragma unroll
                for (int s = 0; s < 7; ++s)
#pragma unroll
                    for (int f = 0; f < F; ++f) r[(4 + 2 * F + s * F + f) * 64] = k[s][f];

                weighted_k<T, F, Tab, -1, true>(dt, k, err);

                // ---- step size control (step_size_controllers.py:370-429, 715-774) ----
                bool unordered;
                const T ratio = error_ratio_common<T, F>(cp, y, y1, err, unordered);
                const bool accept = ratio < (T)1;
                bool sane = !unordered && ratio < (T)__builtin_huge_val();  // (the ratio is at least 1e-38)
                bail = bail || (idle && !sane);
                idle = false;
                T factor = step_factor(cp.safety, sane ? ratio : (T)1, e1, e2, e3, active);
                sane = sane && factor == factor;  // (a product of an underflowed and an overflowed power)
                factor = clamp_ordered(factor, cp.fmin, cp.fmax);
                const T dt_next = dt * factor;

                const bool move = accept && active;
                const T t_new = move ? (t0 + dt) : t0;
                const T dt_new = dir * t_new;
                const bool running_new = dt_new < dte_end;
                n_steps += active ? 1 : 0;
                n_acc += move ? 1 : 0;
                r[2 * 64] = dt_new;
                r[3 * 64] = pre_active ? (T)1 : (T)0;

                // ---- state update (adjoints.py:150-155, 247-255) ----
#pragma unroll
                for (int f = 0; f < F; ++f) {
                    y[f] = move ? y1[f] : y[f];
                    k[0][f] = move ? k[6][f] : k[0][f];
                }
                t = t_new;
                {
                    const T dtn = running_new ? dt_next : dt;
                    const T dtc = clamp_ordered(dtn, tlo - t, thi - t);
                    dt = active ? dtc : dt;
                }
                if (NHIST >= 1) step_factor.shift(active && running_new && accept);
                if (RECORD && CTRL == 1) {
                    const bool shift = active && running_new && accept;
                    ratio_prev_prev = shift ? ratio_prev : ratio_prev_prev;
                    ratio_prev = shift ? ratio : ratio_prev;
                }
                {
                    const bool failed = active && (!sane || n_steps >= step_limit);
                    const bool finished = active && !failed && !running_new;
                    if (__any(finished)) {
                        // a sample whose state or derivative at the end is not finite shows up in later iterations of
                        // the reference loop with another status, and so does, without evaluation points, one that
                        // landed past t_end (in the interpolant of the batch's last step); with evaluation points
                        // such a sample is looked at in the next iteration
                        bool odd = end_only && !(t == te);
#pragma unroll
                        for (int f = 0; f < F; ++f) odd = odd || !settles_(y[f], k[0][f]);
                        bail = bail || (finished && odd);
                        idle = finished && !odd && !(t == te);
                    }
                    bail = bail || failed;
                    active = active && !failed && running_new;
                }
            }
            if (lane == 0) ctl[phase & 1] = any ? 0 : 1;
            __syncthreads();
            if (!any) break;
        }

        if (RECORD) {  // the state every sample is left in, for every later iteration of the batch
            for (long long at = phase; at < p.rec_capacity; ++at) keep(at, false);
            if (phase >= p.rec_capacity) record_full = true;
            bail = bail || record_full;
        }
        if (live) {
            o.n_steps[b] = n_steps;
            o.n_accepted[b] = n_acc;
            o.status[b] = 0;
            if (end_only) {
#pragma unroll
                for (int f = 0; f < F; ++f) p.y_idle[b * F + f] = y[f];
            }
        }
        int my_steps = live ? n_steps : 0, my_bail = (live && bail) ? 1 : 0;
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) {
            my_steps = max(my_steps, __shfl_xor(my_steps, off));
            my_bail = max(my_bail, __shfl_xor(my_bail, off));
        }
        if (lane == 0) {
            if (my_steps > 0) atomicMax(&p.flags[TODE_FLAG_MAX_ITERATIONS], my_steps);
            if (my_bail) atomicMax(&p.flags[TODE_FLAG_NEEDS_GENERAL], 1);
        }
    } else {
        // ============================== evaluator ==============================
        const T *tev_g = p.t_eval + bs * (long long)E;
        if (STAGE_TE && !end_only) {
            // this group's block of t_eval (rows * E contiguous values), transposed into LDS
            const T *src = p.t_eval + b0 * E;
            const int n = rows * E;
            int row = lane / E, e = lane - row * E;
            const int drow = 64 / E, de = 64 - drow * E;
            for (int g = lane; g < n; g += 64) {
                te_s[e * 64 + row] = src[g];
                e += de;
                row += drow;
                if (e >= E) {
                    e -= E;
                    row += 1;
                }
            }
        }
        // (LDS accesses of one wavefront complete in order; te_s is private to this wave)
        auto te_at = [&](int e) -> T { return end_only ? te : (STAGE_TE ? te_s[e * 64 + lane] : tev_g[e]); };
        bool bail = false;
        {
            T prev_te = te_at(0);
            for (int e = 1; e < E; ++e) {
                T cur = te_at(e);
                if (!(fwd ? cur >= prev_te : cur <= prev_te)) bail = true;
                prev_te = cur;
            }
        }
        T *ys_g = p.ys + bs * (long long)E * F;
        int cursor = 0;
        if (te_at(0) == ts) {
            if (live) {
#pragma unroll
                for (int f = 0; f < F; ++f) ys_g[f] = p.y0[bs * F + f];
            }
            cursor = 1;
        }
        T dte_next = dir * te_at(cursor < E ? cursor : E - 1);

        for (int phase = 0;; ++phase) {
            if (phase > 0) {
                const T *r = rec + ((phase - 1) & 1) * NF * 64 + lane;
                const T dt_new = r[2 * 64];
                const bool was_active = live && !bail && r[3 * 64] != (T)0;
                bool hit = was_active && cursor < E && dt_new >= dte_next;
                if (__any(hit)) {
                    const T t0 = r[0 * 64], dt = r[1 * 64];
                    T y[F], y1[F], k[7][F], q[5][F];
#pragma unroll
                    for (int f = 0; f < F; ++f) {
                        y[f] = r[(4 + f) * 64];
                        y1[f] = METHOD != 1 ? r[(4 + F + f) * 64] : (T)0;
                    }
#pragma unroll
                    for (int s = 0; s < 7; ++s)
#pragma unroll
                        for (int f = 0; f < F; ++f) k[s][f] = r[(4 + 2 * F + s * F + f) * 64];
                    quartic<T, F, METHOD>(dt, y, y1, k, q);
                    do {
                        T out[F];
                        quartic_eval<T, F>(q, t0, dt, dir * dte_next, out);
                        if (hit) {
#pragma unroll
                            for (int f = 0; f < F; ++f) ys_g[cursor * F + f] = out[f];
                        }
                        cursor += hit ? 1 : 0;
                        const T nxt = dir * te_at(cursor < E ? cursor : E - 1);
                        dte_next = hit ? nxt : dte_next;
                        hit = hit && cursor < E && dt_new >= dte_next;
                    } while (__any(hit));
                }
            }
            __syncthreads();
            if (ctl[phase & 1]) break;
        }

        if (live) o.n_initialized[b] = cursor;
        int my_bail = (live && bail) ? 1 : 0;
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) my_bail = max(my_bail, __shfl_xor(my_bail, off));
        if (lane == 0 && my_bail) atomicMax(&p.flags[TODE_FLAG_NEEDS_GENERAL], 1);
    }
    publish_flags(p);
}

template <typename T, int METHOD, int CTRL, typename Term>
static int launch_pair(const tode_solve_args &a, const tode_controller &c, const PairOut<T> &o, hipStream_t stream, bool *used) {
    *used = false;
    constexpr int NF = 4 + 9 * Term::F;
    const long long blocks = (a.batch + 63) / 64;
    // worthwhile only while the single-wave kernel would leave SIMDs with <= 2 wavefronts
    if (blocks == 0 || blocks > 2 * 1024) return TODE_OK;
    const size_t rec_bytes = (size_t)2 * NF * 64 * sizeof(T) + 16;
    const size_t te_bytes = (size_t)a.n_eval * 64 * sizeof(T);
    const size_t budget = (size_t)(160 * 1024) / 4 - 512;  // four workgroups (eight wavefronts) per CU
    if (rec_bytes > budget) return TODE_OK;
    const bool stage_te = rec_bytes + te_bytes <= budget;
    const size_t lds = rec_bytes + (stage_te ? te_bytes : 0);
    constexpr bool RECORD = TODE_INSTANTIATE_RECORD != 0;
    if (RECORD != (a.record != nullptr)) return fail(TODE_E_INVALID, "internal: record variant mismatch");
    SolveParams<T> p = make_params<T>(a, c);
    if (p.cp.shortcut_exponent()) return TODE_OK;  // left to the caller's other kernels
    const int nhist = CTRL == 0 ? 0 : (p.cp.skip3 ? 1 : 2);
    const dim3 grid((unsigned)blocks), block(128);
    reset_flags(a.flags, stream);
    timing_before(stream, "tode::solve_pair_kernel");
#define TODE_PAIR_LAUNCH(NH, ST) hipLaunchKernelGGL((solve_pair_kernel<T, METHOD, CTRL, NH, Term, ST, RECORD>), grid, block, lds, stream, p, o)
    if (nhist == 0) {
        if (stage_te) TODE_PAIR_LAUNCH(0, true); else TODE_PAIR_LAUNCH(0, false);
    } else if (nhist == 1) {
        if (stage_te) TODE_PAIR_LAUNCH(CTRL == 0 ? 0 : 1, true); else TODE_PAIR_LAUNCH(CTRL == 0 ? 0 : 1, false);
    } else {
        if (stage_te) TODE_PAIR_LAUNCH(CTRL == 0 ? 0 : 2, true); else TODE_PAIR_LAUNCH(CTRL == 0 ? 0 : 2, false);
    }
#undef TODE_PAIR_LAUNCH
    timing_after(stream);
    *used = true;
    return check_hip(hipGetLastError(), "tode_solve_builtin_fast (pair kernel) launch");
}

template <typename T, typename Term>
static int pair_mc(const tode_solve_args &a, const tode_controller &c, const PairOut<T> &o, hipStream_t s, bool *used) {
    if (a.method == TODE_DOPRI5 && c.kind == TODE_CTRL_INTEGRAL) return launch_pair<T, 0, 0, Term>(a, c, o, s, used);
    if (a.method == TODE_DOPRI5 && c.kind == TODE_CTRL_PID) return launch_pair<T, 0, 1, Term>(a, c, o, s, used);
    if (a.method == TODE_TSIT5 && c.kind == TODE_CTRL_INTEGRAL) return launch_pair<T, 1, 0, Term>(a, c, o, s, used);
    if (a.method == TODE_TSIT5 && c.kind == TODE_CTRL_PID) return launch_pair<T, 1, 1, Term>(a, c, o, s, used);
    *used = false;
    return TODE_OK;
}

// Tries the two-wavefront kernel; *used tells whether it was launched (otherwise the caller
// falls through to the single-wavefront kernel).
template <typename T>
static int pair_term(const tode_solve_args &a, const tode_controller &c, int64_t *ns, int64_t *na, int64_t *ni, int64_t *st, hipStream_t s,
                     bool *used) {
    PairOut<T> o{ns, na, ni, st};
    *used = false;
    switch (a.term) {
    case TODE_TERM_VAN_DER_POL:
        if (a.n_features != 2 || a.n_params != 1) return TODE_OK;
        return pair_mc<T, VanDerPolTerm<T>>(a, c, o, s, used);
    case TODE_TERM_LORENZ63:
        if (a.n_features != 3 || a.n_params != 1) return TODE_OK;
        return pair_mc<T, Lorenz63Term<T>>(a, c, o, s, used);
    case TODE_TERM_LINEAR_DECAY:
        if (a.n_params != a.n_features) return TODE_OK;
        switch (a.n_features) {
        case 1: return pair_mc<T, LinearDecayTerm<T, 1>>(a, c, o, s, used);
        case 2: return pair_mc<T, LinearDecayTerm<T, 2>>(a, c, o, s, used);
        case 3: return pair_mc<T, LinearDecayTerm<T, 3>>(a, c, o, s, used);
        case 4: return pair_mc<T, LinearDecayTerm<T, 4>>(a, c, o, s, used);
        default: return TODE_OK;
        }
    default:
        return TODE_OK;
    }
}

// (each translation unit instantiates one type, with or without the record: TODE_INSTANTIATE_RECORD)
#if TODE_INSTANTIATE_RECORD
#define TODE_PAIR_ENTRY(name) name##_record
#else
#define TODE_PAIR_ENTRY(name) name
#endif
#if TODE_INSTANTIATE_F32
int TODE_PAIR_ENTRY(solve_pair_f32)(const tode_solve_args &a, const tode_controller &c, int64_t *ns, int64_t *na, int64_t *ni, int64_t *st, hipStream_t s, bool *used) {
    return pair_term<float>(a, c, ns, na, ni, st, s, used);
}
#endif
#if TODE_INSTANTIATE_F64
int TODE_PAIR_ENTRY(solve_pair_f64)(const tode_solve_args &a, const tode_controller &c, int64_t *ns, int64_t *na, int64_t *ni, int64_t *st, hipStream_t s, bool *used) {
    return pair_term<double>(a, c, ns, na, ni, st, s, used);
}
#endif

}  // namespace tode
