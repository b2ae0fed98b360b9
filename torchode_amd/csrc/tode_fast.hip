// Fast whole-solve kernel for the common case: evaluation points given and
// monotone in each sample's direction of time, no dt_min / dt_max, and every
// sample succeeds.  One wavefront per workgroup, one sample per lane.
//
// What makes it fast on CDNA4, where B = 65536 samples is exactly one wavefront
// per SIMD and therefore every instruction of any kind costs an issue slot:
//   * the loop body is straight-line code executed by the whole wavefront until
//     its slowest lane has finished (finished lanes keep their state through
//     selects), so control flow is wave-uniform scalar branches;
//   * each sample's evaluation times are staged in LDS (transposed, so that a
//     lane's reads hit its own bank) instead of being fetched from HBM inside
//     the loop, and -- when it fits -- the dense output is collected in LDS and
//     written back at the end as one contiguous, fully coalesced block per wave;
//   * the controller's powers share one double-word logarithm per step.
// The arithmetic is the same sequence of IEEE operations as in the general
// kernel (tode_persistent.hip), so the two produce identical bits.
//
// Anything outside the common case (a non-success status, max_steps reached, a
// non-monotone row, a sample that ends past t_end) raises TODE_FLAG_NEEDS_GENERAL
// and the caller repeats the solve through tode_solve_builtin.
#include "tode_solve.h"

namespace tode {

template <typename T> struct FastOut {
    int64_t *n_steps, *n_accepted, *n_initialized, *status;
};

// NHIST: how many history factors the controller multiplies in (0 integral, 1 PI, 2 PID).
// RECORD: the loop state before every iteration of the wavefront goes to p.rec_* (tode_solve_record), as the general
// kernel writes it: entry i is the state before iteration i; a sample that has finished repeats its last state with
// `running` 0, up to the record's capacity.  A record that is too short raises TODE_FLAG_NEEDS_GENERAL.
template <typename T, int METHOD, int CTRL, int NHIST, typename Term, bool STAGE_YS, bool RECORD = false>
__global__ void __launch_bounds__(64) solve_fast_kernel(const SolveParams<T> p, const FastOut<T> o) {
    using Tab = typename std::conditional<METHOD == 1, Tsit5Tab, Dopri5Tab>::type;
    constexpr int F = Term::F;
    constexpr int P = Term::P;
    extern __shared__ __align__(16) unsigned char smem_raw[];
    const int lane = threadIdx.x;
    const long long b0 = (long long)blockIdx.x * 64;
    const long long b = b0 + lane;
    const int rows = (int)min((long long)64, p.batch - b0);
    const bool live = lane < rows;
    const long long bs = live ? b : b0;  // safe index for loads of dead lanes
    const CtrlParams<T> &cp = p.cp;
    const int E = p.n_eval;
    const int EF = E * F;

    T *te_s = reinterpret_cast<T *>(smem_raw);  // [E][64]
    T *ys_s = te_s + (size_t)E * 64;            // [E*F][65] when STAGE_YS

    // ---- stage this wave's block of t_eval (rows * E contiguous values) into LDS ----
    {
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
    __syncthreads();

    Term rhs;
    rhs.load(p.params + bs * P, p.scalars);
    T y[F], k[7][F];
#pragma unroll
    for (int f = 0; f < F; ++f) y[f] = p.y0[bs * F + f];
    const T ts = p.t_start[bs * p.ts_stride], te = p.t_end[bs * p.te_stride];
    const bool fwd = te > ts;
    const T dir = fwd ? (T)1 : (T)-1;
    const T tlo = tmin(ts, te), thi = tmax(te, ts);

    bool bail = false;
    {
        T prev_te = te_s[lane];
        for (int e = 1; e < E; ++e) {
            T cur = te_s[e * 64 + lane];
            if (!(fwd ? cur >= prev_te : cur <= prev_te)) bail = true;
            prev_te = cur;
        }
    }

    T t = ts, dt;
    if (p.dt0) {
        dt = p.dt0[bs];
        rhs(ts, y, k[0]);
    } else {
        dt = initial_step<T, CTRL, Term>(cp, rhs, ts, y, dir, abs_(te - ts), k[0]);
    }
    dt = tclamp(dt, tlo - t, thi - t);
    // logarithms of the previous two accepted error ratios (both start at 1, log 1 = 0)
    StepFactor<T, NHIST> step_factor;  // with the logarithms of the previous two accepted error ratios (both start at 1)
    int cursor = 0;
    T *ys_g = p.ys + bs * (long long)EF;
    if (te_s[lane] == ts) {
#pragma unroll
        for (int f = 0; f < F; ++f) {
            if (STAGE_YS)
                ys_s[f * 65 + lane] = y[f];
            else if (live)
                ys_g[f] = y[f];
        }
        cursor = 1;
    }
    // direction-normalised times: multiplying by +-1 is exact, so dir*a >= dir*b decides
    // "a has reached b in the direction of time" without a branch
    T dte_next = dir * te_s[(cursor < E ? cursor : E - 1) * 64 + lane];
    const T dte_end = dir * te;

    int n_steps = 0, n_acc = 0;
    // The loop below uses the hardware's minimum and maximum, which is the reference's arithmetic as long as no
    // operand is NaN: a sample that starts with a NaN or infinite time, step or state goes to the general kernel,
    // and so does one that produces a non-finite error ratio, step factor or step later.
    {
        bool odd_start = !finite_(dt) || !finite_(ts) || !finite_(te);
#pragma unroll
        for (int f = 0; f < F; ++f) odd_start = odd_start || !finite_(y[f]) || !finite_(k[0][f]);
        bail = bail || (live && odd_start);
    }
    bool active = live && !bail;
    const T e1 = (T)cp.e1, e2 = (T)cp.e2, e3 = (T)cp.e3;
    const int step_limit = p.max_steps < TODE_HARD_STEP_LIMIT ? p.max_steps : TODE_HARD_STEP_LIMIT;

    // (RECORD) iterations of this wavefront so far = the record's next entry; the last two accepted error ratios as
    // values (the step factor keeps their logarithms)
    long long iteration = 0;
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

    // A sample that has landed past t_end (t + (t_end - t) rounded upwards) keeps stepping in the reference's later
    // iterations with the clamped step t_end - t: with evaluation points that is seen only in the status of that step,
    // which is a success unless its error ratio is not finite.  The sample sits through one more iteration here, as
    // an inactive lane whose error ratio is looked at.
    bool idle = false;
    while (__any(active || idle)) {
        if (RECORD) keep(iteration++, active);
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
        weighted_k<T, F, Tab, -1, true>(dt, k, err);

        // ---- step size control (step_size_controllers.py:370-429, 715-774) ----
        bool unordered;
        const T ratio = error_ratio_common<T, F>(cp, y, y1, err, unordered);
        const bool accept = ratio < (T)1;
        // a NaN or infinite ratio is a non-success status: leave it to the general kernel (the ratio is at least 1e-38)
        bool sane = !unordered && ratio < (T)__builtin_huge_val();
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

        // ---- dense output (adjoints.py:215-234) ----
        bool hit = active && cursor < E && dt_new >= dte_next;
        if (__any(hit)) {
            T q[5][F];
            quartic<T, F, METHOD>(dt, y, y1, k, q);
            do {
                T out[F];
                quartic_eval<T, F>(q, t0, dt, dir * dte_next, out);
                if (hit) {
#pragma unroll
                    for (int f = 0; f < F; ++f) {
                        if (STAGE_YS)
                            ys_s[(cursor * F + f) * 65 + lane] = out[f];
                        else
                            ys_g[cursor * F + f] = out[f];
                    }
                }
                cursor += hit ? 1 : 0;
                const T nxt = dir * te_s[(cursor < E ? cursor : E - 1) * 64 + lane];
                dte_next = hit ? nxt : dte_next;
                hit = hit && cursor < E && dt_new >= dte_next;
            } while (__any(hit));
        }

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
            // non-finite error ratio or max_steps reached: not the common case
            const bool failed = active && (!sane || n_steps >= step_limit);
            const bool finished = active && !failed && !running_new;
            if (__any(finished)) {
                // a sample whose state or derivative at the end is not finite shows up in later iterations of the
                // reference loop with another status; one that landed past t_end is looked at in the next iteration
                bool odd = false;
#pragma unroll
                for (int f = 0; f < F; ++f) odd = odd || !settles_(y[f], k[0][f]);
                bail = bail || (finished && odd);
                idle = finished && !odd && !(t == te);
            }
            bail = bail || failed;
            active = active && !failed && running_new;
        }
    }

    if (live) {
        o.n_steps[b] = n_steps;
        o.n_accepted[b] = n_acc;
        o.n_initialized[b] = cursor;
        o.status[b] = 0;
    }
    if (RECORD) {  // the state every sample is left in, for every later iteration of the batch
        for (long long at = iteration; at < p.rec_capacity; ++at) keep(at, false);
        if (iteration >= p.rec_capacity) record_full = true;
        bail = bail || record_full;
    }

    // ---- dense output: one contiguous block of rows * E * F values per wave ----
    if (STAGE_YS) {
        __syncthreads();
        T *dst = p.ys + b0 * EF;
        const int n = rows * EF;
        int row = lane / EF, rem = lane - row * EF;
        const int drow = 64 / EF, drem = 64 - drow * EF;
        for (int g = lane; g < n; g += 64) {
            dst[g] = ys_s[rem * 65 + row];
            rem += drem;
            row += drow;
            if (rem >= EF) {
                rem -= EF;
                row += 1;
            }
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
    publish_flags(p);
}

// LDS bytes per workgroup: evaluation times [E][64], plus the staged output [E*F][65].
static size_t lds_bytes(int E, int F, size_t item, bool stage_ys) {
    return ((size_t)E * 64 + (stage_ys ? (size_t)E * F * 65 : 0)) * item;
}

template <typename T, int METHOD, int CTRL, typename Term>
static int launch_fast(const tode_solve_args &a, const tode_controller &c, const FastOut<T> &o, hipStream_t stream) {
    SolveParams<T> p = make_params<T>(a, c);
    const long long blocks = (a.batch + 63) / 64;
    reset_flags(a.flags, stream);
    if (blocks == 0) return check_hip(hipGetLastError(), "tode_solve_builtin_fast launch");
    // Occupancy target: enough workgroups per CU to give every SIMD its share of the batch, up
    // to 4 per SIMD; LDS (160 KiB per CU) is spent on staging only while that target holds.
    const long long simd_slots = 256 * 4;
    long long per_simd = (blocks + simd_slots - 1) / simd_slots;
    if (per_simd > 4) per_simd = 4;
    const size_t budget = (size_t)(160 * 1024) / (size_t)(4 * per_simd) - 512;
    const size_t need_te = lds_bytes(a.n_eval, Term::F, sizeof(T), false);
    const size_t need_all = lds_bytes(a.n_eval, Term::F, sizeof(T), true);
    if (need_te > 64 * 1024) return fail(TODE_E_UNSUPPORTED, "n_eval=%d is too large for the fast kernel", a.n_eval);
    const CtrlParams<T> &cp = p.cp;
    if (cp.shortcut_exponent()) return fail(TODE_E_UNSUPPORTED, "a controller exponent that is not computed through pow: use the general kernel");
    const int nhist = CTRL == 0 ? 0 : (cp.skip3 ? 1 : 2);
    constexpr bool RECORD = TODE_INSTANTIATE_RECORD != 0;
    if (RECORD != (a.record != nullptr)) return fail(TODE_E_INVALID, "internal: record variant mismatch");
    if (a.record) {
        const tode_solve_record &r = *a.record;
        if (r.capacity < 1 || !r.t || !r.dt || !r.y || !r.k0 || !r.prev || !r.pprev || !r.running || !r.n_accepted)
            return fail(TODE_E_INVALID, "tode_solve_record: capacity %lld, or a null array", (long long)r.capacity);
    }
    const bool stage = !RECORD && need_all <= budget;  // (the recording variant is built without the staged output)
    const size_t lds = stage ? need_all : need_te;
    const dim3 grid((unsigned)blocks), block(64);
    timing_before(stream, "tode::solve_fast_kernel");
#define TODE_FAST_LAUNCH(NH, ST) hipLaunchKernelGGL((solve_fast_kernel<T, METHOD, CTRL, NH, Term, (ST) && !RECORD, RECORD>), grid, block, lds, stream, p, o)
    if (nhist == 0) {
        if (stage) TODE_FAST_LAUNCH(0, true); else TODE_FAST_LAUNCH(0, false);
    } else if (nhist == 1) {
        if (stage) TODE_FAST_LAUNCH(CTRL == 0 ? 0 : 1, true); else TODE_FAST_LAUNCH(CTRL == 0 ? 0 : 1, false);
    } else {
        if (stage) TODE_FAST_LAUNCH(CTRL == 0 ? 0 : 2, true); else TODE_FAST_LAUNCH(CTRL == 0 ? 0 : 2, false);
    }
#undef TODE_FAST_LAUNCH
    timing_after(stream);
    return check_hip(hipGetLastError(), "tode_solve_builtin_fast launch");
}

template <typename T, typename Term>
static int fast_mc(const tode_solve_args &a, const tode_controller &c, const FastOut<T> &o, hipStream_t s) {
    if (a.method == TODE_DOPRI5 && c.kind == TODE_CTRL_INTEGRAL) return launch_fast<T, 0, 0, Term>(a, c, o, s);
    if (a.method == TODE_DOPRI5 && c.kind == TODE_CTRL_PID) return launch_fast<T, 0, 1, Term>(a, c, o, s);
    if (a.method == TODE_TSIT5 && c.kind == TODE_CTRL_INTEGRAL) return launch_fast<T, 1, 0, Term>(a, c, o, s);
    if (a.method == TODE_TSIT5 && c.kind == TODE_CTRL_PID) return launch_fast<T, 1, 1, Term>(a, c, o, s);
    return fail(TODE_E_INVALID, "unknown method %d or controller kind %d", a.method, c.kind);
}

template <typename T>
static int fast_term(const tode_solve_args &a, const tode_controller &c, int64_t *ns, int64_t *na, int64_t *ni, int64_t *st, hipStream_t s) {
    FastOut<T> o{ns, na, ni, st};
    switch (a.term) {
    case TODE_TERM_VAN_DER_POL:
        if (a.n_features != 2 || a.n_params != 1) return fail(TODE_E_INVALID, "Van der Pol needs F=2, P=1");
        return fast_mc<T, VanDerPolTerm<T>>(a, c, o, s);
    case TODE_TERM_LORENZ63:
        if (a.n_features != 3 || a.n_params != 1) return fail(TODE_E_INVALID, "Lorenz-63 needs F=3, P=1");
        return fast_mc<T, Lorenz63Term<T>>(a, c, o, s);
    case TODE_TERM_LINEAR_DECAY:
        if (a.n_params != a.n_features) return fail(TODE_E_INVALID, "linear decay needs P == F");
        switch (a.n_features) {
        case 1: return fast_mc<T, LinearDecayTerm<T, 1>>(a, c, o, s);
        case 2: return fast_mc<T, LinearDecayTerm<T, 2>>(a, c, o, s);
        case 3: return fast_mc<T, LinearDecayTerm<T, 3>>(a, c, o, s);
        case 4: return fast_mc<T, LinearDecayTerm<T, 4>>(a, c, o, s);
        case 8: return fast_mc<T, LinearDecayTerm<T, 8>>(a, c, o, s);
        default: return fail(TODE_E_UNSUPPORTED, "linear decay is built for F in {1,2,3,4,8}, got %d", a.n_features);
        }
    default:
        return fail(TODE_E_INVALID, "unknown built-in term %d", a.term);
    }
}

// (each translation unit instantiates one type, with or without the record: TODE_INSTANTIATE_RECORD)
#if TODE_INSTANTIATE_RECORD
#define TODE_FAST_ENTRY(name) name##_record
#else
#define TODE_FAST_ENTRY(name) name
#endif
#if TODE_INSTANTIATE_F32
int TODE_FAST_ENTRY(solve_fast_f32)(const tode_solve_args &a, const tode_controller &c, int64_t *ns, int64_t *na, int64_t *ni, int64_t *st, hipStream_t s) {
    return fast_term<float>(a, c, ns, na, ni, st, s);
}
#endif
#if TODE_INSTANTIATE_F64
int TODE_FAST_ENTRY(solve_fast_f64)(const tode_solve_args &a, const tode_controller &c, int64_t *ns, int64_t *na, int64_t *ni, int64_t *st, hipStream_t s) {
    return fast_term<double>(a, c, ns, na, ni, st, s);
}
#endif

}  // namespace tode
