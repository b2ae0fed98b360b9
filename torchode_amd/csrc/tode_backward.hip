// Reverse sweep over a whole recorded solve with a built-in right-hand side, in one kernel.
//
// The reference differentiates its loop through the graph of torch operations that autograd kept of it
// (adjoints.py:33-40, 111-113, 135-260).  Here the forward pass left a record of the loop state before every
// iteration (tode_solve_record).  One thread per sample walks its iterations from the last to the first: it forms
// the six stages again from the recorded state (registers, the right-hand side evaluated in the kernel), pulls the
// cotangents of the state after the iteration and of the evaluation points the iteration wrote through everything
// after the stages (finish_backward_sample), then through the stages from the last to the first, with the
// right-hand side's own vector-Jacobian product in closed form where the per-iteration path asks autograd for it.
// Everything a sample's thread works on -- stage derivatives, their cotangents, the cotangents of the state -- is an
// array private to the thread, indexed by constants once the shared reverse functions are inlined with the row length
// known (registers): those functions get index 0 and every array in global memory moved forward to the thread's sample.
// The record of the next iteration down is loaded while the current one is worked on.
#include "tode_adjoint.h"

namespace tode {

template <typename T> struct WholeBackward {
    AdjointParams<T, T> base;  // problem and controller; the per-iteration fields and the working arrays are set in the kernel
    long long iterations;      // L: the record holds entries 0..L
    const T *rec_t, *rec_dt, *rec_y, *rec_k0, *rec_prev, *rec_pprev;
    const int32_t *rec_running, *rec_n_accepted;
    const T *params;
    double scalars[4];
    T *a_y, *a_k0, *a_t, *a_dt, *a_prev, *a_pprev;  // results: cotangents of the state before the first iteration
    T *g_params;  // [B,P] result
    // the evaluation points of every sample ordered by the iteration that wrote them: [B,E] point indices and, in the
    // same order, the iterations (-1 first: points no iteration wrote)
    const int32_t *points_by_iteration, *iterations_sorted;
    long long ts_stride, te_stride;  // t_start / t_end: sample b at element b * stride
    int through_start;  // also carry the cotangents through the start of the loop (start_backward)
    int dt0_given;      // the first step was the caller's, not the start rule's
};

template <typename T, int F> struct RecordEntry {
    T t, dt, prev, pprev, y[F], k0[F];
    int32_t running, n_accepted;
};

template <typename T, int F> __device__ __forceinline__ RecordEntry<T, F> load_entry(const WholeBackward<T> &w, long long entry, long long sample) {
    const long long at = entry * w.base.batch + sample;
    RecordEntry<T, F> r;
    r.t = w.rec_t[at], r.dt = w.rec_dt[at], r.prev = w.rec_prev[at], r.pprev = w.rec_pprev[at];
#pragma unroll
    for (int f = 0; f < F; ++f) r.y[f] = w.rec_y[at * F + f], r.k0[f] = w.rec_k0[at * F + f];
    r.running = w.rec_running[at], r.n_accepted = w.rec_n_accepted[at];
    return r;
}

// cotangent shares of minimum(a, b) (or maximum with the comparison turned round) for operand a: all of it where a
// is the one taken, half on a tie (torch.minimum / torch.maximum)
template <typename T> __device__ __forceinline__ T share_of_min(T a, T b) { return a < b ? (T)1 : (a == b ? (T)0.5 : (T)0); }
template <typename T> __device__ __forceinline__ T share_of_max(T a, T b) { return a > b ? (T)1 : (a == b ? (T)0.5 : (T)0); }

// cotangent of v given that of rms(v) = |v / sqrt(F)|_2 (zero where the norm is zero, as torch.linalg.vector_norm)
template <typename T, int F> __device__ __forceinline__ void rms_backward(const T (&v)[F], T norm, T g, T (&gv)[F]) {
    const T sf = (T)__builtin_sqrt((double)F);
#pragma unroll
    for (int f = 0; f < F; ++f) gv[f] = norm != (T)0 ? (g * ((v[f] / sf) / norm)) / sf : (T)0;
}

// The start of the loop reversed: y = y0, k0 = f(t_start, y0) and, unless the caller gave the first step, the step of
// the start rule (step_size_controllers.py:431-490 / 776-835, written out in initial_step) clamped to the time range
// (adjoints.py:86-93).  In: the cotangents a_y, a_k0, a_dt of that first loop state.  Out: a_y becomes the cotangent
// of y0, gpar gains the right-hand side's parameters' share.  The times are constants here (a caller that wants their
// gradients takes the first state's cotangents and does this part itself), and the right-hand side does not depend
// on t (none of the built-in ones does).
template <typename T, int CTRL, typename Term>
__device__ __forceinline__ void start_backward(const CtrlParams<T> &cp, const Term &rhs, const bool through_rule, const T ts, const T te,
                                               const T (&y0)[Term::F], const T (&f0)[Term::F], T (&a_y)[Term::F], const T (&a_k0)[Term::F],
                                               const T a_dt, T (&gpar)[Term::P]) {
    constexpr int F = Term::F;
    T g_y0[F], g_f0[F];
#pragma unroll
    for (int f = 0; f < F; ++f) g_y0[f] = a_y[f], g_f0[f] = a_k0[f];
    if (through_rule && a_dt != (T)0) {
        // ---- forward values (initial_step) ----
        const T dir = te > ts ? (T)1 : (T)-1, span = abs_(te - ts);
        T inv[F], u[F], v[F], w[F], y1[F], f1[F];
#pragma unroll
        for (int f = 0; f < F; ++f) inv[f] = (T)1 / fma_(cp.rtol, abs_(y0[f]), cp.atol), u[f] = y0[f] * inv[f], v[f] = f0[f] * inv[f];
        const T d0 = rms<T, F>(u), d1 = rms<T, F>(v);
        const bool small = d0 < (T)1e-5 || d1 < (T)1e-5;
        const T h0a = small ? (T)1e-6 : ((T)0.01 * d0) / d1;
        const T h0 = tmin(h0a, span);
        const T dh = dir * h0;
#pragma unroll
        for (int f = 0; f < F; ++f) y1[f] = fma_(dh, f0[f], y0[f]);
        const T t1 = fma_(dir, h0, ts);
        rhs(t1, y1, f1);
#pragma unroll
        for (int f = 0; f < F; ++f) w[f] = (f1[f] - f0[f]) * inv[f];
        const T r2 = rms<T, F>(w);
        const bool blocked = CTRL == 0 && h0 == (T)0;  // (the integral controller's copy of the rule: d2 = inf)
        const T d2 = blocked ? (T)__builtin_huge_val() : r2 / h0;
        const T m = tmax(d1, d2);
        const bool tiny = m <= (T)1e-15;
        const T z = ((T)1 / m) * (T)0.01;
        const T h1 = tiny ? tmax((T)1e-6, h0 * (T)1e-3) : rpow<T>(z, 1.0 / 5.0);
        const T first = dir * tmin((T)100 * h0, h1);
        const T lo = tmin(ts, te) - ts, hi = tmax(te, ts) - ts;
        // ---- reversed ----
        // torch.clamp(first, lo, hi) (adjoints.py:107): the whole cotangent stays with the step where it lies within
        // the bounds, the bounds included (another rule than minimum / maximum, which halve it on a tie)
        const T g_first = (first >= lo && first <= hi) ? a_dt : (T)0;
        const T g_min = g_first * dir;
        T g_h0 = (T)100 * (g_min * share_of_min<T>((T)100 * h0, h1));
        const T g_h1 = g_min * share_of_min<T>(h1, (T)100 * h0);
        T g_d1 = 0, g_d2 = 0;
        if (tiny) {
            g_h0 += (h0 * (T)1e-3 >= (T)1e-6) ? g_h1 * (T)1e-3 : (T)0;
        } else {
            const T g_z = g_h1 * ((T)(1.0 / 5.0) * rpow<T>(z, 1.0 / 5.0 - 1.0));
            const T rm = (T)1 / m;
            const T g_m = -(g_z * (T)0.01) * rm * rm;
            g_d1 = g_m * share_of_max<T>(d1, d2);
            g_d2 = g_m * share_of_max<T>(d2, d1);
        }
        T g_inv[F];
#pragma unroll
        for (int f = 0; f < F; ++f) g_inv[f] = 0;
        if (!blocked && g_d2 != (T)0) {
            const T g_r2 = g_d2 / h0;
            g_h0 += -g_d2 * r2 / (h0 * h0);
            T g_w[F], g_f1[F], g_y1[F];
            rms_backward<T, F>(w, r2, g_r2, g_w);
#pragma unroll
            for (int f = 0; f < F; ++f) g_f1[f] = g_w[f] * inv[f], g_f0[f] -= g_w[f] * inv[f], g_inv[f] += g_w[f] * (f1[f] - f0[f]);
            rhs.vjp(t1, y1, g_f1, g_y1, gpar);
            T g_step = 0;
#pragma unroll
            for (int f = 0; f < F; ++f) g_y0[f] += g_y1[f], g_f0[f] += g_y1[f] * dh, g_step += g_y1[f] * f0[f];
            g_h0 += g_step * dir;
        }
        const T g_h0a = g_h0 * share_of_min<T>(h0a, span);
        if (!small) {
            const T q = (T)0.01 * d0;
            g_d1 += -g_h0a * q / (d1 * d1);
            const T g_d0 = (T)0.01 * (g_h0a / d1);
            T g_u[F];
            rms_backward<T, F>(u, d0, g_d0, g_u);
#pragma unroll
            for (int f = 0; f < F; ++f) g_y0[f] += g_u[f] * inv[f], g_inv[f] += g_u[f] * y0[f];
        }
        {
            T g_v[F];
            rms_backward<T, F>(v, d1, g_d1, g_v);
#pragma unroll
            for (int f = 0; f < F; ++f) g_f0[f] += g_v[f] * inv[f], g_inv[f] += g_v[f] * f0[f];
        }
#pragma unroll
        for (int f = 0; f < F; ++f) g_y0[f] += (-g_inv[f] * inv[f] * inv[f]) * cp.rtol * sign_(y0[f]);
    }
    T g_from_f0[F];
    rhs.vjp(ts, y0, g_f0, g_from_f0, gpar);
#pragma unroll
    for (int f = 0; f < F; ++f) a_y[f] = g_y0[f] + g_from_f0[f];
}

template <typename T, int METHOD, int CTRL, typename Term>
__global__ void __launch_bounds__(64) whole_backward_kernel(const WholeBackward<T> w) {
    using Tab = typename std::conditional<METHOD == 1, Tsit5Tab, Dopri5Tab>::type;
    constexpr int F = Term::F, P = Term::P;
    const long long B = w.base.batch;
    const long long g = (long long)blockIdx.x * 64 + threadIdx.x;  // this thread's sample
    if (g >= B) return;
    Term rhs;
    rhs.load(w.params + g * P, w.scalars);
    T gpar[P];
#pragma unroll
    for (int j = 0; j < P; ++j) gpar[j] = 0;

    // ---- the thread's own arrays; the shared functions reach them through q with index 0 ----
    T k[7][F], g_k[7][F], y[F], y1[F], g_ystage[F], g_y[F], g_y1[F], a_y[F], a_k0[F];
    T t0 = 0, dt = 0, prev = 1, pprev = 1, g_t = 0, g_dt = 0, g_prev = 0, g_pprev = 0;
    T a_t = 0, a_dt = 0, a_prev = 0, a_pprev = 0;  // cotangents of the state after the iteration: zeros behind the last one
    int32_t moved = 0, running_next = 0;
#pragma unroll
    for (int f = 0; f < F; ++f) a_y[f] = 0, a_k0[f] = 0;
    AdjointParams<T, T> q = w.base;
#pragma unroll
    for (int s = 0; s < 7; ++s) q.k[s] = k[s], q.g_k[s] = g_k[s];
    q.t = &t0, q.dt = &dt, q.y = y, q.y1 = y1, q.prev = &prev, q.pprev = &pprev;
    q.moved = &moved, q.running_next = &running_next;
    q.g_y = g_y, q.g_y1 = g_y1, q.g_t = &g_t, q.g_dt = &g_dt, q.g_prev = &g_prev, q.g_pprev = &g_pprev;
    q.a_y = a_y, q.a_k0 = a_k0, q.a_t = &a_t, q.a_dt = &a_dt, q.a_prev = &a_prev, q.a_pprev = &a_pprev;
    // ---- what lives in global memory, moved forward to this sample ----
    const int E = q.E;
    q.t_start += g * w.ts_stride, q.t_end += g * w.te_stride;
    if (q.t_eval) q.t_eval += g * E;
    q.grad_ys += g * (long long)(E > 0 ? E : 1) * F;
    if (q.g_t_start) q.g_t_start += g;
    if (q.g_t_end) q.g_t_end += g;
    if (q.g_t_eval) q.g_t_eval += g * E;
    const int32_t *iterations_sorted = w.iterations_sorted + g * E, *points_by_iteration = w.points_by_iteration + g * E;

    const long long L = w.iterations;
    int cursor = E - 1;  // into the sample's points ordered by iteration, walked from the end as the iterations are
    RecordEntry<T, F> after = load_entry<T, F>(w, L, g), here = load_entry<T, F>(w, L > 0 ? L - 1 : 0, g);
    for (long long i = L - 1; i >= 0; --i) {
        const RecordEntry<T, F> before = load_entry<T, F>(w, i > 0 ? i - 1 : 0, g);  // (used by the next pass of this loop)
        q.iteration = (int)i;
        q.end_point = (E == 0 && i == L - 1) ? 1 : 0;
        // An iteration that none of the wavefront's samples took part in (all had finished before it) changes nothing for
        // them -- no move, no point written, the step and the history kept -- so its reverse hands every cotangent on as
        // it is.  (Without evaluation points the batch's last iteration is the one whose interpolant gives the result.)
        if (!q.end_point && !__any(here.running != 0)) {
            after = here, here = before;
            continue;
        }
        t0 = here.t, dt = here.dt, prev = here.prev, pprev = here.pprev;
        moved = (after.n_accepted - here.n_accepted) > 0 ? 1 : 0;
        running_next = after.running != 0 ? 1 : 0;

        // ---- the stages again (runge_kutta.py:255-263) ----
#pragma unroll
        for (int f = 0; f < F; ++f) y[f] = here.y[f], k[0][f] = here.k0[f];
#pragma unroll
        for (int s = 1; s < 7; ++s) {
            T yi[F];
#pragma unroll
            for (int f = 0; f < F; ++f) {
                T sum = 0;
#pragma unroll
                for (int j = 0; j < s; ++j) sum = fma_((T)Tab::a[s][j], k[j][f], sum);
                yi[f] = fma_(dt, sum, y[f]);
            }
            rhs(fma_((T)Tab::c[s], dt, t0), yi, k[s]);
            if (s == 6) {
#pragma unroll
                for (int f = 0; f < F; ++f) y1[f] = yi[f];
            }
        }

        // ---- everything after the stages, reversed ----
        // (The points of this iteration are counted in a loop that the whole wavefront runs together, with a clamped
        // index in place of a guarded load: no lane leaves and rejoins here.  Written as each lane's own loop, this was a
        // divergent region at whose end the compiler, for four instantiations on long float64 rows, copied registers of
        // the parameter cotangents to accumulation registers ahead of the instruction that restores the execution mask;
        // lanes that had no point left skipped the copy and went on with the values of an earlier iteration.)
        int n_here = 0;
        while (E > 0) {
            const int at = cursor - n_here;
            const bool more = at >= 0 && iterations_sorted[at < 0 ? 0 : at] == (int)i;
            if (!__any(more)) break;
            n_here += more ? 1 : 0;
        }
        cursor -= n_here;
        finish_backward_sample<T, T, METHOD, CTRL, false, F>(q, 0, 0, 1, points_by_iteration + cursor + 1, n_here);

        // ---- the stages reversed ----
#pragma unroll
        for (int s = 6; s >= 1; --s) {
            T yi[F], gk[F], gy[F];
#pragma unroll
            for (int f = 0; f < F; ++f) {
                T sum = 0;
#pragma unroll
                for (int j = 0; j < s; ++j) sum = fma_((T)Tab::a[s][j], k[j][f], sum);
                yi[f] = fma_(dt, sum, y[f]);
                gk[f] = g_k[s][f];
            }
            rhs.vjp(fma_((T)Tab::c[s], dt, t0), yi, gk, gy, gpar);
#pragma unroll
            for (int f = 0; f < F; ++f) g_ystage[f] = gy[f] + (s == 6 ? g_y1[f] : (T)0);
            stage_backward_sample<T, T, METHOD, false, F>(q, 0, s, g_ystage, (const T *)nullptr, 0, 1);
        }

        // ---- the cotangents of the state before this iteration are those behind the one before it ----
#pragma unroll
        for (int f = 0; f < F; ++f) a_y[f] = g_y[f], a_k0[f] = g_k[0][f];
        a_t = g_t, a_dt = g_dt, a_prev = g_prev, a_pprev = g_pprev;
        after = here, here = before;
    }
    // (no iteration: nothing flows back through the loop, and the cotangents are still the zeros they started as)
    if (w.through_start)  // (`here` is the record's first entry now: t_start, y0, f(t_start, y0))
        start_backward<T, CTRL, Term>(q.cp, rhs, q.through_control && !w.dt0_given, q.t_start[0], q.t_end[0], here.y, here.k0, a_y, a_k0, a_dt, gpar);
#pragma unroll
    for (int f = 0; f < F; ++f) w.a_y[g * F + f] = a_y[f], w.a_k0[g * F + f] = a_k0[f];
    w.a_t[g] = a_t, w.a_dt[g] = a_dt, w.a_prev[g] = a_prev, w.a_pprev[g] = a_pprev;
#pragma unroll
    for (int j = 0; j < P; ++j) w.g_params[g * P + j] = gpar[j];
}

// Which iteration wrote which evaluation point (adjoints.py:215-234: the first whose new time has reached it; none for
// a point at t_start, which the loop's set-up writes, and for one the solve never reached): one thread per point, a
// binary search over the sample's recorded times.
template <typename T> __global__ void __launch_bounds__(256) backward_hits_kernel(long long B, int E, long long L, const T *t_start, long long ts_stride, const T *t_end, long long te_stride,
                                                                                  const T *t_eval, const T *rec_t, int32_t *iterations_sorted, int32_t *points_by_iteration) {
    const long long at_point = (long long)blockIdx.x * 256 + threadIdx.x;
    if (at_point >= B * E) return;
    const long long b = at_point / E;
    const int e = (int)(at_point - b * E);
    const T ts = t_start[b * ts_stride], dir = t_end[b * te_stride] > ts ? (T)1 : (T)-1;
    const T at = t_eval[at_point], v = dir * at;
    long long lo = 0, hi = L;
    while (lo < hi) {
        const long long mid = (lo + hi) / 2;
        if (dir * rec_t[(mid + 1) * B + b] < v) lo = mid + 1;
        else hi = mid;
    }
    int32_t hit = lo < L ? (int32_t)lo : -1;
    if (e == 0 && at == ts) hit = -1;
    iterations_sorted[at_point] = hit, points_by_iteration[at_point] = e;
}

// Each sample's points ordered by the iteration that wrote them (stable: points of one iteration stay in their order).
// One thread per sample.  Rows whose evaluation times run in the direction of the solve are in order already, which a
// look along the row shows; the others are sorted by insertion.
// (a template only so that each translation unit that instantiates the sweep has its own copy)
template <typename T> __global__ void __launch_bounds__(256) backward_order_kernel(long long B, int E, int32_t *iterations_sorted, int32_t *points_by_iteration) {
    const long long b = (long long)blockIdx.x * 256 + threadIdx.x;
    if (b >= B) return;
    int32_t *its = iterations_sorted + b * E, *pts = points_by_iteration + b * E;
    bool ordered = true;
    for (int e = 1; e < E; ++e) ordered = ordered && its[e - 1] <= its[e];
    if (ordered) return;
    for (int e = 1; e < E; ++e) {
        const int32_t hit = its[e], point = pts[e];
        int j = e - 1;
        for (; j >= 0 && its[j] > hit; --j) its[j + 1] = its[j], pts[j + 1] = pts[j];
        its[j + 1] = hit, pts[j + 1] = point;
    }
}

template <typename T, int METHOD, int CTRL, typename Term>
static int launch_backward(const tode_solve_args &a, const tode_controller &c, const tode_solve_adjoint &adj, hipStream_t stream) {
    const long long B = a.batch;
    constexpr int F = Term::F;
    WholeBackward<T> w = {};
    AdjointParams<T, T> &p = w.base;
    p.batch = B, p.F = F, p.E = a.n_eval, p.through_control = adj.through_control;
    p.t_start = (const T *)a.t_start, p.t_end = (const T *)a.t_end, p.t_eval = (const T *)a.t_eval, p.fixed_dt = nullptr;
    p.grad_ys = (const T *)adj.grad_ys, p.hit_iteration = nullptr, p.running = nullptr;
    p.g_t_start = (T *)adj.g_t_start, p.g_t_end = (T *)adj.g_t_end, p.g_t_eval = (T *)adj.g_t_eval, p.g_fixed_dt = nullptr;
    p.cp = make_ctrl<T>(c);
    p.dt_min = (T)c.dt_min, p.dt_max = (T)c.dt_max;
    w.a_y = (T *)adj.a_y, w.a_k0 = (T *)adj.a_k0, w.a_t = (T *)adj.a_t, w.a_dt = (T *)adj.a_dt, w.a_prev = (T *)adj.a_prev, w.a_pprev = (T *)adj.a_pprev;
    const tode_solve_record &r = *a.record;
    w.iterations = adj.iterations;
    w.rec_t = (const T *)r.t, w.rec_dt = (const T *)r.dt, w.rec_y = (const T *)r.y, w.rec_k0 = (const T *)r.k0;
    w.rec_prev = (const T *)r.prev, w.rec_pprev = (const T *)r.pprev, w.rec_running = r.running, w.rec_n_accepted = r.n_accepted;
    w.params = (const T *)a.params;
    for (int i = 0; i < 4; ++i) w.scalars[i] = a.term_scalars[i];
    w.g_params = (T *)adj.g_params;
    w.points_by_iteration = adj.points_by_iteration, w.iterations_sorted = adj.iterations_sorted;
    if (a.n_eval > 0 && !adj.points_by_iteration) {  // (not handed in: worked out here, into the caller's scratch)
        int32_t *lists = (int32_t *)adj.scratch;
        w.iterations_sorted = lists, w.points_by_iteration = lists + B * a.n_eval;
        hipLaunchKernelGGL((backward_hits_kernel<T>), dim3((unsigned)((B * a.n_eval + 255) / 256)), dim3(256), 0, stream, B, a.n_eval, (long long)adj.iterations, (const T *)a.t_start,
                           (long long)a.t_start_stride, (const T *)a.t_end, (long long)a.t_end_stride, (const T *)a.t_eval, (const T *)a.record->t, lists, lists + B * a.n_eval);
        hipLaunchKernelGGL((backward_order_kernel<T>), dim3((unsigned)((B + 255) / 256)), dim3(256), 0, stream, B, a.n_eval, lists, lists + B * a.n_eval);
    }
    w.through_start = adj.through_start, w.dt0_given = a.dt0 != nullptr;
    w.ts_stride = a.t_start_stride, w.te_stride = a.t_end_stride;
    hipLaunchKernelGGL((whole_backward_kernel<T, METHOD, CTRL, Term>), dim3((unsigned)((B + 63) / 64)), dim3(64), 0, stream, w);
    return check_hip(hipGetLastError(), "tode_solve_builtin_backward launch");
}

template <typename T, typename Term> static int backward_mc(const tode_solve_args &a, const tode_controller &c, const tode_solve_adjoint &adj, hipStream_t s) {
    if (a.method == TODE_DOPRI5 && c.kind == TODE_CTRL_INTEGRAL) return launch_backward<T, 0, 0, Term>(a, c, adj, s);
    if (a.method == TODE_DOPRI5 && c.kind == TODE_CTRL_PID) return launch_backward<T, 0, 1, Term>(a, c, adj, s);
    if (a.method == TODE_TSIT5 && c.kind == TODE_CTRL_INTEGRAL) return launch_backward<T, 1, 0, Term>(a, c, adj, s);
    if (a.method == TODE_TSIT5 && c.kind == TODE_CTRL_PID) return launch_backward<T, 1, 1, Term>(a, c, adj, s);
    return fail(TODE_E_INVALID, "unknown method %d or controller kind %d", a.method, c.kind);
}

template <typename T> static int backward_term(const tode_solve_args &a, const tode_controller &c, const tode_solve_adjoint &adj, hipStream_t s) {
    switch (a.term) {
    case TODE_TERM_VAN_DER_POL:
        if (a.n_features != 2 || a.n_params != 1) return fail(TODE_E_INVALID, "Van der Pol needs F=2, P=1");
        return backward_mc<T, VanDerPolTerm<T>>(a, c, adj, s);
    case TODE_TERM_LORENZ63:
        if (a.n_features != 3 || a.n_params != 1) return fail(TODE_E_INVALID, "Lorenz-63 needs F=3, P=1");
        return backward_mc<T, Lorenz63Term<T>>(a, c, adj, s);
    case TODE_TERM_LINEAR_DECAY:
        if (a.n_params != a.n_features) return fail(TODE_E_INVALID, "linear decay needs P == F");
        switch (a.n_features) {
        case 1: return backward_mc<T, LinearDecayTerm<T, 1>>(a, c, adj, s);
        case 2: return backward_mc<T, LinearDecayTerm<T, 2>>(a, c, adj, s);
        case 3: return backward_mc<T, LinearDecayTerm<T, 3>>(a, c, adj, s);
        case 4: return backward_mc<T, LinearDecayTerm<T, 4>>(a, c, adj, s);
        case 8: return backward_mc<T, LinearDecayTerm<T, 8>>(a, c, adj, s);
        default: return fail(TODE_E_UNSUPPORTED, "linear decay is built for F in {1,2,3,4,8}, got %d", a.n_features);
        }
    default:
        return fail(TODE_E_UNSUPPORTED, "the whole reverse sweep is built for the three small systems (term %d)", a.term);
    }
}

int solve_backward_f32(const tode_solve_args &a, const tode_controller &c, const tode_solve_adjoint &adj, hipStream_t s);
int solve_backward_f64(const tode_solve_args &a, const tode_controller &c, const tode_solve_adjoint &adj, hipStream_t s);
#if TODE_INSTANTIATE_F32
int solve_backward_f32(const tode_solve_args &a, const tode_controller &c, const tode_solve_adjoint &adj, hipStream_t s) { return backward_term<float>(a, c, adj, s); }
#endif
#if TODE_INSTANTIATE_F64
int solve_backward_f64(const tode_solve_args &a, const tode_controller &c, const tode_solve_adjoint &adj, hipStream_t s) { return backward_term<double>(a, c, adj, s); }
#endif

}  // namespace tode

#if TODE_INSTANTIATE_F32
extern "C" {

int64_t tode_solve_backward_scratch_bytes(const tode_solve_args *a) {
    if (!a || a->n_features <= 0 || a->batch < 0 || a->n_eval < 0) return -1;
    return 2 * a->batch * a->n_eval * (int64_t)sizeof(int32_t);  // (the two lists of evaluation points, where the caller does not hand them in)
}

int tode_solve_builtin_backward(const tode_solve_args *a, const tode_controller *c, const tode_solve_adjoint *adj, void *stream) {
    using namespace tode;
    if (!a || !c || !adj) return fail(TODE_E_INVALID, "null argument struct");
    if (a->batch < 0 || a->n_features <= 0 || a->n_eval < 0 || a->n_params < 0) return fail(TODE_E_INVALID, "bad sizes");
    if (!known_dtype(a->dtype)) return fail(TODE_E_INVALID, "unknown dtype %d", a->dtype);
    if (a->dtype & TODE_DTYPE_PAIR) return fail(TODE_E_UNSUPPORTED, "the whole reverse sweep is built for time and data in one dtype");
    if (c->kind != TODE_CTRL_INTEGRAL && c->kind != TODE_CTRL_PID) return fail(TODE_E_INVALID, "unknown controller kind %d", c->kind);
    if (!a->record) return fail(TODE_E_INVALID, "args->record is null: the sweep starts from the record of the forward pass");
    if (adj->iterations < 0 || a->record->capacity < adj->iterations + 1)
        return fail(TODE_E_INVALID, "the record holds %lld entries, %lld iterations need %lld", (long long)a->record->capacity, (long long)adj->iterations, (long long)adj->iterations + 1);
    if (a->t_start_stride < 1 || a->t_end_stride < 1) return fail(TODE_E_INVALID, "t_start_stride / t_end_stride must be >= 1");
    if ((a->t_start_stride != 1 && adj->g_t_start) || (a->t_end_stride != 1 && adj->g_t_end)) return fail(TODE_E_INVALID, "g_t_start / g_t_end are dense arrays: ask for them with dense t_start / t_end");
    if (a->batch == 0) return TODE_OK;
    const tode_solve_record &r = *a->record;
    if (!r.t || !r.dt || !r.y || !r.k0 || !r.prev || !r.pprev || !r.running || !r.n_accepted) return fail(TODE_E_INVALID, "a null array in the record");
    if (!a->t_start || !a->t_end || (a->n_eval > 0 && (!a->t_eval || !adj->points_by_iteration != !adj->iterations_sorted)) || (a->n_params > 0 && !a->params) || !adj->grad_ys || !adj->a_y ||
        !adj->a_k0 || !adj->a_t || !adj->a_dt || !adj->a_prev || !adj->a_pprev || !adj->g_params)
        return fail(TODE_E_INVALID, "null pointer");
    const bool own_lists = a->n_eval > 0 && !adj->points_by_iteration;
    if (own_lists && (a->batch * (int64_t)a->n_eval + 255) / 256 > 2147483647) return fail(TODE_E_UNSUPPORTED, "too many evaluation points for the library to order them: hand the two lists in");
    if (own_lists && (!adj->scratch || adj->scratch_bytes < tode_solve_backward_scratch_bytes(a)))
        return fail(TODE_E_INVALID, "the scratch buffer holds %lld bytes, this sweep needs %lld (tode_solve_backward_scratch_bytes)", (long long)(adj->scratch ? adj->scratch_bytes : 0),
                    (long long)tode_solve_backward_scratch_bytes(a));
    hipStream_t s = (hipStream_t)stream;
    return a->dtype == TODE_F32 ? solve_backward_f32(*a, *c, *adj, s) : solve_backward_f64(*a, *c, *adj, s);
}

}  // extern "C"
#endif
