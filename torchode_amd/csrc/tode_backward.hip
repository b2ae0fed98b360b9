// Reverse sweep over a whole recorded solve with a built-in right-hand side, in one kernel.
//
// The reference differentiates its loop through the graph of torch operations that autograd kept of it
// (adjoints.py:33-40, 111-113, 135-260).  Here the forward pass left a record of the loop state before every
// iteration (tode_solve_record).  One thread per sample walks its iterations from the last to the first: it forms
// the six stages again from the recorded state (registers, the right-hand side evaluated in the kernel), pulls the
// cotangents of the state after the iteration and of the evaluation points the iteration wrote through everything
// after the stages (finish_backward_sample), then through the stages from the last to the first, with the
// right-hand side's own vector-Jacobian product in closed form where the per-iteration path asks autograd for it.
// The per-sample arrays that the shared reverse functions read and write (stage derivatives, their cotangents,
// the cotangents of the state) are rows in LDS that only the sample's own thread touches: the functions index them
// by the sample's number within its workgroup, and every array in global memory is handed to them moved forward by the
// workgroup's first sample, so that the same index fits.
#include "tode_adjoint.h"

namespace tode {

template <typename T> struct WholeBackward {
    AdjointParams<T, T> base;  // problem and controller; the per-iteration fields and the LDS rows are set in the kernel
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
};

// Elements of T per sample in LDS: k_1..k_6, g_k_0..g_k_6, y1, g_ystage, g_y, g_y1, the cotangents of the state after
// the iteration (a_y, a_k0) [F each]; g_t, g_dt, g_prev, g_pprev, a_t, a_dt, a_prev, a_pprev, moved, running_next [1 each].
__host__ __device__ constexpr int backward_row_elements(int F) { return (6 + 7 + 1 + 1 + 2 + 2) * F + 10; }

template <typename T, int METHOD, int CTRL, typename Term>
__global__ void __launch_bounds__(256) whole_backward_kernel(const WholeBackward<T> w) {
    using Tab = typename std::conditional<METHOD == 1, Tsit5Tab, Dopri5Tab>::type;
    constexpr int F = Term::F, P = Term::P;
    extern __shared__ __align__(16) unsigned char lds_raw[];
    const long long B = w.base.batch;
    const int n = blockDim.x;                        // samples of this workgroup
    const long long b0 = (long long)blockIdx.x * n;  // its first sample
    const int b = threadIdx.x;                       // the sample's number within the workgroup: the index the shared functions use
    if (b0 + b >= B) return;
    Term rhs;
    rhs.load(w.params + (b0 + b) * P, w.scalars);
    T gpar[P];
#pragma unroll
    for (int j = 0; j < P; ++j) gpar[j] = 0;

    // ---- the rows in LDS, [n, F] or [n] each ----
    T *lds = reinterpret_cast<T *>(lds_raw);
    auto rows = [&](int per_sample) {
        T *at = lds;
        lds += per_sample * n;
        return at;
    };
    AdjointParams<T, T> q = w.base;  // (a_* start as null pointers: zeros behind the last iteration)
    T *k_rows[7];
    for (int s = 1; s < 7; ++s) k_rows[s] = rows(F), q.k[s] = k_rows[s];
    for (int s = 0; s < 7; ++s) q.g_k[s] = rows(F);
    T *y1_row = rows(F), *g_ystage = rows(F);
    q.y1 = y1_row, q.g_y = rows(F), q.g_y1 = rows(F);
    T *a_y = rows(F), *a_k0 = rows(F);
    q.g_t = rows(1), q.g_dt = rows(1), q.g_prev = rows(1), q.g_pprev = rows(1);
    T *a_t = rows(1), *a_dt = rows(1), *a_prev = rows(1), *a_pprev = rows(1);
    int32_t *moved = reinterpret_cast<int32_t *>(rows(1)), *running_next = reinterpret_cast<int32_t *>(rows(1));
    q.moved = moved, q.running_next = running_next;
    // ---- what lives in global memory, moved forward to the workgroup's first sample ----
    const int E = q.E;
    q.t_start += b0, q.t_end += b0;
    if (q.t_eval) q.t_eval += b0 * E;
    q.grad_ys += b0 * (long long)(E > 0 ? E : 1) * F;
    if (q.g_t_start) q.g_t_start += b0;
    if (q.g_t_end) q.g_t_end += b0;
    if (q.g_t_eval) q.g_t_eval += b0 * E;
    const int32_t *iterations_sorted = w.iterations_sorted + b0 * E, *points_by_iteration = w.points_by_iteration + b0 * E;

    int cursor = E - 1;  // into the sample's points ordered by iteration, walked from the end as the iterations are
    for (long long i = w.iterations - 1; i >= 0; --i) {
        const long long at = i * B + b0, next = (i + 1) * B + b0;
        q.iteration = (int)i;
        q.end_point = (E == 0 && i == w.iterations - 1) ? 1 : 0;
        q.t = w.rec_t + at, q.dt = w.rec_dt + at, q.y = w.rec_y + at * F;
        q.prev = w.rec_prev + at, q.pprev = w.rec_pprev + at;
        q.k[0] = w.rec_k0 + at * F;
        moved[b] = (w.rec_n_accepted[next + b] - w.rec_n_accepted[at + b]) > 0 ? 1 : 0;
        running_next[b] = w.rec_running[next + b] != 0 ? 1 : 0;

        // ---- the stages again (runge_kutta.py:255-263) ----
        const T t0 = q.t[b], dt = q.dt[b];
        T y[F], k[7][F];
#pragma unroll
        for (int f = 0; f < F; ++f) y[f] = q.y[b * F + f], k[0][f] = q.k[0][b * F + f];
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
#pragma unroll
            for (int f = 0; f < F; ++f) k_rows[s][b * F + f] = k[s][f];
            if (s == 6) {
#pragma unroll
                for (int f = 0; f < F; ++f) y1_row[b * F + f] = yi[f];
            }
        }

        // ---- everything after the stages, reversed ----
        int n_here = 0;
        while (cursor - n_here >= 0 && iterations_sorted[b * E + cursor - n_here] == (int)i) ++n_here;
        cursor -= n_here;
        finish_backward_sample<T, T, METHOD, CTRL, false>(q, b, 0, 1, points_by_iteration + b * E + cursor + 1, n_here);

        // ---- the stages reversed ----
#pragma unroll
        for (int s = 6; s >= 1; --s) {
            T yi[F], g[F], gy[F];
#pragma unroll
            for (int f = 0; f < F; ++f) {
                T sum = 0;
#pragma unroll
                for (int j = 0; j < s; ++j) sum = fma_((T)Tab::a[s][j], k[j][f], sum);
                yi[f] = fma_(dt, sum, y[f]);
                g[f] = q.g_k[s][b * F + f];
            }
            rhs.vjp(fma_((T)Tab::c[s], dt, t0), yi, g, gy, gpar);
#pragma unroll
            for (int f = 0; f < F; ++f) g_ystage[b * F + f] = gy[f] + (s == 6 ? q.g_y1[b * F + f] : (T)0);
            stage_backward_sample<T, T, METHOD, false>(q, b, s, g_ystage, (const T *)nullptr, 0, 1);
        }

        // ---- the cotangents of the state before this iteration are those behind the one before it ----
#pragma unroll
        for (int f = 0; f < F; ++f) a_y[b * F + f] = q.g_y[b * F + f], a_k0[b * F + f] = q.g_k[0][b * F + f];
        a_t[b] = q.g_t[b], a_dt[b] = q.g_dt[b], a_prev[b] = q.g_prev[b], a_pprev[b] = q.g_pprev[b];
        q.a_y = a_y, q.a_k0 = a_k0, q.a_t = a_t, q.a_dt = a_dt, q.a_prev = a_prev, q.a_pprev = a_pprev;
    }
    const bool any = w.iterations > 0;  // (no iteration: nothing flows back through the loop)
    const long long g = b0 + b;
#pragma unroll
    for (int f = 0; f < F; ++f) w.a_y[g * F + f] = any ? a_y[b * F + f] : (T)0, w.a_k0[g * F + f] = any ? a_k0[b * F + f] : (T)0;
    w.a_t[g] = any ? a_t[b] : (T)0, w.a_dt[g] = any ? a_dt[b] : (T)0, w.a_prev[g] = any ? a_prev[b] : (T)0, w.a_pprev[g] = any ? a_pprev[b] : (T)0;
#pragma unroll
    for (int j = 0; j < P; ++j) w.g_params[g * P + j] = gpar[j];
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
    // (the t_start / t_end strides of the forward entry point are not taken here: the caller passes dense arrays)
    // samples per workgroup: whole wavefronts, as many as 48 KiB of LDS rows hold, at most 256
    const size_t row_bytes = (size_t)backward_row_elements(F) * sizeof(T);
    int threads = (int)((48 * 1024) / row_bytes) / 64 * 64;
    threads = threads > 256 ? 256 : (threads < 64 ? 64 : threads);
    if ((size_t)threads * row_bytes > 64 * 1024)
        return fail(TODE_E_UNSUPPORTED, "rows of %d values of %d bytes: one wavefront of samples does not fit the sweep's working rows into 64 KiB of LDS", F, (int)sizeof(T));
    hipLaunchKernelGGL((whole_backward_kernel<T, METHOD, CTRL, Term>), dim3((unsigned)((B + threads - 1) / threads)), dim3(threads), threads * row_bytes, stream, w);
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
    if (!a || a->n_features <= 0 || a->batch < 0) return -1;
    return 0;  // (the sweep's working rows live in LDS)
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
    if (a->t_start_stride != 1 || a->t_end_stride != 1) return fail(TODE_E_INVALID, "t_start and t_end must be dense arrays here");
    if (a->batch == 0) return TODE_OK;
    const tode_solve_record &r = *a->record;
    if (!r.t || !r.dt || !r.y || !r.k0 || !r.prev || !r.pprev || !r.running || !r.n_accepted) return fail(TODE_E_INVALID, "a null array in the record");
    if (!a->t_start || !a->t_end || (a->n_eval > 0 && (!a->t_eval || !adj->points_by_iteration || !adj->iterations_sorted)) || (a->n_params > 0 && !a->params) || !adj->grad_ys || !adj->a_y ||
        !adj->a_k0 || !adj->a_t || !adj->a_dt || !adj->a_prev || !adj->a_pprev || !adj->g_params)
        return fail(TODE_E_INVALID, "null pointer");
    if (adj->scratch_bytes < tode_solve_backward_scratch_bytes(a) || (tode_solve_backward_scratch_bytes(a) > 0 && !adj->scratch))
        return fail(TODE_E_INVALID, "the scratch buffer holds %lld bytes, this sweep needs %lld (tode_solve_backward_scratch_bytes)", (long long)adj->scratch_bytes,
                    (long long)tode_solve_backward_scratch_bytes(a));
    hipStream_t s = (hipStream_t)stream;
    return a->dtype == TODE_F32 ? solve_backward_f32(*a, *c, *adj, s) : solve_backward_f64(*a, *c, *adj, s);
}

}  // extern "C"
#endif
